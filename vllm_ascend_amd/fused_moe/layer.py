"""Owner of one MoE layer's expert weights and the runner that strings the stages
together: router -> ``quant_method.apply`` -> result.  Counterpart of
``AscendRoutedExperts.forward_impl`` (``vllm_ascend/ops/fused_moe/routed_experts.py:496-609``)
and of the weight registration in ``AscendFusedMoEMethod.create_weights``
(``vllm_ascend/quantization/method_adapters.py:214-245``), without vLLM."""
from __future__ import annotations

import torch

from ..quantization.base import AscendMoEScheme
from ..quantization.checkpoint import moe_weight_loader
from .contracts import FusedExpertsResult, FusedMoEConfig
from .moe_comm_method import setup_moe_comm_method
from .router import AscendFusedTopKRouter


class AscendRoutedExperts(torch.nn.Module):
    def __init__(self, moe_config: FusedMoEConfig, quant_method: AscendMoEScheme, router: AscendFusedTopKRouter,
                 params_dtype: torch.dtype = torch.bfloat16, device="cuda", shared_experts=None, gate=None,
                 dynamic_eplb: bool = False, expert_heat_collection_interval: int | None = None):
        super().__init__()
        self.shared_experts = shared_experts
        # the router's own gate (an AscendGateLinear) when the layer computes its logits itself
        # (is_internal_router, vllm_ascend/ops/fused_moe/fused_moe.py:264-271)
        self.gate = gate
        self.moe_config = moe_config
        self.quant_method = quant_method
        self.router = router
        self.activation = moe_config.activation
        self.apply_router_weight_on_input = False
        self.ascend_expert_map = None
        self.global_redundant_expert_num = 0
        self.ascend_mc2_mask = None
        self.ascend_pertoken_scale = None
        self.enable_force_load_balance = False  # profile runs only (routed_experts.py:484-492)
        # logical -> physical expert ids when the layer holds redundant copies of experts (dynamic load balancing,
        # routed_experts.py:250, 452-453): the router scores the logical experts, the weights are the physical ones
        self.log2phy = None
        # small batches (decode): gating and dispatch in one launch when the scheme has the fused form
        self.use_fused_small_batch = True
        # ... and, for at most 1024 (token, slot) pairs, without sorting them: every intermediate row belongs to a
        # pair, the GEMMs' workgroups collect the pairs of their expert themselves (W8A8 scheme)
        self.use_pair_order = True
        specs = dict(quant_method.get_weight(moe_config.num_experts, moe_config.intermediate_size_per_partition,
                                             moe_config.hidden_dim, params_dtype))
        specs.update(quant_method.get_dynamic_quant_param(moe_config.num_experts,
                                                          moe_config.intermediate_size_per_partition,
                                                          moe_config.hidden_dim, params_dtype))
        for name, t in specs.items():
            self.register_parameter(name, torch.nn.Parameter(t.to(device), requires_grad=False))
        self.moe_comm_method = setup_moe_comm_method(moe_config)
        # tokens per local expert, summed over forward passes, for the load balancer
        # (routed_experts.py:343-373): one int64 row, or, with a collection interval, one int32 row per
        # pass of the interval, indexed by a device-side pass counter
        self.dynamic_eplb = dynamic_eplb
        self.eplb_heat_collection_status = True
        self.multi_stage = bool(dynamic_eplb and expert_heat_collection_interval)
        self.num_iter = int(expert_heat_collection_interval) if self.multi_stage else None
        if not self.multi_stage:
            self.load_counter = None
        if not dynamic_eplb:
            self.moe_load = None
        else:
            if self.multi_stage:
                self.register_buffer("load_counter", torch.zeros((), dtype=torch.int32, device=device),
                                     persistent=False)
                self.register_buffer("moe_load", torch.zeros((self.num_iter, moe_config.num_experts),
                                                             dtype=torch.int32, device=device), persistent=False)
            else:
                self.register_buffer("moe_load", torch.zeros(moe_config.num_experts, dtype=torch.int64,
                                                             device=device), persistent=False)
        # per-expert checkpoint tensors -> slices of the stacked parameters (quantization/checkpoint.py)
        self.weight_loader = moe_weight_loader

    def load_weights(self, tensors: dict[str, torch.Tensor]) -> None:
        """Copy checkpoint-layout tensors into the registered parameters, then run the scheme's
        post-load processing (format cast, scale reshapes)."""
        for name, t in tensors.items():
            p = getattr(self, name)
            p.data.copy_(t.reshape(p.data.shape).to(p.data.dtype))
        self.quant_method.process_weights_after_loading(self)

    def get_log2phy_map(self) -> torch.Tensor | None:
        return self.log2phy

    def clear_moe_load(self) -> None:
        """Zero the collected expert loads (routed_experts.py:423-428)."""
        assert self.moe_load is not None
        self.moe_load.zero_()
        if self.multi_stage:
            self.load_counter.zero_()

    def _record_expert_load(self, result: FusedExpertsResult) -> None:
        """Add this pass's tokens per expert to ``moe_load`` (routed_experts.py:567-587)."""
        expert_tokens, group_list_type = result.expert_tokens, result.group_list_type
        assert expert_tokens is not None and group_list_type is not None, (
            "expert_tokens and group_list_type should not be None when dynamic_eplb is enabled.")
        if group_list_type == 1:
            local_load = expert_tokens
        else:  # running totals -> counts
            local_load = torch.cat([expert_tokens[:1], expert_tokens[1:] - expert_tokens[:-1]])
        if self.multi_stage:
            cur_iter = torch.remainder(self.load_counter, self.num_iter)
            self.moe_load.index_add_(0, cur_iter.view(1), local_load.to(torch.int32).view(1, -1))
            self.load_counter.add_(1)
        else:
            self.moe_load.add_(local_load)

    def forward_impl(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> FusedExpertsResult:
        result = self._run_experts(hidden_states, router_logits)
        if self.dynamic_eplb and self.eplb_heat_collection_status:
            self._record_expert_load(result)
        result.routed_out = self.moe_comm_method.finalize(result.routed_out, reduce_results=False)
        return result

    def _run_experts(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> FusedExpertsResult:
        hidden_states, router_logits, _, _ = self.moe_comm_method.prepare(hidden_states, router_logits)
        fused = getattr(self.quant_method, "supports_small_batch", None)
        if self.use_fused_small_batch and fused is not None and fused(self, hidden_states, router_logits, self.router):
            return self.quant_method.apply_small_batch(self, hidden_states, router_logits, self.router,
                                                       self.shared_experts, None)
        # int8 hidden states = activations the caller quantised (their scales in ascend_pertoken_scale): the
        # routing weights then take the model dtype of the scheme
        weights_dtype = None
        if hidden_states.dtype == torch.int8:
            weights_dtype = getattr(self.quant_method, "in_dtype", torch.bfloat16)
        topk_weights, topk_ids = self.router.select_experts(
            hidden_states, router_logits, enable_force_load_balance=self.enable_force_load_balance,
            weights_dtype=weights_dtype)
        # The reference maps the router's ids through log2phy first and then, in a profile run, replaces them by
        # random ids in [0, num_logical_experts) that are not mapped again (routed_experts.py:452-492).  The
        # router here draws those random ids itself, so with forced load balance the map is skipped.
        if self.log2phy is not None and not self.enable_force_load_balance:
            topk_ids = self.log2phy[topk_ids.long()].to(topk_ids.dtype)
        return self.quant_method.apply(self, hidden_states, topk_weights, topk_ids, self.shared_experts, None)

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor | None = None) -> torch.Tensor:
        if router_logits is None:
            if self.gate is None:
                raise ValueError("router_logits is required: this layer was built without an internal gate")
            router_logits, _ = self.gate(hidden_states)
        return self.forward_impl(hidden_states, router_logits).routed_out
