"""Top-k router on the fused gating kernel (``AscendFusedTopKRouter._compute_routing``,
``vllm_ascend/ops/fused_moe/router/fused_topk_router.py:84-159``): softmax or sigmoid
scoring, optional correction bias, group-limited selection with the sum-of-top-2 group
score (the reference always passes ``group_select_mode=1``), eps = 1e-20."""
from __future__ import annotations

import torch

from ..device_op import DeviceOperator


class AscendFusedTopKRouter:
    def __init__(self, top_k: int, global_num_experts: int, *, renormalize: bool = True, use_grouped_topk: bool = False,
                 num_expert_group: int | None = None, topk_group: int | None = None, scoring_func: str = "softmax",
                 routed_scaling_factor: float = 1.0, e_score_correction_bias: torch.Tensor | None = None):
        if scoring_func not in ("softmax", "sigmoid"):
            raise NotImplementedError(f"scoring_func {scoring_func!r} (hash routing) is outside this build")
        self.top_k = top_k
        self.global_num_experts = global_num_experts
        self.renormalize = renormalize
        self.num_expert_group = num_expert_group if use_grouped_topk or num_expert_group else None
        self.topk_group = topk_group if use_grouped_topk or topk_group else None
        self.scoring_func = scoring_func
        self.routed_scaling_factor = routed_scaling_factor
        self.e_score_correction_bias = e_score_correction_bias

    def select_experts(self, hidden_states: torch.Tensor, router_logits: torch.Tensor,
                       indices_type: torch.dtype | None = None, enable_force_load_balance: bool = False,
                       weights_dtype: torch.dtype | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """-> (topk_weights in the hidden-state dtype, topk_ids int32)
        (``vllm_ascend/ops/fused_moe/routed_experts.py:438-494``).  ``enable_force_load_balance`` (profile runs
        only, ``routed_experts.py:484-492``): the ids are replaced by the first k entries of a random
        permutation of the experts per token, so that no expert collects the whole dummy batch; the weights
        stay.  ``weights_dtype``: dtype of the returned weights when the hidden states are int8 (pre-quantised)."""
        if weights_dtype is None:
            weights_dtype = hidden_states.dtype
        topk_weights, topk_ids = self._compute_routing(hidden_states, router_logits, indices_type,
                                                       weights_dtype=weights_dtype)
        if enable_force_load_balance:
            random_matrix = torch.rand(topk_ids.size(0), self.global_num_experts, device=topk_ids.device)
            topk_ids = torch.argsort(random_matrix, dim=1)[:, : topk_ids.size(1)].to(topk_ids.dtype)
        return topk_weights.to(weights_dtype), topk_ids

    def is_fused_supported(self, hidden_states: torch.Tensor) -> bool:
        """The reference's guard in front of the fused gating op, taken over as it stands (it measures the last
        dimension of the hidden states, ``fused_topk_router.py:66-82``)."""
        topk_group = self.topk_group if self.topk_group is not None else 1
        num_expert_group = self.num_expert_group if self.num_expert_group is not None else 1
        last = hidden_states.shape[-1]
        if not (num_expert_group > 0 and last % num_expert_group == 0 and last // num_expert_group > 2):
            return False
        if self.top_k > (last / (num_expert_group * topk_group)):
            return False
        return not topk_group * last / num_expert_group < self.top_k

    def _compute_routing(self, hidden_states, router_logits, indices_type=None, weights_dtype=None):
        if not self.is_fused_supported(hidden_states):
            # the reference falls back to its torch-native grouped top-k here, whose group score (max instead of the
            # sum of the top two) and tie order differ from the fused op's (grouped_topk_router.py:51-67)
            raise NotImplementedError("router: shapes the fused gating op refuses take the torch-native router in "
                                      "the reference, which this build does not have")
        bias = self.e_score_correction_bias
        if bias is not None and bias.dtype != router_logits.dtype:
            bias = self.e_score_correction_bias = bias.to(router_logits.dtype)
        topk_weights, topk_ids, _ = DeviceOperator.moe_gating_top_k(
            router_logits,
            k=self.top_k,
            k_group=self.topk_group if self.topk_group is not None else 1,
            group_count=self.num_expert_group if self.num_expert_group is not None else 1,
            group_select_mode=1,
            renorm=int(self.renormalize),
            norm_type=0 if self.scoring_func == "softmax" else 1,
            out_flag=False,
            routed_scaling_factor=self.routed_scaling_factor,
            eps=1e-20,
            bias_opt=bias,
            weights_dtype=weights_dtype,
        )
        if indices_type is not None and topk_ids.dtype != indices_type:
            topk_ids = topk_ids.to(indices_type)
        return topk_weights, topk_ids
