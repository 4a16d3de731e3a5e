"""Token dispatch / combine for the single-device (all-gather) communication method.
Mirrors ``TokenDispatcherWithAllGather`` (``vllm_ascend/ops/fused_moe/token_dispatcher.py:358-461``):
``token_dispatch`` = expert histogram + stable permutation + gather with the first dynamic
int8 quantisation fused in; ``token_combine`` = weighted un-permute."""
from __future__ import annotations

import torch

from ..device_op import DeviceOperator
from ..quant_type import QuantType
from .contracts import MoEAllGatherCombineMetadata, MoETokenDispatchInput, MoETokenDispatchOutput


class TokenDispatcherWithAllGather:
    def __init__(self, **kwargs):
        self.top_k = kwargs.get("top_k", 0)
        self.num_experts = kwargs.get("num_experts", 0)
        self.max_num_tokens = kwargs.get("max_num_tokens")
        local = kwargs.get("num_local_experts", 0)
        self.num_experts_local = local.item() if torch.is_tensor(local) else int(local)
        self.lora_context = None

    def set_lora_context(self, lora_context) -> None:
        if lora_context is not None:
            raise NotImplementedError("MoE LoRA is outside this build")

    def token_dispatch(self, token_dispatch_input: MoETokenDispatchInput) -> MoETokenDispatchOutput:
        tdi = token_dispatch_input
        quant_type = tdi.quant.quant_type
        if quant_type not in (QuantType.NONE, QuantType.W8A8, QuantType.W4A8):
            raise NotImplementedError(f"token_dispatch: quant type {quant_type} has no MI355X kernels")
        routing = tdi.routing
        if routing.expert_map is not None or routing.global_redundant_expert_num:
            raise NotImplementedError("expert_map / redundant experts (expert parallelism) need more than one GPU")
        if routing.mc2_mask is not None:
            raise NotImplementedError("mc2_mask belongs to the MC2 communication method (expert parallelism)")

        hidden_states = tdi.hidden_states
        topk_weights = tdi.topk_weights
        dynamic_scale = routing.pertoken_scale
        with_quant = tdi.quant.dispatch_with_quant
        # the first quantisation of the MLP is folded into the gather unless the caller
        # already quantised the activations (then hidden_states is int8 and only moves)
        # (pertoken_scale given: quant_mode -1 and the scale travels with the rows, token_dispatcher.py:399-435)
        quant_mode = 1 if (with_quant and dynamic_scale is None) else -1
        if dynamic_scale is not None and hidden_states.dtype != torch.int8:
            raise ValueError("pertoken_scale goes with int8 hidden states (activations quantised by the caller), "
                             f"got {hidden_states.dtype}")
        restore_shape = hidden_states.shape
        num_tokens = hidden_states.shape[:-1].numel()
        if routing.apply_router_weight_on_input:
            assert topk_weights.dim() == 2, "`topk_weights` should be in shape (num_tokens, topk)"
            assert topk_weights.shape[1] == 1, "Only support topk=1 when `apply_router_weight_on_input` is True"
            hidden_states = hidden_states * topk_weights.to(hidden_states.dtype)

        sorted_hidden_states, expanded_row_idx, expert_tokens, dynamic_scale = DeviceOperator.npu_moe_init_routing(
            hidden_states, tdi.topk_ids, scale=dynamic_scale, active_num=num_tokens * self.top_k,
            expert_num=self.num_experts_local, expert_tokens_num_type=1, expert_tokens_num_flag=True,
            active_expert_range=[0, self.num_experts_local], quant_mode=quant_mode)
        return MoETokenDispatchOutput(
            hidden_states=sorted_hidden_states,
            dynamic_scale=dynamic_scale if with_quant else None,
            group_list=expert_tokens.to(torch.int64),
            group_list_type=1,  # per-expert counts
            combine_metadata=MoEAllGatherCombineMetadata(topk_weights=topk_weights,
                                                         expanded_row_idx=expanded_row_idx,
                                                         restore_shape=restore_shape),
        )

    def token_combine(self, hidden_states, combine_metadata: MoEAllGatherCombineMetadata, bias=None, residual=None):
        """``residual`` (not in the reference): a [T, H] tensor added in fp32 before the bf16 rounding --
        the shared-expert output, which upstream vLLM would add afterwards."""
        assert bias is None, "bias is not supported by the combine"
        out = DeviceOperator.npu_moe_token_unpermute(permuted_tokens=hidden_states,
                                                     sorted_indices=combine_metadata.expanded_row_idx,
                                                     probs=combine_metadata.topk_weights, residual=residual)
        if len(combine_metadata.restore_shape) == 3:
            out = out.view(combine_metadata.restore_shape)
        return out
