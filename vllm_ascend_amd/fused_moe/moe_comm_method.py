"""dispatch -> MLP -> combine orchestration (``MoECommMethod.fused_experts``,
``vllm_ascend/ops/fused_moe/moe_comm_method.py:117-162``) for the all-gather method,
the only one that exists on a single device (``:55-62``)."""
from __future__ import annotations

import torch

from .contracts import (FusedExpertsResult, FusedMoEConfig, MoEFusedExpertsInput, build_mlp_compute_input,
                        build_token_dispatch_input)
from .forward_context import _EXTRA_CTX, MoECommType
from .moe_mlp import unified_apply_mlp
from .token_dispatcher import TokenDispatcherWithAllGather

_MoECommMethods: dict = {}


def get_moe_comm_method(moe_comm_type: MoECommType | None):
    return _MoECommMethods.get(moe_comm_type)


def setup_moe_comm_method(moe_config: FusedMoEConfig):
    if moe_config.ep_size > 1:
        raise NotImplementedError("expert parallelism (all-to-all / MC2 methods) needs more than one GPU")
    _MoECommMethods[MoECommType.ALLGATHER] = AllGatherCommImpl(moe_config)
    _EXTRA_CTX.moe_comm_type = MoECommType.ALLGATHER
    _EXTRA_CTX.moe_comm_method = _MoECommMethods[MoECommType.ALLGATHER]
    return _EXTRA_CTX.moe_comm_method


class _IdentityPrepareFinalize:
    """dp_size == pcp_size == tp_size == 1: nothing to pad, gather or reduce
    (``prepare_finalize.py:439-476,534-541``)."""

    def prepare(self, hidden_states, router_logits, replace_allreduce=False, quant_type=None):
        return hidden_states, router_logits, None, None

    def finalize(self, hidden_states, reduce_results, padded_hidden_states_shape=None):
        return hidden_states


class AllGatherCommImpl:
    def __init__(self, moe_config: FusedMoEConfig):
        self.moe_config = moe_config
        self.token_dispatcher = TokenDispatcherWithAllGather(
            top_k=moe_config.experts_per_token, num_experts=moe_config.num_experts,
            num_local_experts=moe_config.num_local_experts)
        self.prepare_finalize = _IdentityPrepareFinalize()

    def prepare(self, hidden_states, router_logits, replace_allreduce=False, quant_type=None):
        return self.prepare_finalize.prepare(hidden_states, router_logits, replace_allreduce, quant_type)

    def finalize(self, hidden_states, reduce_results, padded_hidden_states_shape=None):
        return self.prepare_finalize.finalize(hidden_states, reduce_results, padded_hidden_states_shape)

    def fused_experts(self, fused_experts_input: MoEFusedExpertsInput) -> FusedExpertsResult:
        f = fused_experts_input
        assert f.hidden_states.dtype in (torch.bfloat16, torch.float16, torch.int8), (
            f"Unsupported hidden_states dtype: {f.hidden_states.dtype}")
        assert _EXTRA_CTX.moe_comm_method is not None, "Missing communication context"
        stream = torch.cuda.current_stream() if f.hidden_states.is_cuda else None
        before_dispatch_evt = stream.record_event() if stream else None
        dispatched = self.token_dispatcher.token_dispatch(build_token_dispatch_input(fused_experts_input=f))
        mlp_out, before_gmm2_evt = unified_apply_mlp(mlp_compute_input=build_mlp_compute_input(
            fused_experts_input=f, token_dispatch_output=dispatched, moe_config=self.moe_config))
        before_combine_evt = stream.record_event() if stream else None
        shared_out = f.shared_out
        if f.shared_experts is not None and shared_out is not None:
            f.shared_experts.wait()  # side-stream MLP must be done before its output is added
        routed_out = self.token_dispatcher.token_combine(hidden_states=mlp_out,
                                                         combine_metadata=dispatched.combine_metadata,
                                                         residual=shared_out)
        return FusedExpertsResult(routed_out=routed_out, before_dispatch_evt=before_dispatch_evt,
                                  before_gmm2_evt=before_gmm2_evt, before_combine_evt=before_combine_evt,
                                  group_list_type=dispatched.group_list_type, expert_tokens=dispatched.group_list,
                                  shared_out=shared_out)
