"""Frozen records that carry one MoE invocation through dispatch -> MLP -> combine.
Field names follow the reference's ``vllm_ascend/ops/fused_moe/dataclass/*.py`` so that
code reading them (``fused_experts_input.weights.w1_scale`` ...) is unchanged."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from ..quant_type import QuantType


@dataclass(frozen=True)
class FusedMoEConfig:
    """Stand-in for vLLM's ``FusedMoEConfig``: the fields this path reads
    (``moe_comm_method.py:55-62,195-200``, ``dataclass/moe_mlp.py:67-78``)."""

    num_experts: int
    experts_per_token: int
    hidden_dim: int
    intermediate_size_per_partition: int
    num_local_experts: int | None = None
    in_dtype: torch.dtype = torch.bfloat16
    activation: str = "silu"
    swiglu_limit: float = 0.0
    swiglu_alpha: float = 1.0
    swiglu_beta: float = 0.0
    ep_size: int = 1
    dp_size: int = 1
    pcp_size: int = 1
    tp_size: int = 1
    is_sequence_parallel: bool = False

    def __post_init__(self):
        if self.num_local_experts is None:
            object.__setattr__(self, "num_local_experts", self.num_experts)
        if (self.ep_size, self.dp_size, self.pcp_size, self.tp_size) != (1, 1, 1, 1):
            raise NotImplementedError("this build runs the whole layer on one GPU: ep/dp/pcp/tp sizes must be 1")


@dataclass(frozen=True)
class MoEWeights:
    w1: torch.Tensor | list[torch.Tensor]
    w2: torch.Tensor | list[torch.Tensor]
    w1_bias: torch.Tensor | None = None
    w2_bias: torch.Tensor | None = None
    w1_scale: torch.Tensor | list[torch.Tensor] | None = None
    w2_scale: torch.Tensor | list[torch.Tensor] | None = None
    w1_scale_bias: torch.Tensor | list[torch.Tensor] | None = None
    w2_scale_bias: torch.Tensor | list[torch.Tensor] | None = None
    w1_offset: torch.Tensor | None = None
    w2_offset: torch.Tensor | None = None


@dataclass(frozen=True)
class MoeRouterInput:
    expert_map: torch.Tensor | None = None
    global_redundant_expert_num: int = 0
    mc2_mask: torch.Tensor | None = None
    apply_router_weight_on_input: bool = False
    log2phy: torch.Tensor | None = None
    pertoken_scale: torch.Tensor | None = None


@dataclass(frozen=True)
class MoEQuantParams:
    quant_type: QuantType = QuantType.NONE
    comm_quant_mode: int | None = None
    is_per_channel_weight: bool = False
    w4_group_size: int = 0

    @property
    def is_quant(self) -> bool:
        return self.quant_type != QuantType.NONE

    @property
    def is_int_quant(self) -> bool:
        return self.quant_type in (QuantType.W8A8, QuantType.W4A8)

    @property
    def dispatch_with_quant(self) -> bool:
        return self.is_int_quant

    @property
    def use_w4a8_per_channel_gmm_swiglu(self) -> bool:
        return self.quant_type == QuantType.W4A8 and self.is_per_channel_weight


@dataclass(frozen=True)
class MoEFusedExpertsInput:
    hidden_states: torch.Tensor
    topk_weights: torch.Tensor
    topk_ids: torch.Tensor
    weights: MoEWeights
    routing: MoeRouterInput
    quant: MoEQuantParams
    activation: Any = "silu"
    need_trans: bool = False
    dynamic_eplb: bool = False
    lora_context: Any = None
    # not in the reference: output of the shared expert, added in fp32 inside the combine kernel
    # (the reference returns both tensors and upstream vLLM adds them)
    shared_out: torch.Tensor | None = None
    shared_experts: Any = None


@dataclass(frozen=True)
class MoETokenDispatchInput:
    hidden_states: torch.Tensor
    topk_weights: torch.Tensor
    topk_ids: torch.Tensor
    routing: MoeRouterInput
    quant: MoEQuantParams


@dataclass(frozen=True)
class MoEAllGatherCombineMetadata:
    topk_weights: torch.Tensor
    expanded_row_idx: torch.Tensor
    restore_shape: torch.Size


@dataclass(frozen=True)
class MoETokenDispatchOutput:
    hidden_states: torch.Tensor
    group_list: torch.Tensor
    group_list_type: int
    combine_metadata: MoEAllGatherCombineMetadata
    dynamic_scale: torch.Tensor | None = None
    topk_scales: torch.Tensor | None = None


@dataclass(frozen=True)
class MoEMlpComputeInput:
    hidden_states: torch.Tensor
    group_list: torch.Tensor
    group_list_type: int
    dynamic_scale: torch.Tensor | None
    topk_scales: torch.Tensor | None
    weights: MoEWeights
    quant: MoEQuantParams
    fusion: bool
    activation: Any = "silu"
    need_trans: bool = False
    dynamic_eplb: bool = False
    swiglu_limit: float = 0.0
    swiglu_alpha: float = 1.0
    swiglu_beta: float = 0.0
    expanded_row_idx: torch.Tensor | None = None
    topk_ids: torch.Tensor | None = None
    lora_context: Any = None
    # dtype of the layer's hidden states (the dispatcher may already have quantised them to int8): what the down
    # projection writes.  Not in the reference, which takes it from the dtype of the w2 scale.
    output_dtype: torch.dtype | None = None


@dataclass
class FusedExpertsResult:
    """What ``fused_experts`` hands back (``moe_comm_method.py:65-76``): the routed output,
    the stream events a shared expert would wait on, and the per-expert token counts."""

    routed_out: torch.Tensor
    before_dispatch_evt: Any = None
    before_gmm2_evt: Any = None
    before_combine_evt: Any = None
    group_list_type: int = 1
    expert_tokens: torch.Tensor | None = None
    # set when a shared expert ran with the layer: its output is already added into routed_out
    shared_out: torch.Tensor | None = None


def build_fused_experts_input(*, hidden_states, topk_weights, topk_ids, w1, w2, quant_type: QuantType,
                              dynamic_eplb: bool = False, expert_map=None, global_redundant_expert_num: int = 0,
                              mc2_mask=None, apply_router_weight_on_input: bool = False, pertoken_scale=None,
                              activation="silu", need_trans: bool = False, w1_bias=None, w2_bias=None,
                              comm_quant_mode=None, is_per_channel_weight: bool = False, w4_group_size: int = 0,
                              w1_scale=None, w2_scale=None, w1_scale_bias=None, w2_scale_bias=None, w1_offset=None,
                              w2_offset=None, lora_context=None, shared_out=None,
                              shared_experts=None) -> MoEFusedExpertsInput:
    return MoEFusedExpertsInput(
        hidden_states=hidden_states,
        topk_weights=topk_weights,
        topk_ids=topk_ids,
        weights=MoEWeights(w1=w1, w2=w2, w1_bias=w1_bias, w2_bias=w2_bias, w1_scale=w1_scale, w2_scale=w2_scale,
                           w1_scale_bias=w1_scale_bias, w2_scale_bias=w2_scale_bias, w1_offset=w1_offset,
                           w2_offset=w2_offset),
        routing=MoeRouterInput(expert_map=expert_map, global_redundant_expert_num=global_redundant_expert_num,
                               mc2_mask=mc2_mask, apply_router_weight_on_input=apply_router_weight_on_input,
                               pertoken_scale=pertoken_scale),
        quant=MoEQuantParams(quant_type=quant_type, comm_quant_mode=comm_quant_mode,
                             is_per_channel_weight=is_per_channel_weight, w4_group_size=w4_group_size),
        activation=activation,
        need_trans=need_trans,
        dynamic_eplb=dynamic_eplb,
        lora_context=lora_context,
        shared_out=shared_out,
        shared_experts=shared_experts,
    )


def build_token_dispatch_input(*, fused_experts_input: MoEFusedExpertsInput) -> MoETokenDispatchInput:
    f = fused_experts_input
    return MoETokenDispatchInput(hidden_states=f.hidden_states, topk_weights=f.topk_weights, topk_ids=f.topk_ids,
                                 routing=f.routing, quant=f.quant)


def build_mlp_compute_input(*, fused_experts_input: MoEFusedExpertsInput,
                            token_dispatch_output: MoETokenDispatchOutput, moe_config: FusedMoEConfig | None = None,
                            use_fusion_ops: bool | None = None) -> MoEMlpComputeInput:
    f, d = fused_experts_input, token_dispatch_output
    cfg = moe_config
    fusion_on = True if use_fusion_ops is None else use_fusion_ops
    return MoEMlpComputeInput(
        hidden_states=d.hidden_states,
        group_list=d.group_list,
        group_list_type=d.group_list_type,
        dynamic_scale=d.dynamic_scale,
        topk_scales=d.topk_scales,
        weights=f.weights,
        quant=f.quant,
        fusion=f.quant.quant_type == QuantType.W8A8 and fusion_on,
        activation=f.activation if cfg is None else getattr(cfg, "activation", f.activation),
        need_trans=f.need_trans,
        dynamic_eplb=f.dynamic_eplb,
        swiglu_limit=0.0 if cfg is None else (getattr(cfg, "swiglu_limit", 0.0) or 0.0),
        swiglu_alpha=1.0 if cfg is None else (getattr(cfg, "swiglu_alpha", 1.0) or 1.0),
        swiglu_beta=0.0 if cfg is None else (getattr(cfg, "swiglu_beta", 0.0) or 0.0),
        expanded_row_idx=getattr(d.combine_metadata, "expanded_row_idx", None),
        topk_ids=f.topk_ids,
        lora_context=f.lora_context,
        output_dtype=f.hidden_states.dtype if f.hidden_states.dtype in (torch.bfloat16, torch.float16) else None,
    )
