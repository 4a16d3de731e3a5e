"""Scheme base class and registry (``vllm_ascend/quantization/methods/base.py:206-287``,
``methods/registry.py:24-62``)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any

import torch

from ..quant_type import QuantType

_SCHEMES: dict[tuple[str, str], type] = {}


def register_scheme(quant_name: str, layer_kind: str):
    def deco(cls):
        _SCHEMES[(quant_name, layer_kind)] = cls
        return cls

    return deco


def get_scheme_class(quant_name: str, layer_kind: str) -> type:
    try:
        return _SCHEMES[(quant_name, layer_kind)]
    except KeyError:
        raise NotImplementedError(f"no MI355X scheme registered for ({quant_name!r}, {layer_kind!r})") from None


class AscendMoEScheme(ABC):
    """A MoE quantisation scheme: weight specs, post-load layout and ``apply``."""

    quant_type: QuantType = QuantType.NONE

    @abstractmethod
    def get_weight(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                   params_dtype: torch.dtype) -> dict[str, Any]: ...

    @abstractmethod
    def get_dynamic_quant_param(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                                params_dtype: torch.dtype) -> dict[str, Any]: ...

    @abstractmethod
    def apply(self, layer: torch.nn.Module, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              shared_experts: Any | None, shared_experts_input: torch.Tensor | None): ...

    def get_eplb_weight_views(self, layer: torch.nn.Module) -> list:
        return []

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        return


# ---------------------------------------------------------------------- router + token quantisation, fused
def fused_front_supported(layer, x: torch.Tensor, router_logits: torch.Tensor, router) -> bool:
    """Whether :func:`route_and_quantize` can take the call: 2-D logits of a supported type, no forced load
    balance, at most 256 experts."""
    from .. import kernels

    if router_logits.dim() != 2 or router_logits.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        return False
    if getattr(layer, "enable_force_load_balance", False):
        return False
    guard = getattr(router, "is_fused_supported", None)
    if guard is not None and not guard(x):
        return False  # the router's own guard decides (and refuses) on the operator-by-operator path
    if getattr(layer, "log2phy", None) is not None:  # the ids are remapped between gating and dispatch
        return kernels.gate_quant_supported(x.shape[0], router.top_k, router_logits.shape[1])
    return (kernels.route_quant_small_supported(x.shape[0], router.top_k, router_logits.shape[1])
            or kernels.gate_quant_supported(x.shape[0], router.top_k, router_logits.shape[1]))


def route_and_quantize(layer, x: torch.Tensor, router_logits: torch.Tensor, router):
    """The router (``select_experts``), the per-token quantisation of the hidden states and the index maps of the
    dispatch, in one launch for at most 1024 (token, slot) pairs and in two for larger batches (gating and
    quantisation side by side, then the maps).  Returns ``(topk_weights, topk_ids, xq, x_scale,
    expanded_row_idx, row_token, expert_tokens)``; the token rows stay in token order and the gate_up GEMM reads
    them through ``row_token``.  Same values, bit for bit, as ``router.select_experts`` + ``npu_dynamic_quant`` +
    ``npu_moe_init_routing_v2`` (``vllm_ascend/ops/fused_moe/routed_experts.py:496-540``,
    ``token_dispatcher.py:404-420``)."""
    from .. import kernels

    bias = router.e_score_correction_bias
    if bias is not None and bias.dtype != router_logits.dtype:
        bias = router.e_score_correction_bias = bias.to(router_logits.dtype)
    gate_args = (router.top_k, router.topk_group if router.topk_group is not None else 1,
                 router.num_expert_group if router.num_expert_group is not None else 1, 1,
                 int(router.renormalize), 0 if router.scoring_func == "softmax" else 1,
                 router.routed_scaling_factor, 1e-20, bias)
    log2phy = getattr(layer, "log2phy", None)
    if log2phy is None and kernels.route_quant_small_supported(x.shape[0], router.top_k, router_logits.shape[1]):
        # the routing kernel's arrival counter: one zeroed int32 per layer (and device), which every call leaves
        # at zero; created on the first call (run the layer once before capturing it into a graph)
        counter = getattr(layer, "_small_batch_counter", None)
        if counter is None or counter.device != x.device:
            counter = layer._small_batch_counter = torch.zeros((1,), dtype=torch.int32, device=x.device)
        return kernels.route_quant_small(x, router_logits, *gate_args, sync_counter=counter)
    topk_weights, topk_ids, xq, x_scale = kernels.gate_quant(x, router_logits, *gate_args)
    num_experts = router_logits.shape[1]
    if log2phy is not None:
        # logical -> physical expert ids (redundant experts of dynamic load balancing,
        # vllm_ascend/ops/fused_moe/routed_experts.py:452-453): the dispatch runs over the physical experts
        topk_ids = log2phy[topk_ids.long()].to(torch.int32)
        num_experts = layer.moe_config.num_experts
    expanded_row_idx, row_token, expert_tokens = kernels.route_map(topk_ids, num_experts, 1)
    return topk_weights, topk_ids, xq, x_scale, expanded_row_idx, row_token, expert_tokens
