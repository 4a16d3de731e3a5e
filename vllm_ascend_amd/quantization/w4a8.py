"""W4A8-dynamic fused-MoE scheme: int4 weights, int8 per-token activations quantised on the fly.
Same ``apply()`` contract as ``AscendW4A8DynamicFusedMoEMethod``
(``vllm_ascend/quantization/methods/w4a8.py:36-421``), for the checkpoint form that stores one
int4 value per int8 (``[E, 2I, H]`` / ``[E, H, I]``).

Differences that come from the hardware, not from the mathematics:
- the Ascend kernel feeds its int4 cube with ``x = 16*hi + (lo - 8) + 8`` and therefore needs the
  ``scale_bias = 8 * sum_k w*scale`` correction (``w4a8.py:385-394``); MI355X unpacks the nibbles to
  int8 and multiplies them with the int8 activations directly, so no correction term exists;
- scales stay fp32 tensors (the reference widens their bits into int64, ``w4a8.py:320-325``);
- per-group scales along K (``group_size > 0``) are supported, as the reference's kernel does
  (``csrc/gmm/grouped_matmul_swiglu_quant/op_host/grouped_matmul_swiglu_quant_tiling.cpp:157-163``)
  although its Python scheme rejects them (``w4a8.py:113-120``)."""
from __future__ import annotations

from typing import Any

import torch

from .. import kernels
from ..fused_moe.contracts import MoEMlpComputeInput, build_fused_experts_input
from ..fused_moe.forward_context import _EXTRA_CTX
from ..quant_type import QuantType
from .base import AscendMoEScheme, fused_front_supported, register_scheme, route_and_quantize


@register_scheme("W4A8_DYNAMIC", "moe")
class AscendW4A8DynamicFusedMoEMethod(AscendMoEScheme):
    supports_eplb = True
    quant_type: QuantType = QuantType.W4A8

    def __init__(self, group_size: int = 0, in_dtype: torch.dtype = torch.bfloat16):
        if group_size < 0 or group_size % 64 != 0:
            raise ValueError("group_size must be 0 (per channel) or a multiple of 64")
        self.group_size = group_size
        self.in_dtype = in_dtype
        self.dynamic_eplb = False
        self.use_expert_weight_list = False
        self.moe_all_to_all_group_name = ""

    def get_weight(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                   params_dtype: torch.dtype) -> dict[str, Any]:
        # one int4 value (-8..7) per int8, as LLM-Compressor checkpoints store them (w4a8.py:146-157)
        return {
            "w13_weight": torch.empty(num_experts, 2 * intermediate_size_per_partition, hidden_sizes,
                                      dtype=torch.int8),
            "w2_weight": torch.empty(num_experts, hidden_sizes, intermediate_size_per_partition, dtype=torch.int8),
        }

    def get_dynamic_quant_param(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                                params_dtype: torch.dtype) -> dict[str, Any]:
        g = self.group_size
        g13 = hidden_sizes // g if g else 1
        g2 = intermediate_size_per_partition // g if g else 1
        return {
            "w13_weight_scale": torch.empty(num_experts, 2 * intermediate_size_per_partition, g13,
                                            dtype=torch.float32),
            "w2_weight_scale": torch.empty(num_experts, hidden_sizes, g2, dtype=torch.float32),
        }

    def process_weights_after_loading(self, layer) -> None:
        """int4 values -> tiled int4 storage (two per byte); scales [E, N, G] -> fp32 [E, G, N]."""
        e, n13, k13 = layer.w13_weight.data.shape
        _, n2, k2 = layer.w2_weight.data.shape
        layer.w4_shapes = {"w13": (n13, k13), "w2": (n2, k2)}
        layer.w13_weight.data = kernels.format_cast_nz_int4(layer.w13_weight.data, 0, n13, k13)
        layer.w2_weight.data = kernels.format_cast_nz_int4(layer.w2_weight.data, 0, n2, k2)
        layer.w13_weight_scale.data = layer.w13_weight_scale.data.to(torch.float32).transpose(1, 2).contiguous()
        layer.w2_weight_scale.data = layer.w2_weight_scale.data.to(torch.float32).transpose(1, 2).contiguous()

    def apply(self, layer, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              shared_experts: Any | None = None, shared_experts_input: torch.Tensor | None = None):
        topk_weights = topk_weights.to(x.dtype)
        moe_comm_method = _EXTRA_CTX.moe_comm_method
        if moe_comm_method is None:
            raise RuntimeError("no MoE communication method is set up (call setup_moe_comm_method first)")
        if (getattr(layer, "use_fused_small_batch", True) and shared_experts_input is None
                and self._plain_call(layer, x) and topk_ids.dim() == 2 and topk_ids.shape[0] == x.shape[0]):
            return self._apply_row_map(layer, x, topk_weights, topk_ids, shared_experts)
        shared_out = None
        if shared_experts is not None:
            # the shared expert sees the same hidden states unless the caller hands over others
            shared_out = shared_experts(x if shared_experts_input is None else shared_experts_input)
        return moe_comm_method.fused_experts(
            fused_experts_input=build_fused_experts_input(
                hidden_states=x,
                topk_weights=topk_weights,
                topk_ids=topk_ids,
                w1=[layer.w13_weight],
                w2=[layer.w2_weight],
                quant_type=self.quant_type,
                dynamic_eplb=self.use_expert_weight_list,
                expert_map=getattr(layer, "ascend_expert_map", None),
                global_redundant_expert_num=getattr(layer, "global_redundant_expert_num", 0),
                mc2_mask=getattr(layer, "ascend_mc2_mask", None),
                apply_router_weight_on_input=getattr(layer, "apply_router_weight_on_input", False),
                pertoken_scale=getattr(layer, "ascend_pertoken_scale", None),
                activation=getattr(layer, "activation", "silu"),
                shared_out=shared_out,
                shared_experts=shared_experts,
                w1_scale=[layer.w13_weight_scale],
                w2_scale=[layer.w2_weight_scale],
                w1_scale_bias=None,
                w2_scale_bias=None,
                is_per_channel_weight=self.group_size == 0,
                w4_group_size=self.group_size,
            ))

    # ------------------------------------------------------------------ token rows quantised once, read through a map
    def _plain_call(self, layer, x: torch.Tensor) -> bool:
        """16-bit hidden states as a [T, H] matrix, none of the optional inputs of ``apply``, SiLU."""
        if self.use_expert_weight_list or not x.is_cuda or x.dim() != 2 or x.shape[0] == 0:
            return False
        if x.dtype not in (torch.bfloat16, torch.float16) or x.dtype != self.in_dtype:
            return False
        if (getattr(layer, "apply_router_weight_on_input", False) or getattr(layer, "ascend_pertoken_scale", None)
                is not None or getattr(layer, "ascend_expert_map", None) is not None
                or getattr(layer, "ascend_mc2_mask", None) is not None
                or getattr(layer, "global_redundant_expert_num", 0)):
            return False
        act = getattr(layer, "activation", "silu")
        return (getattr(act, "value", act) or "silu") == "silu"

    def _apply_row_map(self, layer, x, topk_weights, topk_ids, shared_experts=None):
        """``apply`` without the permuted copy of the activations, as the W8A8 scheme does it: every token row is
        quantised once, routing builds the index maps only, the gate_up GEMM reads its rows through the
        row -> token map.  Same results, bit for bit, as the op-by-op path
        (``vllm_ascend/ops/fused_moe/moe_comm_method.py:117-162``, ``moe_mlp.py:425-451, 552-569``)."""
        before_dispatch_evt = torch.cuda.current_stream().record_event()
        xq, x_scale = kernels.dynamic_quant(x)
        shared_out = None
        if shared_experts is not None:
            shared_out = shared_experts(x, quantized=(xq, x_scale))
        expanded_row_idx, row_token, expert_tokens = kernels.route_map(topk_ids, layer.w13_weight.shape[0], 1)
        return self._experts_on_row_map(layer, x, xq, x_scale, row_token, expanded_row_idx, expert_tokens,
                                        topk_weights, shared_experts, shared_out, before_dispatch_evt)

    def supports_small_batch(self, layer, x: torch.Tensor, router_logits: torch.Tensor, router) -> bool:
        """Whether ``apply_small_batch`` can take this call, router included (the W8A8 scheme's rule)."""
        return self._plain_call(layer, x) and fused_front_supported(layer, x, router_logits, router)

    def apply_small_batch(self, layer, x: torch.Tensor, router_logits: torch.Tensor, router,
                          shared_experts: Any | None = None, shared_experts_input: torch.Tensor | None = None):
        """router + ``apply`` with gating, token quantisation and (for small batches) the dispatch maps in one
        launch; same results, bit for bit, as ``router.select_experts`` followed by ``apply``."""
        before_dispatch_evt = torch.cuda.current_stream().record_event()
        topk_weights, topk_ids, xq, x_scale, expanded_row_idx, row_token, expert_tokens = \
            route_and_quantize(layer, x, router_logits, router)
        shared_out = None
        if shared_experts is not None:
            if shared_experts_input is None:
                shared_out = shared_experts(x, quantized=(xq, x_scale))
            else:
                shared_out = shared_experts(shared_experts_input)
        return self._experts_on_row_map(layer, x, xq, x_scale, row_token, expanded_row_idx, expert_tokens,
                                        topk_weights, shared_experts, shared_out, before_dispatch_evt)

    def _experts_on_row_map(self, layer, x, xq, x_scale, row_token, expanded_row_idx, expert_tokens, topk_weights,
                            shared_experts, shared_out, before_dispatch_evt):
        from ..fused_moe.contracts import FusedExpertsResult

        stream = torch.cuda.current_stream()
        w1, w2 = layer.w13_weight, layer.w2_weight
        s1, s2 = layer.w13_weight_scale, layer.w2_weight_scale
        k1, n1 = x.shape[1], s1.shape[-1]
        g1 = k1 // s1.shape[1]
        k2, n2 = n1 // 2, s2.shape[-1]
        g2 = k2 // s2.shape[1]
        cfg = getattr(layer, "moe_config", None)
        swiglu_limit = (getattr(cfg, "swiglu_limit", 0.0) or 0.0) if cfg is not None else 0.0
        q1, q1_scale = kernels.gmm1_swiglu_quant_w4_gather(xq, x_scale, row_token, w1, s1, g1, expert_tokens, 1, n1, k1,
                                                           swiglu_limit=swiglu_limit)
        before_gmm2_evt = stream.record_event()
        out = kernels.gmm2_dequant_w4(q1, w2, s2, g2, q1_scale, expert_tokens, 1, n2, k2, out_dtype=x.dtype)
        before_combine_evt = stream.record_event()
        if shared_experts is not None and shared_out is not None:
            shared_experts.wait()
        routed_out = kernels.token_unpermute(out, expanded_row_idx, topk_weights, shared_out)
        return FusedExpertsResult(routed_out=routed_out, before_dispatch_evt=before_dispatch_evt,
                                  before_gmm2_evt=before_gmm2_evt, before_combine_evt=before_combine_evt,
                                  group_list_type=1, expert_tokens=expert_tokens, shared_out=shared_out)

    @staticmethod
    def get_eplb_weight_views(layer) -> list:
        return [layer.w13_weight, layer.w2_weight, layer.w13_weight_scale, layer.w2_weight_scale]


def _one(t):
    return t[0] if isinstance(t, (list, tuple)) else t


def w4a8_apply_mlp(m: MoEMlpComputeInput):
    """gate_up GEMM (int4 weights) + SwiGLU + re-quant, then the down GEMM: the W4A8 branch of
    ``quant_apply_mlp`` (``vllm_ascend/ops/fused_moe/moe_mlp.py:425-451, 552-569``)."""
    act = getattr(m.activation, "value", m.activation) or "silu"
    if act != "silu":
        raise NotImplementedError(f"activation {act!r}: only 'silu' (SwiGLU) has a fused MI355X kernel")
    if m.dynamic_eplb:
        raise NotImplementedError("per-expert weight lists (dynamic EPLB) are not built yet")
    if m.dynamic_scale is None:
        raise NotImplementedError("the W4A8 path expects activations quantised by the dispatcher")
    w1, w2 = _one(m.weights.w1), _one(m.weights.w2)
    s1, s2 = _one(m.weights.w1_scale), _one(m.weights.w2_scale)
    x = m.hidden_states
    k1, n1 = x.shape[1], s1.shape[-1]
    g1 = k1 // s1.shape[1]
    k2, n2 = n1 // 2, s2.shape[-1]
    g2 = k2 // s2.shape[1]
    q1, q1_scale = kernels.gmm1_swiglu_quant_w4(x, w1, s1, g1, m.dynamic_scale, m.group_list, m.group_list_type, n1, k1,
                                                swiglu_limit=m.swiglu_limit)
    evt = torch.cuda.current_stream().record_event() if x.is_cuda else None
    out = kernels.gmm2_dequant_w4(q1, w2, s2, g2, q1_scale, m.group_list, m.group_list_type, n2, k2,
                                  out_dtype=m.output_dtype or torch.bfloat16)
    return out, evt
