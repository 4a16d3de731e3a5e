"""W8A8-dynamic fused-MoE scheme: int8 per-channel weights, int8 per-token activations
quantised on the fly.  Same contract as ``AscendW8A8DynamicFusedMoEMethod``
(``vllm_ascend/quantization/methods/w8a8_dynamic.py:165-399``): parameter names and
shapes, ``process_weights_after_loading`` and ``apply(layer, x, topk_weights, topk_ids,
shared_experts, shared_experts_input)``."""
from __future__ import annotations

from typing import Any

import torch

from .. import npu_ops
from ..fused_moe.contracts import build_fused_experts_input
from ..fused_moe.forward_context import _EXTRA_CTX
from ..quant_type import QuantType
from .base import AscendMoEScheme, fused_front_supported, register_scheme, route_and_quantize


@register_scheme("W8A8_DYNAMIC", "moe")
class AscendW8A8DynamicFusedMoEMethod(AscendMoEScheme):
    supports_eplb = True
    quant_type: QuantType = QuantType.W8A8

    def __init__(self, in_dtype: torch.dtype = torch.bfloat16, dynamic_eplb: bool = False):
        # The reference reads these from the vLLM / Ascend configs (w8a8_dynamic.py:173-196);
        # there is no vLLM here, so they are constructor arguments with the 1-GPU defaults.
        self.in_dtype = in_dtype
        self.dynamic_eplb = dynamic_eplb
        # per-expert tensors that can be swapped one by one (w8a8_dynamic.py:180-183, 365-389)
        self.use_expert_weight_list = dynamic_eplb
        self.use_aclgraph = False
        self.moe_all_to_all_group_name = ""  # no MC2 group on one device

    def get_weight(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                   params_dtype: torch.dtype) -> dict[str, Any]:
        return {
            "w13_weight": torch.empty(num_experts, 2 * intermediate_size_per_partition, hidden_sizes,
                                      dtype=torch.int8),
            "w2_weight": torch.empty(num_experts, hidden_sizes, intermediate_size_per_partition, dtype=torch.int8),
        }

    def get_dynamic_quant_param(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                                params_dtype: torch.dtype) -> dict[str, Any]:
        two_i = 2 * intermediate_size_per_partition
        return {
            "w13_weight_scale": torch.empty(num_experts, two_i, 1, dtype=params_dtype),
            "w13_weight_offset": torch.empty(num_experts, two_i, 1, dtype=params_dtype),
            "w2_weight_scale": torch.empty(num_experts, hidden_sizes, 1, dtype=params_dtype),
            "w2_weight_offset": torch.empty(num_experts, hidden_sizes, 1, dtype=params_dtype),
        }

    def process_weights_after_loading(self, layer) -> None:
        """Checkpoint order ``[E, N, K]`` -> logical ``[E, K, N]`` in the MFMA-tiled storage the
        grouped GEMMs stream (the reference transposes, then casts to FRACTAL_NZ:
        w8a8_dynamic.py:345-357); scales squeezed to ``[E, N]``; fp32 copies of both scales
        (the reference keeps the w2 scale in the model dtype; the kernels take fp32)."""
        layer.w13_weight.data = npu_ops.format_cast_from_checkpoint(layer.w13_weight.data)
        layer.w2_weight.data = npu_ops.format_cast_from_checkpoint(layer.w2_weight.data)
        for name in ("w13_weight_scale", "w13_weight_offset", "w2_weight_scale", "w2_weight_offset"):
            p = getattr(layer, name, None)
            if p is not None:
                p.data = p.data.view(p.data.shape[0], -1)
        layer.w13_weight_scale_fp32 = layer.w13_weight_scale.data.to(torch.float32)
        layer.w2_weight_scale_fp32 = layer.w2_weight_scale.data.to(torch.float32)
        if self.use_expert_weight_list:
            # each list carries the device table of its tensors' addresses, built here once; swapping an expert
            # (lst[e] = tensor) rewrites one entry of that table
            from ..kernels import ExpertTensorList

            layer.w13_weight_list = ExpertTensorList([w.clone() for w in layer.w13_weight.data.unbind(dim=0)],
                                                     "w13_weight")
            layer.w2_weight_list = ExpertTensorList([w.clone() for w in layer.w2_weight.data.unbind(dim=0)],
                                                    "w2_weight")
            layer.w13_weight_scale_fp32_list = ExpertTensorList(
                [s.clone() for s in layer.w13_weight_scale_fp32.unbind(dim=0)], "w13_weight_scale")
            layer.w2_weight_scale_list = ExpertTensorList(
                [s.clone() for s in layer.w2_weight_scale_fp32.unbind(dim=0)], "w2_weight_scale")
            del layer.w13_weight, layer.w2_weight, layer.w13_weight_scale, layer.w2_weight_scale
            del layer.w13_weight_scale_fp32, layer.w2_weight_scale_fp32

    def apply(self, layer, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              shared_experts: Any | None = None, shared_experts_input: torch.Tensor | None = None):
        assert topk_ids is not None
        assert topk_weights is not None
        topk_weights = topk_weights.to(self.in_dtype)
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
                w1=layer.w13_weight_list if self.use_expert_weight_list else [layer.w13_weight],
                w2=layer.w2_weight_list if self.use_expert_weight_list else [layer.w2_weight],
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
                w1_scale=(layer.w13_weight_scale_fp32_list if self.use_expert_weight_list
                          else [layer.w13_weight_scale_fp32]),
                w2_scale=layer.w2_weight_scale_list if self.use_expert_weight_list else [layer.w2_weight_scale_fp32],
            ))

    # ------------------------------------------------------------------ token rows quantised once, read through a map
    def _plain_call(self, layer, x: torch.Tensor) -> bool:
        """Plain W8A8 weights (no per-expert lists), 16-bit hidden states as a [T, H] matrix, none of the optional
        inputs of ``apply``, SiLU: the calls whose token rows need not be copied k times."""
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

    def _apply_row_map(self, layer, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                       shared_experts: Any | None = None):
        """``apply`` without the permuted copy of the activations: every token row is quantised once
        (the k copies that ``npu_moe_init_routing_v2(quant_mode=1)`` writes hold the same bytes and the same
        scale), the routing step only builds the two index maps, and the gate_up GEMM reads its rows through the
        row -> token map.  The shared expert takes the same quantised rows.  Same results, bit for bit, as the
        op-by-op path (``vllm_ascend/ops/fused_moe/moe_comm_method.py:117-162``)."""
        from .. import kernels
        from ..fused_moe.contracts import FusedExpertsResult

        stream = torch.cuda.current_stream()
        before_dispatch_evt = stream.record_event()
        xq, x_scale = kernels.dynamic_quant(x)
        shared_out = None
        if shared_experts is not None:
            shared_out = shared_experts(x, quantized=(xq, x_scale))
        expanded_row_idx, row_token, expert_tokens = kernels.route_map(topk_ids, layer.w13_weight.shape[0], 1)
        return self._experts_on_row_map(layer, x, xq, x_scale, row_token, expanded_row_idx, expert_tokens,
                                        topk_weights, shared_experts, shared_out, before_dispatch_evt)

    def _experts_on_row_map(self, layer, x, xq, x_scale, row_token, expanded_row_idx, expert_tokens, topk_weights,
                            shared_experts, shared_out, before_dispatch_evt):
        from .. import kernels
        from ..fused_moe.contracts import FusedExpertsResult

        stream = torch.cuda.current_stream()
        w13, w2 = layer.w13_weight, layer.w2_weight
        cfg = getattr(layer, "moe_config", None)
        swiglu_limit = (getattr(cfg, "swiglu_limit", 0.0) or 0.0) if cfg is not None else 0.0
        q1, q1_scale = kernels.gmm1_swiglu_quant_gather(xq, x_scale, row_token, w13, layer.w13_weight_scale_fp32,
                                                        expert_tokens, 1, w13.shape[2], w13.shape[1], swiglu_limit)
        before_gmm2_evt = stream.record_event()
        out = kernels.gmm2_dequant(q1, w2, layer.w2_weight_scale_fp32, q1_scale, expert_tokens, 1, w2.shape[2],
                                   w2.shape[1], out_dtype=x.dtype)
        before_combine_evt = stream.record_event()
        if shared_experts is not None and shared_out is not None:
            shared_experts.wait()
        routed_out = kernels.token_unpermute(out, expanded_row_idx, topk_weights, shared_out)
        return FusedExpertsResult(routed_out=routed_out, before_dispatch_evt=before_dispatch_evt,
                                  before_gmm2_evt=before_gmm2_evt, before_combine_evt=before_combine_evt,
                                  group_list_type=1, expert_tokens=expert_tokens, shared_out=shared_out)

    # ------------------------------------------------------------------ small batches (decode)
    def supports_small_batch(self, layer, x: torch.Tensor, router_logits: torch.Tensor, router) -> bool:
        """Whether ``apply_small_batch`` can take this call, router included: a plain call (see ``_plain_call``),
        no forced load balance, at most 256 experts.  (The name is from the time when only batches of at most 1024
        (token, slot) pairs had such a form; those still get gating, dispatch and quantisation in ONE launch,
        larger ones gating and quantisation.)"""
        return self._plain_call(layer, x) and fused_front_supported(layer, x, router_logits, router)

    def apply_small_batch(self, layer, x: torch.Tensor, router_logits: torch.Tensor, router,
                          shared_experts: Any | None = None, shared_experts_input: torch.Tensor | None = None):
        """router + ``apply`` for a small batch in four launches instead of six: gating and dispatch are one
        kernel (the token rows are quantised once, in token order, and the gate_up GEMM reads them through the
        row -> token map), then the gate_up GEMM with SwiGLU and re-quantisation, the down GEMM and the combine.
        Same results, bit for bit, as ``router.select_experts`` followed by ``apply``
        (``vllm_ascend/ops/fused_moe/routed_experts.py:496-609``, ``w8a8_dynamic.py:224-301``)."""
        before_dispatch_evt = torch.cuda.current_stream().record_event()
        if self._pair_order(layer, x, router_logits, router):
            return self._experts_in_pair_order(layer, x, router_logits, router, shared_experts, shared_experts_input,
                                               before_dispatch_evt)
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

    # ------------------------------------------------------------------ decode batches: no sort at all
    @staticmethod
    def _pair_order(layer, x: torch.Tensor, router_logits: torch.Tensor, router) -> bool:
        """At most 1024 (token, slot) pairs that the grouped GEMMs would stream the weights for anyway, ids
        straight from the gate (always in range)."""
        from .. import kernels

        if not getattr(layer, "use_pair_order", True):
            return False
        T, k, E = x.shape[0], router.top_k, router_logits.shape[1]
        w13, w2 = layer.w13_weight, layer.w2_weight
        if not (kernels.gmm_pairs_supported(T, k, w13.shape[2], w13.shape[1])
                and kernels.gmm_pairs_supported(T, k, w2.shape[2], w2.shape[1])):
            return False
        experts = layer.w13_weight.shape[0]  # physical experts (more than E with redundant copies behind log2phy)
        if not kernels.gate_quant_supported(T, k, E) or experts > 2048:
            return False
        if experts * w13.shape[1] * w13.shape[2] >= 1 << 30 and T * k > 768:
            # A product of a GiB and more has a second kernel family for hot experts on the sorted path (csrc/gmm.hip:
            # gemm_plan), pair order streams every expert: DeepSeek-V3 shape under Zipf(1.1) routing, 112 / 128 tokens
            # 668 / 742 us in pair order, 625 / 641 us sorted; on uniform routing pair order leads by 1 % there.
            return False
        return T * k < 1024 or (T * k) // experts < 12  # where the sorted form streams as well (csrc/gmm.hip: tiled_bm)

    def _experts_in_pair_order(self, layer, x, router_logits, router, shared_experts, shared_experts_input,
                               before_dispatch_evt):
        """Five launches and no hand-off between workgroups: gating + token quantisation, the gate_up GEMM (its
        workgroups collect the pairs of their expert from the ids themselves), the re-quantisation, the down GEMM,
        and the combine, which also counts the pairs per expert.  Every intermediate row t * k + s belongs to slot
        s of token t; nothing is sorted.  Same results, bit for bit, as the sorted form."""
        from .. import kernels
        from ..fused_moe.contracts import FusedExpertsResult

        stream = torch.cuda.current_stream()
        bias = router.e_score_correction_bias
        if bias is not None and bias.dtype != router_logits.dtype:
            bias = router.e_score_correction_bias = bias.to(router_logits.dtype)
        topk_weights, topk_ids, xq, x_scale = kernels.gate_quant(
            x, router_logits, router.top_k, router.topk_group if router.topk_group is not None else 1,
            router.num_expert_group if router.num_expert_group is not None else 1, 1, int(router.renormalize),
            0 if router.scoring_func == "softmax" else 1, router.routed_scaling_factor, 1e-20, bias)
        log2phy = getattr(layer, "log2phy", None)
        if log2phy is not None:
            # logical -> physical expert ids (redundant experts of dynamic load balancing,
            # vllm_ascend/ops/fused_moe/routed_experts.py:452-453): the experts run over the physical ones
            topk_ids = log2phy[topk_ids.long()].to(torch.int32)
        shared_out = None
        if shared_experts is not None:
            if shared_experts_input is None:
                shared_out = shared_experts(x, quantized=(xq, x_scale))
            else:
                shared_out = shared_experts(shared_experts_input)
        w13, w2 = layer.w13_weight, layer.w2_weight
        cfg = getattr(layer, "moe_config", None)
        swiglu_limit = (getattr(cfg, "swiglu_limit", 0.0) or 0.0) if cfg is not None else 0.0
        T, k = topk_ids.shape
        if kernels.gmm2_requant_pairs_supported(T, k, w2.shape[2], w2.shape[1], w2.shape[0]):
            # four launches: the down GEMM re-quantises the SwiGLU values of its expert's rows itself
            y = kernels.gmm1_swiglu_pairs(xq, x_scale, topk_ids, w13, layer.w13_weight_scale_fp32, w13.shape[2],
                                          w13.shape[1], swiglu_limit)
            before_gmm2_evt = stream.record_event()
            out = kernels.gmm2_requant_dequant_pairs(y, w2, layer.w2_weight_scale_fp32, topk_ids, w2.shape[2],
                                                     w2.shape[1], out_dtype=x.dtype)
        else:
            q1, q1_scale = kernels.gmm1_swiglu_quant_pairs(xq, x_scale, topk_ids, w13, layer.w13_weight_scale_fp32,
                                                           w13.shape[2], w13.shape[1], swiglu_limit)
            before_gmm2_evt = stream.record_event()
            out = kernels.gmm2_dequant_pairs(q1, w2, layer.w2_weight_scale_fp32, q1_scale, topk_ids, w2.shape[2],
                                             w2.shape[1], out_dtype=x.dtype)
        before_combine_evt = stream.record_event()
        if shared_experts is not None and shared_out is not None:
            shared_experts.wait()
        routed_out, expert_tokens = kernels.token_unpermute_pairs(out, topk_weights, topk_ids, w13.shape[0], shared_out)
        return FusedExpertsResult(routed_out=routed_out, before_dispatch_evt=before_dispatch_evt,
                                  before_gmm2_evt=before_gmm2_evt, before_combine_evt=before_combine_evt,
                                  group_list_type=1, expert_tokens=expert_tokens, shared_out=shared_out)

    @staticmethod
    def get_eplb_weight_views(layer) -> list:
        if hasattr(layer, "w13_weight_list"):
            return [layer.w13_weight_list, layer.w2_weight_list, layer.w13_weight_scale_fp32_list,
                    layer.w2_weight_scale_list]
        return [layer.w13_weight, layer.w2_weight, layer.w13_weight_scale_fp32, layer.w2_weight_scale_fp32]
