"""Grouped-GEMM expert MLP.  Counterpart of ``quant_apply_mlp`` / ``unified_apply_mlp``
(``vllm_ascend/ops/fused_moe/moe_mlp.py:174-570, 690-794``) for the branches a single
device takes: gate_up GEMM fused with dequant + SwiGLU + re-quant, then the down GEMM
with per-token x per-channel dequant."""
from __future__ import annotations

import torch

from ..device_op import DeviceOperator
from ..quant_type import QuantType
from .contracts import MoEMlpComputeInput


def cumsum_group_list(group_list: torch.Tensor, src_list_type: int, dst_list_type: int, active_num: int = 0,
                      expert_num: int = 0) -> torch.Tensor:
    """Convert a group list between 0 = running sum, 1 = counts, 2 = sparse (expert, count) pairs
    (``moe_mlp.py:54-83``)."""
    if src_list_type not in [0, 1, 2]:
        raise ValueError(f"group_list_type should be in [0, 1, 2], but received {src_list_type}")
    if src_list_type == dst_list_type:
        return group_list
    if (src_list_type, dst_list_type) == (1, 0):
        return group_list.cumsum(dim=0)
    if (src_list_type, dst_list_type) == (0, 1):
        return torch.cat([group_list[:1], torch.diff(group_list)], dim=0)
    if (src_list_type, dst_list_type) == (2, 0):
        out = torch.full((expert_num,), active_num, dtype=group_list.dtype, device=group_list.device)
        bounds = torch.nn.functional.pad(group_list[:, 0], (1, 0)).tolist()
        sums = torch.nn.functional.pad(group_list[:, 1].cumsum(dim=0), (1, 0))
        for i, (lo, hi) in enumerate(zip(bounds[:-1], bounds[1:])):
            if hi > lo:
                out[lo:hi] = sums[i]
        return out
    raise NotImplementedError(
        f"Conversion from src_list_type={src_list_type} to dst_list_type={dst_list_type} is not implemented yet. "
        "This feature is under development.")


def _single(tensor_or_list, name: str) -> torch.Tensor:
    if isinstance(tensor_or_list, (list, tuple)):
        if len(tensor_or_list) != 1:
            raise ValueError(f"{name} must be one tensor (or a list holding one) for the fused SwiGLU-quant op")
        return tensor_or_list[0]
    return tensor_or_list


def quant_apply_mlp(hidden_states, w1, w1_scale, w2, w2_scale, group_list, group_list_type: int = 1,
                    dynamic_scale=None, w1_scale_bias=None, w2_scale_bias=None, w1_offset=None, w2_offset=None,
                    fusion: bool = False, dynamic_eplb: bool = False, activation=None, swiglu_limit: float = 0.0,
                    swiglu_alpha: float = 1.0, swiglu_beta: float = 0.0,
                    use_w4a8_per_channel_gmm_swiglu: bool = False, output_dtype=None, **unsupported):
    act_name = getattr(activation, "value", activation) or "silu"
    from ..kernels import ACTIVATIONS

    if act_name == "swigluoai":
        # The reference's quantised MLP asks only for "swigluoai_uninterleave" (moe_mlp.py:213, 522-538); the
        # interleaved name takes its default branch, the fused SwiGLU with swiglu_limit, alpha and beta unused.
        act_name, swiglu_alpha, swiglu_beta = "silu", 1.0, 0.0

    if act_name != "silu" and act_name not in ACTIVATIONS:
        raise NotImplementedError(f"activation {act_name!r}: supported are 'silu' and {sorted(ACTIVATIONS)}")
    if act_name != "swigluoai_uninterleave" and (swiglu_alpha != 1.0 or swiglu_beta != 0.0):
        raise NotImplementedError("swiglu_alpha / swiglu_beta belong to the swigluoai activation")
    if w1_offset is not None or w2_offset is not None:
        raise NotImplementedError("asymmetric weight offsets are not supported")
    if unsupported.get("use_mxfp_quant"):
        raise NotImplementedError("MXFP quantisation is not supported on this path")
    if w1_scale_bias is not None or use_w4a8_per_channel_gmm_swiglu:
        raise NotImplementedError("W4A8 weights go through the W4A8 scheme's own MLP")
    input_dtype = hidden_states.dtype if hidden_states.dtype != torch.int8 else (output_dtype or torch.bfloat16)

    if dynamic_scale is None:
        hidden_states, pertoken_scale = DeviceOperator.npu_dynamic_quant(hidden_states=hidden_states)
    else:
        pertoken_scale = dynamic_scale

    if act_name != "silu":
        # No fused op for these: gate_up product dequantised to the hidden dtype, activation * up and the dynamic
        # quantiser in one pass, down product (the unfused branch of the reference, moe_mlp.py:484-569).
        from ..kernels import act_mul_quant

        gate_up = DeviceOperator.npu_grouped_matmul_gmm2(
            hidden_states=hidden_states, weight=w1 if isinstance(w1, (list, tuple)) and len(w1) > 1 else _single(w1, "w1"),
            weight_scale=(w1_scale if isinstance(w1_scale, (list, tuple)) and len(w1_scale) > 1
                          else _single(w1_scale, "w1_scale")),
            per_token_scale=pertoken_scale, group_list=group_list, group_list_type=group_list_type,
            input_dtype=input_dtype)
        limit = (swiglu_limit or 7.0) if act_name == "swiglustep" else swiglu_limit
        gl_ok = group_list_type in (0, 1)
        hidden_states, swiglu_out_scale = act_mul_quant(
            gate_up, act_name, limit, swiglu_alpha, swiglu_beta,
            group_list if gl_ok else cumsum_group_list(group_list, group_list_type, 0), group_list_type if gl_ok else 0)
        before_gmm2_evt = torch.cuda.current_stream().record_event() if hidden_states.is_cuda else None
        out = DeviceOperator.npu_grouped_matmul_gmm2(
            hidden_states=hidden_states, weight=w2 if isinstance(w2, (list, tuple)) and len(w2) > 1 else _single(w2, "w2"),
            weight_scale=(w2_scale if isinstance(w2_scale, (list, tuple)) and len(w2_scale) > 1
                          else _single(w2_scale, "w2_scale")),
            per_token_scale=swiglu_out_scale, group_list=group_list, group_list_type=group_list_type,
            input_dtype=input_dtype)
        return out, before_gmm2_evt
    if dynamic_eplb or (isinstance(w1, (list, tuple)) and len(w1) > 1):
        # per-expert weight lists (the form dynamic expert load balancing swaps in place)
        from ..kernels import ExpertTensorList, gmm1_swiglu_quant_list

        if isinstance(w1, ExpertTensorList) and isinstance(w1_scale, ExpertTensorList) and group_list_type in (0, 1):
            # the layer's own lists: their address tables were built at load time and are reused (a Tensor[]
            # argument of a torch operator arrives as a plain list and would need a table of its own per call)
            hidden_states, swiglu_out_scale = gmm1_swiglu_quant_list(hidden_states, w1, w1_scale, pertoken_scale,
                                                                     group_list, group_list_type, swiglu_limit)
        else:
            hidden_states, swiglu_out_scale, _ = (
                torch.ops._C_ascend.grouped_matmul_swiglu_quant_weight_nz_tensor_list(
                    x=hidden_states, weight=list(w1), weight_scale=list(w1_scale), x_scale=pertoken_scale,
                    group_list=cumsum_group_list(group_list, group_list_type, 0), bias=None,
                    swiglu_limit=swiglu_limit))
        before_gmm2_evt = torch.cuda.current_stream().record_event() if hidden_states.is_cuda else None
        out = DeviceOperator.npu_grouped_matmul_gmm2(
            hidden_states=hidden_states, weight=w2 if isinstance(w2, ExpertTensorList) else list(w2),
            weight_scale=w2_scale if isinstance(w2_scale, ExpertTensorList) else list(w2_scale),
            per_token_scale=swiglu_out_scale, group_list=group_list, group_list_type=group_list_type,
            input_dtype=input_dtype)
        return out, before_gmm2_evt
    # gmm1: gate_up_proj + dequant + SwiGLU + dynamic re-quant in one op
    hidden_states, swiglu_out_scale, _ = DeviceOperator.npu_grouped_matmul_swiglu_quant(
        x=hidden_states, weight=_single(w1, "w1"),
        group_list=group_list if group_list_type in (0, 1) else cumsum_group_list(group_list, group_list_type, 0),
        group_list_type=group_list_type if group_list_type in (0, 1) else 0,
        weight_scale=_single(w1_scale, "w1_scale"), x_scale=pertoken_scale, bias=None, swiglu_limit=swiglu_limit)
    before_gmm2_evt = torch.cuda.current_stream().record_event() if hidden_states.is_cuda else None
    # gmm2: down_proj + dequant
    out = DeviceOperator.npu_grouped_matmul_gmm2(
        hidden_states=hidden_states, weight=_single(w2, "w2"), weight_scale=_single(w2_scale, "w2_scale"), per_token_scale=swiglu_out_scale,
        group_list=group_list, group_list_type=group_list_type,
        input_dtype=input_dtype)
    return out, before_gmm2_evt


def unified_apply_mlp(*, mlp_compute_input: MoEMlpComputeInput):
    m = mlp_compute_input
    if m.quant.quant_type == QuantType.NONE:
        raise NotImplementedError("unquantised experts are outside this build (W8A8 / W4A8 dynamic only)")
    if m.quant.quant_type == QuantType.W4A8:
        from ..quantization.w4a8 import w4a8_apply_mlp

        return w4a8_apply_mlp(m)
    w = m.weights
    return quant_apply_mlp(
        hidden_states=m.hidden_states, w1=w.w1, w1_scale=w.w1_scale, w2=w.w2, w2_scale=w.w2_scale,
        group_list=m.group_list, group_list_type=m.group_list_type, dynamic_scale=m.dynamic_scale,
        w1_scale_bias=w.w1_scale_bias, w2_scale_bias=w.w2_scale_bias, w1_offset=w.w1_offset, w2_offset=w.w2_offset,
        fusion=m.fusion, dynamic_eplb=m.dynamic_eplb, activation=m.activation, swiglu_limit=m.swiglu_limit,
        swiglu_alpha=m.swiglu_alpha, swiglu_beta=m.swiglu_beta,
        use_w4a8_per_channel_gmm_swiglu=m.quant.use_w4a8_per_channel_gmm_swiglu, output_dtype=m.output_dtype)
