"""``torch.ops._C_ascend`` operators of the fused-MoE path, backed by libmoe355.so.

The schemas are the reference's (vllm-ascend ``csrc/torch_binding.cpp:2025-2053,
2135-2150, 2495-2512``), so code written against ``torch.ops._C_ascend.<op>``
runs unchanged.  Only the CUDA (= HIP on ROCm) dispatch key has an
implementation, plus Meta shape functions (``csrc/torch_binding_meta.cpp``) for
tracing; CPU tensors raise, there is no fallback.

Weight operands are always read as the tiled storage produced by
``npu_ops.npu_format_cast(w, ACL_FORMAT_FRACTAL_NZ)`` -- the reference's
``grouped_matmul_swiglu_quant`` is itself an alias of the ``_weight_nz`` op
(``csrc/gmm/grouped_matmul_swiglu_quant_weight_nz_tensor_list/grouped_matmul_swiglu_quant_torch_adpt.h:53-61``).
"""
from __future__ import annotations

import torch

from . import kernels

_LIB = None
_ENABLED = False

_SCHEMAS = [
    "moe_gating_top_k(Tensor x, int k, int k_group, int group_count, int group_select_mode, int renorm, "
    "int norm_type, bool out_flag, float routed_scaling_factor, float eps, Tensor? bias_opt=None) "
    "-> (Tensor y, Tensor expert_idx, Tensor out)",
    "grouped_matmul_swiglu_quant(Tensor x, Tensor weight, Tensor weight_scale, Tensor x_scale, Tensor group_list, *, "
    "Tensor? bias=None, Tensor? offset=None, float swiglu_limit=0.0) "
    "-> (Tensor output, Tensor output_scale, Tensor output_offset)",
    "grouped_matmul_swiglu_quant_weight_nz(Tensor x, Tensor weight, Tensor weight_scale, Tensor x_scale, "
    "Tensor group_list, *, Tensor? bias=None, Tensor? offset=None, float swiglu_limit=0.0) "
    "-> (Tensor output, Tensor output_scale, Tensor output_offset)",
    "grouped_matmul_swiglu_quant_weight_nz_tensor_list(Tensor x, Tensor[] weight, Tensor[] weight_scale, "
    "Tensor x_scale, Tensor group_list, *, Tensor? bias=None, Tensor? offset=None, float swiglu_limit=0.0) "
    "-> (Tensor output, Tensor output_scale, Tensor output_offset)",
    "grouped_matmul_swiglu_quant_v2(Tensor x, Tensor[] weight, Tensor[] weight_scale, Tensor x_scale, "
    "Tensor group_list, Tensor? smooth_scale=None, Tensor[]? weight_assist_matrix=None, Tensor? bias=None, "
    "int? dequant_mode=0, int? dequant_dtype=0, int? quant_mode=0, int? quant_dtype=0, bool transpose_weight=False, "
    "int group_list_type=0, int[2] tuning_config=[], float swiglu_limit=0.0) -> (Tensor output, Tensor output_scale)",
    "npu_dequant_swiglu_quant(Tensor x, *, Tensor? weight_scale=None, Tensor? activation_scale=None, "
    "Tensor? bias=None, Tensor? quant_scale=None, Tensor? quant_offset=None, Tensor? group_index=None, "
    "bool activate_left=True, int quant_mode=0, int swiglu_mode=0, float clamp_limit=0.0, float glu_alpha=1.0, "
    "float glu_bias=0.0) -> (Tensor y, Tensor scale)",
]


# ------------------------------------------------------------------ CUDA (HIP) implementations
def _check_gating(x, bias_opt):
    # same argument checks, same messages as csrc/moe/moe_gating_top_k/moe_gating_top_k_torch_adpt.h:33-48
    if x.dim() != 2:
        raise RuntimeError("The x should be 2D")
    if x.dtype not in (torch.float16, torch.float32, torch.bfloat16):
        raise RuntimeError(f"float16、float32 or bfloat16 tensor expected but got a tensor with dtype: {x.dtype}")
    if bias_opt is not None:
        if bias_opt.dtype != x.dtype:
            raise RuntimeError("The dtype of x and bias should be same")
        if bias_opt.dim() != 1:
            raise RuntimeError("The bias should be 1D")
        if bias_opt.shape[0] != x.shape[1]:
            raise RuntimeError("The bias first dim should be same as x second dim")


def _moe_gating_top_k(x, k, k_group, group_count, group_select_mode, renorm, norm_type, out_flag,
                      routed_scaling_factor, eps, bias_opt=None):
    _check_gating(x, bias_opt)
    return kernels.gating_top_k(x, k, k_group, group_count, group_select_mode, renorm, norm_type, out_flag,
                                routed_scaling_factor, eps, bias_opt)


def _moe_gating_top_k_meta(x, k, k_group, group_count, group_select_mode, renorm, norm_type, out_flag,
                           routed_scaling_factor, eps, bias_opt=None):
    _check_gating(x, bias_opt)
    rows, experts = x.shape
    return (x.new_empty((rows, k)), x.new_empty((rows, k), dtype=torch.int32),
            x.new_empty((rows, experts), dtype=torch.float32))


def _reject_unsupported(bias, offset):
    if bias is not None and bias.numel() > 0:
        raise NotImplementedError("grouped_matmul_swiglu_quant: `bias` is only used by the int4-weight form")
    if offset is not None and offset.numel() > 0:
        raise NotImplementedError("grouped_matmul_swiglu_quant: `offset` (asymmetric weights) is not supported")


def _gmm_swiglu_quant_nz(x, weight, weight_scale, x_scale, group_list, *, bias=None, offset=None, swiglu_limit=0.0):
    if weight.dtype == torch.int32:
        # A8W4 form of the same op (eight int4 values per int32; is_a8w4 in
        # csrc/gmm/grouped_matmul_swiglu_quant_weight_nz_tensor_list/grouped_matmul_swiglu_quant_torch_adpt.h:27-31):
        # `bias` is the assist matrix of the int4 kernel
        if offset is not None and offset.numel() > 0:
            raise NotImplementedError("grouped_matmul_swiglu_quant: `offset` is not supported")
        out, out_scale = _gmm_swiglu_quant_v2(x, [weight], [weight_scale], x_scale, group_list,
                                              weight_assist_matrix=None if bias is None else [bias],
                                              group_list_type=0, swiglu_limit=swiglu_limit)
        return out, out_scale, x.new_empty((), dtype=torch.float32)
    if weight.dtype != torch.int8:
        raise NotImplementedError(f"grouped_matmul_swiglu_quant: weight dtype {weight.dtype} is not supported")
    _reject_unsupported(bias, offset)
    if x.dtype != torch.int8 or x.dim() != 2 or weight.dim() != 3:
        raise RuntimeError("grouped_matmul_swiglu_quant expects x int8 [M, K] and weight int8 [E, K, N]")
    k, n = weight.shape[1], weight.shape[2]
    if x.shape[1] != k:
        raise RuntimeError(f"x has K={x.shape[1]} but weight has K={k}")
    out, out_scale = kernels.gmm1_swiglu_quant(x, weight, weight_scale.to(torch.float32), x_scale, group_list, 0, n, k,
                                               swiglu_limit)
    return out, out_scale, x.new_empty((), dtype=torch.float32)


def _gmm_swiglu_quant_nz_meta(x, weight, weight_scale, x_scale, group_list, *, bias=None, offset=None,
                              swiglu_limit=0.0):
    m, n = x.shape[0], weight.shape[2]
    if x.dtype == torch.int8 and weight.dtype == torch.int32:
        n *= 8
    return (x.new_empty((m, n // 2), dtype=torch.int8), x.new_empty((m,), dtype=torch.float32),
            x.new_empty((), dtype=torch.float32))


def _gmm_swiglu_quant_nz_tensor_list(x, weight, weight_scale, x_scale, group_list, *, bias=None, offset=None,
                                     swiglu_limit=0.0):
    """Per-expert weight / scale tensors (each [K, N] tiled / [N]); the kernels follow a device table of
    their addresses, nothing is stacked or copied."""
    _reject_unsupported(bias, offset)
    if len(weight) != len(weight_scale) or len(weight) == 0:
        raise RuntimeError("weight and weight_scale must be lists of the same non-zero length")
    if len(weight) == 1 and weight[0].dim() == 3:
        out, out_scale, _ = _gmm_swiglu_quant_nz(x, weight[0], weight_scale[0], x_scale, group_list,
                                                  swiglu_limit=swiglu_limit)
    else:
        scales = [s if s.dtype == torch.float32 else s.to(torch.float32) for s in weight_scale]
        out, out_scale = kernels.gmm1_swiglu_quant_list(x, list(weight), scales, x_scale, group_list, 0, swiglu_limit)
    return out, out_scale, x.new_empty((x.shape[0],), dtype=torch.float32)


def _gmm_swiglu_quant_nz_tensor_list_meta(x, weight, weight_scale, x_scale, group_list, *, bias=None, offset=None,
                                          swiglu_limit=0.0):
    m, n = x.shape[0], weight[0].shape[1]
    return (x.new_empty((m, n // 2), dtype=torch.int8), x.new_empty((m,), dtype=torch.float32),
            x.new_empty((m,), dtype=torch.float32))


_W4_CORR: dict = {}


def _decode_scale(scale: torch.Tensor) -> torch.Tensor:
    """The reference widens fp32 scale bits into int64 (w4a8.py:320-325); undo that."""
    if scale.dtype == torch.int64:
        return scale.to(torch.int32).view(torch.float32)
    return scale.to(torch.float32)


def _gmm_swiglu_quant_v2(x, weight, weight_scale, x_scale, group_list, smooth_scale=None, weight_assist_matrix=None,
                         bias=None, dequant_mode=0, dequant_dtype=0, quant_mode=0, quant_dtype=0,
                         transpose_weight=False, group_list_type=0, tuning_config=(), swiglu_limit=0.0):
    """A8W4 form: ``x`` int8 [M, K]; ``weight`` = [tiled int4 storage from ``npu_format_cast_int4``, logical
    [E, K, N]]; ``weight_scale`` = [[E, N] per channel or [E, K/g, N] per group, fp32 or int64-encoded fp32];
    ``weight_assist_matrix`` = [[E, N] fp32]: the reference kernel computes (x - 8) . W . scale and adds this
    matrix, so the result here is x . W . scale + (assist - 8 * sum_k W * scale)."""
    if smooth_scale is not None or bias is not None or transpose_weight:
        raise NotImplementedError("grouped_matmul_swiglu_quant_v2: smooth_scale / bias / transpose_weight")
    if (dequant_mode or 0) != 0 or (quant_mode or 0) != 0 or (quant_dtype or 0) != 0:
        raise NotImplementedError("grouped_matmul_swiglu_quant_v2: only dequant_mode=0, quant_mode=0 (int8 out)")
    if len(weight) != 1 or len(weight_scale) != 1 or x.dtype != torch.int8:
        raise NotImplementedError("grouped_matmul_swiglu_quant_v2: one stacked int4 weight and one scale tensor")
    w, s = weight[0], _decode_scale(weight_scale[0])
    k = x.shape[1]
    n = s.shape[-1]
    e = w.shape[0]
    s = s.reshape(e, -1, n).contiguous()
    group = k // s.shape[1]
    w_bytes = w.contiguous().view(torch.uint8).reshape(e, -1)
    if w_bytes.shape[1] * 2 != n * k:
        raise RuntimeError("grouped_matmul_swiglu_quant_v2: weight holds a different number of int4 values than K*N")
    eff_bias = None
    if weight_assist_matrix is not None:
        # keyed on the caller's tensors and their version counters: an in-place swap of an expert's weights or
        # scales bumps the counter, so a stale correction is never reused (the decoded scale `s` may be a
        # temporary whose address means nothing)
        ws0 = weight_scale[0]
        key = (w.data_ptr(), w._version, ws0.data_ptr(), ws0._version, group)
        corr = _W4_CORR.get(key)
        if corr is None:
            if len(_W4_CORR) > 16:
                _W4_CORR.clear()  # safe: a correction is consumed inside the call that looks it up
            corr = kernels.w4_offset_correction(w_bytes, s, group, n, k)
            _W4_CORR[key] = corr
        eff_bias = (weight_assist_matrix[0].to(torch.float32).reshape(e, n) - corr).contiguous()
    return kernels.gmm1_swiglu_quant_w4(x, w_bytes, s, group, x_scale, group_list, group_list_type, n, k,
                                        bias=eff_bias, swiglu_limit=swiglu_limit)


def _gmm_swiglu_quant_v2_meta(x, weight, weight_scale, x_scale, group_list, smooth_scale=None,
                              weight_assist_matrix=None, bias=None, dequant_mode=0, dequant_dtype=0, quant_mode=0,
                              quant_dtype=0, transpose_weight=False, group_list_type=0, tuning_config=(),
                              swiglu_limit=0.0):
    m, n = x.shape[0], weight_scale[0].shape[-1]
    return x.new_empty((m, n // 2), dtype=torch.int8), x.new_empty((m,), dtype=torch.float32)


def _npu_dequant_swiglu_quant(x, *, weight_scale=None, activation_scale=None, bias=None, quant_scale=None,
                              quant_offset=None, group_index=None, activate_left=True, quant_mode=0, swiglu_mode=0,
                              clamp_limit=0.0, glu_alpha=1.0, glu_bias=0.0):
    """The reference runs two kernel families behind this op (csrc/moe/dequant_swiglu_quant/op_host/
    dequant_swiglu_quant_tiling.cpp:555-571): calls with ``group_index``, and calls with ``swiglu_mode=1`` on int32
    x, take the grouped class (``op_kernel/dequant_swiglu_quant.h``: clamp, ``glu_alpha``, ``glu_bias``, its own
    dynamic quantiser); the others the older per-mode kernels, which know neither clamp nor alpha."""
    if quant_mode not in (0, 1):
        raise NotImplementedError("npu_dequant_swiglu_quant: quant_mode must be 0 (static) or 1 (dynamic)")
    if swiglu_mode not in (0, 1):
        raise NotImplementedError("npu_dequant_swiglu_quant: swiglu_mode must be 0 or 1")
    if x.dtype != torch.int32 or weight_scale is None:
        raise RuntimeError("npu_dequant_swiglu_quant expects int32 x with weight_scale")
    if quant_mode == 1:
        for name, val in (("quant_scale", quant_scale), ("quant_offset", quant_offset)):
            if val is not None:
                raise NotImplementedError(f"npu_dequant_swiglu_quant: `{name}` (smooth scale) is not supported "
                                          "in quant_mode=1")
    elif quant_scale is None:
        raise RuntimeError("npu_dequant_swiglu_quant: quant_mode=0 needs quant_scale")
    if group_index is not None and group_index.dim() != 1:
        raise NotImplementedError("npu_dequant_swiglu_quant: group_index must hold one row count per group")
    if group_index is not None or swiglu_mode == 1 or bias is not None or activation_scale is None:
        return kernels.dequant_swiglu_quant_grouped(
            x, weight_scale, activation_scale, group_index, bias, activate_left, swiglu_mode, clamp_limit, glu_alpha,
            glu_bias, quant_mode, quant_scale, quant_offset)
    ws = weight_scale.to(torch.float32).reshape(-1)
    as_ = activation_scale.to(torch.float32).reshape(-1)
    if quant_mode == 0:
        # static: q = rint(y / quant_scale + quant_offset); the scale output carries nothing (zeros here)
        y = kernels.dequant_swiglu_quant_static(x, ws, as_, quant_scale, quant_offset, activate_left, 0.0)
        return y, torch.zeros(x.shape[:-1], dtype=torch.float32, device=x.device)
    return kernels.dequant_swiglu_quant(x, ws, as_, activate_left, 0.0)


def _npu_dequant_swiglu_quant_meta(x, *, weight_scale=None, activation_scale=None, bias=None, quant_scale=None,
                                   quant_offset=None, group_index=None, activate_left=True, quant_mode=0,
                                   swiglu_mode=0, clamp_limit=0.0, glu_alpha=1.0, glu_bias=0.0):
    return (x.new_empty(x.shape[:-1] + (x.shape[-1] // 2,), dtype=torch.int8),
            x.new_empty(x.shape[:-1], dtype=torch.float32))


_IMPLS = {
    "moe_gating_top_k": (_moe_gating_top_k, _moe_gating_top_k_meta),
    "grouped_matmul_swiglu_quant": (_gmm_swiglu_quant_nz, _gmm_swiglu_quant_nz_meta),
    "grouped_matmul_swiglu_quant_weight_nz": (_gmm_swiglu_quant_nz, _gmm_swiglu_quant_nz_meta),
    "grouped_matmul_swiglu_quant_weight_nz_tensor_list": (_gmm_swiglu_quant_nz_tensor_list,
                                                          _gmm_swiglu_quant_nz_tensor_list_meta),
    "grouped_matmul_swiglu_quant_v2": (_gmm_swiglu_quant_v2, _gmm_swiglu_quant_v2_meta),
    "npu_dequant_swiglu_quant": (_npu_dequant_swiglu_quant, _npu_dequant_swiglu_quant_meta),
}


def enable_custom_op() -> bool:
    """Register the ``_C_ascend`` operators once (counterpart of ``vllm_ascend.utils.enable_custom_op``,
    ``vllm_ascend/utils.py:397-445``).  Loading the kernel library is part of it: a missing
    ``libmoe355.so`` raises here."""
    global _LIB, _ENABLED
    if _ENABLED:
        return True
    from . import _lib

    _lib.load()
    lib = torch.library.Library("_C_ascend", "DEF")
    for schema in _SCHEMAS:
        lib.define(schema)
    for name, (impl, meta) in _IMPLS.items():
        lib.impl(name, impl, "CUDA")
        lib.impl(name, meta, "Meta")
    _LIB = lib
    _ENABLED = True
    return True
