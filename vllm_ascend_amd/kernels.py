"""Tensor-level launchers: allocate outputs and scratch with torch, pass raw device
pointers and the current HIP stream to the C ABI.  PyTorch is only the owner of
device memory and streams here; all arithmetic happens in ``libmoe355.so``.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import DT_BF16, DT_F16, DT_F32, GL_COUNT, GL_CUMSUM, W_EKN, W_ENK, check

_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """hipStream_t of torch's current stream on t's device (the raw handle: several times cheaper to look up than
    a torch.cuda.Stream object, and this runs once per kernel launch)."""
    if _raw_stream is not None:
        index = t.device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _dev(t: torch.Tensor, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got device {t.device}); this path has no CPU implementation")
    return t if t.is_contiguous() else t.contiguous()


def _dt(t: torch.Tensor, name: str) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"{name}: float16, float32 or bfloat16 tensor expected but got {t.dtype}") from None


def _half_dtype(dtype) -> torch.dtype:
    if dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"output dtype must be bfloat16 or float16, got {dtype}")
    return dtype


def _workspace(nbytes: int, device) -> torch.Tensor:
    # torch's caching allocator hands out 512-byte aligned blocks
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def dynamic_quant(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 / fp16 [..., H] -> (int8 [..., H], fp32 [...]) per-row absmax/127 quantisation."""
    x = _dev(x, "x")
    lib = _lib.load()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    check(lib.moe355_dynamic_quant(_ptr(x), _dt(x, "x"), rows, cols, _ptr(q), _ptr(s), _stream(x)),
          "moe355_dynamic_quant")
    return q, s


def router_gate(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """x [..., H] bf16 / fp16 / fp32, weight [E, H] fp32 -> fp32 logits [..., E] = x.float() @ weight.T (+ bias)."""
    x = _dev(x, "x")
    weight = _dev(weight, "weight")
    if weight.dtype != torch.float32:
        raise TypeError(f"weight: the router gate keeps its weight in float32, got {weight.dtype}")
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"x: float16, float32 or bfloat16 tensor expected but got {x.dtype}")
    E, H = weight.shape
    if x.shape[-1] != H:
        raise ValueError(f"x has {x.shape[-1]} features, the gate weight {H}")
    if bias is not None:
        bias = _dev(bias, "bias").to(torch.float32)
    T = x.numel() // H if H else 0
    lib = _lib.load()
    out = torch.empty((*x.shape[:-1], E), dtype=torch.float32, device=x.device)
    nbytes = lib.moe355_router_gate_workspace(T, H, E)
    ws = _workspace(nbytes, x.device) if nbytes else None
    check(lib.moe355_router_gate(_ptr(x), _dt(x, "x"), _ptr(weight), _ptr(bias), T, H, E, _ptr(out), _ptr(ws),
                                 ws.numel() if ws is not None else 0, _stream(x)), "moe355_router_gate")
    return out


def gating_top_k(x, k, k_group, group_count, group_select_mode, renorm, norm_type, out_flag, routed_scaling_factor,
                 eps, bias, alt_dtype=None):
    """-> (y, expert_idx, out[, y_alt]); ``alt_dtype`` asks for a second copy of y cast to that dtype."""
    x = _dev(x, "x")
    lib = _lib.load()
    rows, E = x.shape
    if bias is not None:
        bias = _dev(bias, "bias")
    y = torch.empty((rows, k), dtype=x.dtype, device=x.device)
    idx = torch.empty((rows, k), dtype=torch.int32, device=x.device)
    out = torch.empty((rows, E), dtype=torch.float32, device=x.device)
    y_alt = None
    if alt_dtype is not None and alt_dtype != x.dtype:
        y_alt = torch.empty((rows, k), dtype=alt_dtype, device=x.device)
    check(lib.moe355_gating_top_k(_ptr(x), _dt(x, "x"), _ptr(bias), rows, E, k, k_group, group_count,
                                  group_select_mode, renorm, norm_type, int(bool(out_flag)),
                                  float(routed_scaling_factor), float(eps), _ptr(y), _ptr(idx), _ptr(out),
                                  _ptr(y_alt), _DT[alt_dtype] if y_alt is not None else 0, _stream(x)),
          "moe355_gating_top_k")
    if alt_dtype is not None:
        return y, idx, out, (y if y_alt is None else y_alt)
    return y, idx, out


def init_routing(x, expert_idx, num_experts, quant_mode, tokens_num_type):
    x = _dev(x, "x")
    expert_idx = _dev(expert_idx, "expert_idx")
    if expert_idx.dtype != torch.int32:
        expert_idx = expert_idx.to(torch.int32)
    lib = _lib.load()
    T, k = expert_idx.shape
    H = x.shape[-1]
    R = T * k
    dev = x.device
    xs = torch.empty((R, H), dtype=torch.int8 if quant_mode == 1 else x.dtype, device=dev)
    row_idx = torch.empty((R,), dtype=torch.int32, device=dev)
    tokens = torch.empty((num_experts,), dtype=torch.int64, device=dev)
    scale = torch.empty((R,), dtype=torch.float32, device=dev) if quant_mode == 1 else None
    nbytes = lib.moe355_init_routing_workspace(T, k, num_experts)
    ws = _workspace(nbytes, dev)
    check(lib.moe355_init_routing(_ptr(x), _dt(x, "x"), T, H, _ptr(expert_idx), k, num_experts, quant_mode,
                                  tokens_num_type, _ptr(xs), _ptr(row_idx), _ptr(tokens), _ptr(scale), _ptr(ws),
                                  ws.numel(), _stream(x)), "moe355_init_routing")
    return xs, row_idx, tokens, scale


def init_routing_prequant(xq, x_scale, expert_idx, num_experts, tokens_num_type):
    """int8 activations [T, H] with their fp32 per-token scales [T]: rows and scales are moved to the
    expert-sorted order, nothing is quantised again.  -> (expanded_x int8 [R, H], expanded_row_idx, expert_tokens,
    expanded_scale [R])."""
    xq = _dev(xq, "x")
    x_scale = _dev(x_scale, "scale")
    expert_idx = _dev(expert_idx, "expert_idx")
    if xq.dtype != torch.int8:
        raise TypeError(f"x: pre-quantised activations must be int8, got {xq.dtype}")
    if x_scale.dtype != torch.float32:
        x_scale = x_scale.to(torch.float32)
    if expert_idx.dtype != torch.int32:
        expert_idx = expert_idx.to(torch.int32)
    T, k = expert_idx.shape
    H = xq.shape[-1]
    if xq.numel() != T * H or x_scale.numel() != T:
        raise ValueError(f"x {tuple(xq.shape)} / scale {tuple(x_scale.shape)} do not match {T} tokens")
    lib = _lib.load()
    R, dev = T * k, xq.device
    xs = torch.empty((R, H), dtype=torch.int8, device=dev)
    row_idx = torch.empty((R,), dtype=torch.int32, device=dev)
    tokens = torch.empty((num_experts,), dtype=torch.int64, device=dev)
    scale = torch.empty((R,), dtype=torch.float32, device=dev)
    ws = _workspace(lib.moe355_init_routing_workspace(T, k, num_experts), dev)
    check(lib.moe355_init_routing_prequant(_ptr(xq), _ptr(x_scale), T, H, _ptr(expert_idx), k, num_experts,
                                           tokens_num_type, _ptr(xs), _ptr(row_idx), _ptr(tokens), _ptr(scale),
                                           _ptr(ws), ws.numel(), _stream(xq)), "moe355_init_routing_prequant")
    return xs, row_idx, tokens, scale


def route_map(expert_idx, num_experts, tokens_num_type):
    """The maps of the permutation, nothing moved: (expanded_row_idx [T*k] pair -> sorted row, row_token [T*k]
    sorted row -> token, expert_tokens [E])."""
    expert_idx = _dev(expert_idx, "expert_idx")
    if expert_idx.dtype != torch.int32:
        expert_idx = expert_idx.to(torch.int32)
    lib = _lib.load()
    T, k = expert_idx.shape
    dev = expert_idx.device
    row_idx = torch.empty((T * k,), dtype=torch.int32, device=dev)
    row_token = torch.empty((T * k,), dtype=torch.int32, device=dev)
    tokens = torch.empty((num_experts,), dtype=torch.int64, device=dev)
    nbytes = lib.moe355_init_routing_workspace(T, k, num_experts)
    ws = _workspace(nbytes, dev)
    check(lib.moe355_route_map(_ptr(expert_idx), T, k, num_experts, tokens_num_type, _ptr(row_idx), _ptr(row_token),
                               _ptr(tokens), _ptr(ws), nbytes, _stream(expert_idx)), "moe355_route_map")
    return row_idx, row_token, tokens


def route_quant_small_supported(num_tokens: int, top_k: int, num_experts: int) -> bool:
    return bool(_lib.load().moe355_route_quant_small_supported(num_tokens, top_k, num_experts))


def route_quant_small(x, logits, k, k_group, group_count, group_select_mode, renorm, norm_type,
                      routed_scaling_factor, eps, bias, sync_counter=None):
    """Gating and dispatch of a small batch in one launch.  -> (topk_weights [T, k] in x's dtype, topk_ids,
    xq int8 [T, H] in TOKEN order, x_scale [T], expanded_row_idx [T*k], row_token [T*k], expert_tokens [E] counts).
    sync_counter: a one-element int32 GPU tensor that is zero between calls
    (a layer keeps one); without it a zeroed one is made for this call (one more small launch)."""
    x = _dev(x, "x")
    logits = _dev(logits, "router_logits")
    if bias is not None:
        bias = _dev(bias, "bias")
        if bias.dtype != logits.dtype:
            raise RuntimeError("The dtype of x and bias should be same")
    lib = _lib.load()
    T, E = logits.shape
    H = x.shape[-1]
    if x.numel() != T * H:
        raise ValueError(f"hidden states {tuple(x.shape)} do not match {T} rows of router logits")
    dev = x.device
    tw = torch.empty((T, k), dtype=x.dtype, device=dev)
    ids = torch.empty((T, k), dtype=torch.int32, device=dev)
    xq = torch.empty((T, H), dtype=torch.int8, device=dev)
    xs = torch.empty((T,), dtype=torch.float32, device=dev)
    dst = torch.empty((T * k,), dtype=torch.int32, device=dev)
    row_token = torch.empty((T * k,), dtype=torch.int32, device=dev)
    tokens = torch.empty((E,), dtype=torch.int64, device=dev)
    if sync_counter is None:
        sync_counter = torch.zeros((1,), dtype=torch.int32, device=dev)
    elif sync_counter.dtype != torch.int32 or sync_counter.numel() != 1 or sync_counter.device != dev:
        raise ValueError("sync_counter must be a one-element int32 tensor on the device of x")
    check(lib.moe355_route_quant_small(_ptr(x), _dt(x, "x"), _ptr(logits), _dt(logits, "router_logits"), _ptr(bias),
                                       T, H, E, k, k_group, group_count, group_select_mode, int(renorm), norm_type,
                                       float(routed_scaling_factor), float(eps), 1, _ptr(tw), _ptr(ids), _ptr(xq),
                                       _ptr(xs), _ptr(dst), _ptr(row_token), _ptr(tokens), _ptr(sync_counter),
                                       _stream(x)), "moe355_route_quant_small")
    return tw, ids, xq, xs, dst, row_token, tokens


def gate_quant_supported(num_tokens: int, top_k: int, num_experts: int) -> bool:
    return bool(_lib.load().moe355_gate_quant_supported(num_tokens, top_k, num_experts))


def gate_quant(x, logits, k, k_group, group_count, group_select_mode, renorm, norm_type, routed_scaling_factor, eps,
               bias):
    """Gating and token quantisation in one launch, any number of tokens.  -> (topk_weights [T, k] in x's dtype,
    topk_ids [T, k] int32, xq int8 [T, H] in token order, x_scale [T])."""
    x = _dev(x, "x")
    logits = _dev(logits, "router_logits")
    if bias is not None:
        bias = _dev(bias, "bias")
        if bias.dtype != logits.dtype:
            raise RuntimeError("The dtype of x and bias should be same")
    lib = _lib.load()
    T, E = logits.shape
    H = x.shape[-1]
    if x.numel() != T * H:
        raise ValueError(f"hidden states {tuple(x.shape)} do not match {T} rows of router logits")
    dev = x.device
    tw = torch.empty((T, k), dtype=x.dtype, device=dev)
    ids = torch.empty((T, k), dtype=torch.int32, device=dev)
    xq = torch.empty((T, H), dtype=torch.int8, device=dev)
    xs = torch.empty((T,), dtype=torch.float32, device=dev)
    check(lib.moe355_gate_quant(_ptr(x), _dt(x, "x"), _ptr(logits), _dt(logits, "router_logits"), _ptr(bias), T, H, E,
                                k, k_group, group_count, group_select_mode, int(renorm), norm_type,
                                float(routed_scaling_factor), float(eps), _ptr(tw), _ptr(ids), _ptr(xq), _ptr(xs),
                                _stream(x)), "moe355_gate_quant")
    return tw, ids, xq, xs


def gmm1_swiglu_quant_gather(xq, x_scale, row_token, weight_nz, weight_scale, group_list, group_list_type, n, k,
                             swiglu_limit=0.0):
    """gate_up GEMM + SwiGLU + re-quantisation on rows that are read through ``row_token`` from activations kept
    in token order (route_quant_small).  -> (int8 [R, n/2], fp32 [R]) in the expert-sorted order."""
    lib = _lib.load()
    rows = row_token.numel()
    E = weight_nz.shape[0]
    if row_token.dtype != torch.int32:
        raise TypeError(f"row_token must be int32, got {row_token.dtype}")
    _check_gmm_operands("gmm1_swiglu_quant_gather", xq, xq.shape[0], k, n, E, group_list, x_scale, "x_scale",
                        weight_nz, E * n * k, weight_scale, E * n)
    xq = _dev(xq, "x")
    dev = xq.device
    out = torch.empty((rows, n // 2), dtype=torch.int8, device=dev)
    out_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    ws = _workspace(lib.moe355_gmm1_swiglu_quant_workspace(rows, n, k, E), dev)
    check(lib.moe355_gmm1_swiglu_quant_gather(_ptr(xq), _ptr(_dev(x_scale, "x_scale")),
                                              _ptr(_dev(row_token, "row_token")), _ptr(_dev(weight_nz, "weight")),
                                              _ptr(_dev(weight_scale, "scale")), _ptr(_gl(group_list)),
                                              _gl_type(group_list_type), rows, k, n, E, float(swiglu_limit),
                                              _ptr(out), _ptr(out_scale), _ptr(ws), ws.numel(), _stream(xq)),
          "moe355_gmm1_swiglu_quant_gather")
    return out, out_scale


def format_cast_nz(w: torch.Tensor, layout: int) -> torch.Tensor:
    """int8 [E, N, K] (layout W_ENK) or [E, K, N] (W_EKN) -> same shape, MFMA-tiled storage."""
    w = _dev(w, "weight")
    if w.dtype != torch.int8 or w.dim() != 3:
        raise TypeError("format_cast_nz expects a 3-D int8 weight")
    lib = _lib.load()
    E = w.shape[0]
    n, k = (w.shape[1], w.shape[2]) if layout == W_ENK else (w.shape[2], w.shape[1])
    out = torch.empty_like(w)
    check(lib.moe355_format_cast_nz(_ptr(w), layout, E, n, k, _ptr(out), _stream(w)), "moe355_format_cast_nz")
    return out


def _gl_type(group_list_type: int) -> int:
    if group_list_type == 0:
        return GL_CUMSUM
    if group_list_type == 1:
        return GL_COUNT
    raise NotImplementedError(f"group_list_type {group_list_type} is not supported on this path")


def _gl(group_list: torch.Tensor) -> torch.Tensor:
    group_list = _dev(group_list, "group_list")
    return group_list if group_list.dtype == torch.int64 else group_list.to(torch.int64)


def _check_gmm_operands(op, x, rows, k, n, E, group_list, row_scale=None, row_scale_name="x_scale", weight=None,
                        weight_numel=None, channel_scale=None, channel_scale_numel=None):
    """Host-side argument checks of the grouped-GEMM launchers: the C ABI takes raw pointers, so a tensor of the
    wrong dtype or length would be read out of bounds on the device instead of raising."""
    if x.dtype != torch.int8:
        raise TypeError(f"{op}: x must be int8, got {x.dtype}")
    if x.dim() != 2 or x.shape[1] != k:
        raise ValueError(f"{op}: x must be [rows, K = {k}], got {tuple(x.shape)}")
    if group_list.dim() != 1 or group_list.numel() != E:
        raise ValueError(f"{op}: group_list must hold one entry per expert ({E}), got {tuple(group_list.shape)}")
    if row_scale is not None:
        if row_scale.dtype != torch.float32:
            raise TypeError(f"{op}: {row_scale_name} must be float32, got {row_scale.dtype}")
        if row_scale.numel() != rows:
            raise ValueError(f"{op}: {row_scale_name} must hold one scale per row ({rows}), got {row_scale.numel()}")
    if weight is not None:
        if weight.dtype not in (torch.int8, torch.uint8):
            raise TypeError(f"{op}: weight must be int8 tiled storage, got {weight.dtype}")
        if weight.numel() != weight_numel:
            raise ValueError(f"{op}: weight holds {weight.numel()} bytes, E x N x K needs {weight_numel}")
    if channel_scale is not None:
        if channel_scale.dtype != torch.float32:
            raise TypeError(f"{op}: the weight scale must be float32, got {channel_scale.dtype} "
                            "(convert once after loading)")
        if channel_scale.numel() != channel_scale_numel:
            raise ValueError(f"{op}: the weight scale holds {channel_scale.numel()} values, expected "
                             f"{channel_scale_numel}")


def gmm1_swiglu_quant(x, weight_nz, weight_scale, x_scale, group_list, group_list_type, n, k, swiglu_limit=0.0,
                      out=None, out_scale=None):
    lib = _lib.load()
    rows = x.shape[0]
    E = weight_nz.shape[0]
    dev = x.device
    _check_gmm_operands("gmm1_swiglu_quant", x, rows, k, n, E, group_list, x_scale, "x_scale", weight_nz, E * n * k,
                        weight_scale, E * n)
    x = _dev(x, "x")
    if out is None:
        out = torch.empty((rows, n // 2), dtype=torch.int8, device=dev)
    if out_scale is None:
        out_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    ws = _workspace(lib.moe355_gmm1_swiglu_quant_workspace(rows, n, k, E), dev)
    check(lib.moe355_gmm1_swiglu_quant(_ptr(x), _ptr(_dev(weight_nz, "weight")), _ptr(_dev(weight_scale, "scale")),
                                       _ptr(_dev(x_scale, "x_scale")), _ptr(_gl(group_list)),
                                       _gl_type(group_list_type), rows, k, n, E, float(swiglu_limit), _ptr(out),
                                       _ptr(out_scale), _ptr(ws), ws.numel(), _stream(x)),
          "moe355_gmm1_swiglu_quant")
    return out, out_scale


def gmm2_dequant(x, weight_nz, scale, per_token_scale, group_list, group_list_type, n, k, out_dtype=torch.bfloat16):
    lib = _lib.load()
    rows = x.shape[0]
    E = weight_nz.shape[0]
    _check_gmm_operands("gmm2_dequant", x, rows, k, n, E, group_list, per_token_scale, "per_token_scale", weight_nz,
                        E * n * k, scale, E * n)
    x = _dev(x, "x")
    out = torch.empty((rows, n), dtype=_half_dtype(out_dtype), device=x.device)
    ws = _workspace(lib.moe355_gmm2_dequant_workspace(rows, n, k, E), x.device)
    check(lib.moe355_gmm2_dequant(_ptr(x), _ptr(_dev(weight_nz, "weight")), _ptr(_dev(scale, "scale")),
                                  _ptr(_dev(per_token_scale, "per_token_scale")), _ptr(_gl(group_list)),
                                  _gl_type(group_list_type), rows, k, n, E, _ptr(out), _dt(out, "out"), _ptr(ws),
                                  ws.numel(), _stream(x)), "moe355_gmm2_dequant")
    return out


def gmm_i32(x, weight_nz, group_list, group_list_type, n, k, groups_cover_all_rows=False):
    """Raw int32 accumulators of the grouped product (rows outside every group are zero; a caller whose
    groups cover every row says so and saves the fill)."""
    lib = _lib.load()
    rows = x.shape[0]
    E = weight_nz.shape[0]
    _check_gmm_operands("gmm_i32", x, rows, k, n, E, group_list, weight=weight_nz, weight_numel=E * n * k)
    x = _dev(x, "x")
    acc = (torch.empty if groups_cover_all_rows else torch.zeros)((rows, n), dtype=torch.int32, device=x.device)
    ws = _workspace(lib.moe355_gmm_i32_workspace(rows, n, k, E), x.device)
    check(lib.moe355_gmm_i32(_ptr(x), _ptr(_dev(weight_nz, "weight")), _ptr(_gl(group_list)),
                             _gl_type(group_list_type), rows, k, n, E, _ptr(acc), _ptr(ws), ws.numel(), _stream(x)),
          "moe355_gmm_i32")
    return acc


def dequant_swiglu_quant(x, weight_scale, activation_scale, activate_left=True, clamp_limit=0.0):
    x = _dev(x, "x")
    lib = _lib.load()
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    y = torch.empty(x.shape[:-1] + (n // 2,), dtype=torch.int8, device=x.device)
    s = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    check(lib.moe355_dequant_swiglu_quant(_ptr(x), _ptr(_dev(weight_scale, "weight_scale")),
                                          _ptr(_dev(activation_scale, "activation_scale")), rows, n,
                                          int(bool(activate_left)), float(clamp_limit), _ptr(y), _ptr(s), _stream(x)),
          "moe355_dequant_swiglu_quant")
    return y, s


def dequant_swiglu_quant_grouped(x, weight_scale, activation_scale=None, group_index=None, bias=None,
                                 activate_left=True, swiglu_mode=0, clamp_limit=0.0, glu_alpha=1.0, glu_bias=0.0,
                                 quant_mode=1, quant_scale=None, quant_offset=None):
    """The general form of npu_dequant_swiglu_quant: weight_scale [G, n] (or [n]), group_index [G] row counts,
    bias [G, n] int32 or floating, swiglu_mode 1 with clamp_limit / glu_alpha / glu_bias, quant_mode 0 with
    quant_scale [G] or [G, n/2].  -> (y int8, scale fp32; zeros in quant_mode 0)."""
    x = _dev(x, "x")
    if x.dtype != torch.int32:
        raise TypeError(f"x: int32 tensor expected but got {x.dtype}")
    lib = _lib.load()
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    ws = _dev(weight_scale, "weight_scale").to(torch.float32).contiguous()
    if ws.numel() % n:
        raise ValueError(f"weight_scale has {ws.numel()} elements, x {n} columns")
    groups = ws.numel() // n
    gi = None
    if group_index is not None:
        gi = _dev(group_index, "group_index").to(torch.int64).contiguous()
        if gi.dim() != 1 or gi.numel() != groups:
            raise ValueError(f"group_index must hold one row count per group of weight_scale ({groups}), "
                             f"got shape {tuple(gi.shape)}")
    elif groups != 1:
        raise ValueError("weight_scale with several groups needs group_index")
    a = None
    if activation_scale is not None:
        a = _dev(activation_scale, "activation_scale").to(torch.float32).reshape(-1).contiguous()
        if a.numel() != rows:
            raise ValueError(f"activation_scale has {a.numel()} elements for {rows} rows")
    kind = 0
    if bias is not None:
        bias = _dev(bias, "bias")
        kind = 1 if bias.dtype == torch.int32 else 2
        bias = (bias if kind == 1 else bias.to(torch.float32)).contiguous()
        if bias.numel() != groups * n:
            raise ValueError(f"bias must have {groups} x {n} elements, got {bias.numel()}")
    qs = qo = None
    if quant_mode == 0:
        if quant_scale is None:
            raise RuntimeError("quant_mode=0 needs quant_scale")
        qs = _dev(quant_scale, "quant_scale").to(torch.float32).reshape(-1).contiguous()
        if quant_offset is not None:
            qo = _dev(quant_offset, "quant_offset").to(torch.float32).reshape(-1).contiguous()
            if qo.numel() != qs.numel():
                raise ValueError("quant_offset must have as many elements as quant_scale")
    y = torch.empty(x.shape[:-1] + (n // 2,), dtype=torch.int8, device=x.device)
    s = (torch.empty if quant_mode == 1 else torch.zeros)(x.shape[:-1], dtype=torch.float32, device=x.device)
    check(lib.moe355_dequant_swiglu_quant_grouped(
        _ptr(x), _ptr(ws), _ptr(a), _ptr(bias), kind, _ptr(gi), groups, rows, n, int(bool(activate_left)),
        int(swiglu_mode), float(clamp_limit), float(glu_alpha), float(glu_bias), int(quant_mode), _ptr(qs),
        qs.numel() if qs is not None else 0, _ptr(qo), _ptr(y), _ptr(s), _stream(x)),
        "moe355_dequant_swiglu_quant_grouped")
    return y, s


def dequant_swiglu_quant_static(x, weight_scale, activation_scale, quant_scale, quant_offset=None,
                                activate_left=True, clamp_limit=0.0):
    """quant_mode 0 of npu_dequant_swiglu_quant: one scale (and offset) per output channel or per tensor."""
    x = _dev(x, "x")
    lib = _lib.load()
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    quant_scale = _dev(quant_scale, "quant_scale").to(torch.float32).reshape(-1)
    if quant_offset is not None:
        quant_offset = _dev(quant_offset, "quant_offset").to(torch.float32).reshape(-1)
        if quant_offset.numel() != quant_scale.numel():
            raise ValueError("quant_offset must have as many elements as quant_scale")
    y = torch.empty(x.shape[:-1] + (n // 2,), dtype=torch.int8, device=x.device)
    check(lib.moe355_dequant_swiglu_quant_static(_ptr(x), _ptr(_dev(weight_scale, "weight_scale")),
                                                 _ptr(_dev(activation_scale, "activation_scale")), _ptr(quant_scale),
                                                 quant_scale.numel(), _ptr(quant_offset), rows, n,
                                                 int(bool(activate_left)), float(clamp_limit), _ptr(y), _stream(x)),
          "moe355_dequant_swiglu_quant_static")
    return y


ACTIVATIONS = {"gelu": 1, "gelu_tanh": 2, "swiglustep": 3, "swigluoai": 4, "swigluoai_uninterleave": 4}


def act_mul_quant(h, activation: str, limit=0.0, alpha=1.0, beta=0.0, group_list=None, group_list_type=1):
    """activation(gate) * up on a 16-bit [rows, 2I] tensor (gate first) + per-row dynamic int8 quantisation."""
    h = _dev(h, "hidden_states")
    lib = _lib.load()
    rows, n = h.shape
    q = torch.empty((rows, n // 2), dtype=torch.int8, device=h.device)
    s = torch.empty((rows,), dtype=torch.float32, device=h.device)
    E = 0
    if group_list is not None:
        group_list = _dev(group_list, "group_list")
        if group_list.dtype != torch.int64:
            group_list = group_list.to(torch.int64)
        E = group_list.numel()
    check(lib.moe355_act_mul_quant(_ptr(h), _dt(h, "hidden_states"), _ptr(group_list), int(group_list_type), E, rows, n,
                                   ACTIVATIONS[activation], float(limit), float(alpha), float(beta), _ptr(q), _ptr(s),
                                   _stream(h)), "moe355_act_mul_quant")
    return q, s


def token_unpermute(permuted, sorted_indices, probs, residual=None):
    permuted = _dev(permuted, "permuted_tokens")
    sorted_indices = _dev(sorted_indices, "sorted_indices")
    if sorted_indices.dtype != torch.int32:
        sorted_indices = sorted_indices.to(torch.int32)
    lib = _lib.load()
    R, H = permuted.shape
    if probs is not None:
        probs = _dev(probs, "probs")
        if probs.dtype != permuted.dtype:
            probs = probs.to(permuted.dtype)
        T, k = probs.shape
    else:
        T, k = sorted_indices.numel(), 1
    if residual is not None:
        residual = _dev(residual, "residual")
        if residual.dtype != permuted.dtype or tuple(residual.shape) != (T, H):
            raise ValueError(f"residual must be {permuted.dtype} of shape {(T, H)}, got {residual.dtype} "
                             f"{tuple(residual.shape)}")
    out = torch.empty((T, H), dtype=permuted.dtype, device=permuted.device)
    check(lib.moe355_token_unpermute(_ptr(permuted), _dt(permuted, "permuted_tokens"), _ptr(sorted_indices),
                                     _ptr(probs), T, k, H, R, _ptr(residual), _ptr(out), _stream(permuted)),
          "moe355_token_unpermute")
    return out


# ------------------------------------------------------------------ pair order (decode batches)
def gmm_pairs_supported(num_tokens: int, top_k: int, n: int, k: int) -> bool:
    return bool(_lib.load().moe355_gmm_pairs_supported(num_tokens, top_k, n, k))


def _check_pair_operands(name, x, x_rows, k, scale_rows, row_scale, topk_ids, weight_nz, n, ch_scale):
    for t, what in ((x, "x"), (row_scale, "row scale"), (topk_ids, "topk_ids"), (weight_nz, "weight"),
                    (ch_scale, "scale")):
        _dev(t, what)
    E = weight_nz.shape[0]
    if x.dtype != torch.int8 or x.numel() != x_rows * k:
        raise ValueError(f"{name}: x must be int8 with {x_rows} rows of {k} values, got {x.dtype} {tuple(x.shape)}")
    if row_scale.dtype != torch.float32 or row_scale.numel() != scale_rows:
        raise ValueError(f"{name}: {scale_rows} float32 row scales expected, got {row_scale.dtype} "
                         f"{tuple(row_scale.shape)}")
    if topk_ids.dtype != torch.int32:
        raise TypeError(f"{name}: topk_ids must be int32, got {topk_ids.dtype}")
    if weight_nz.dtype != torch.int8 or weight_nz.numel() != E * n * k:
        raise ValueError(f"{name}: weight must be int8 with E x N x K = {E * n * k} values")
    if ch_scale.dtype != torch.float32 or ch_scale.numel() != E * n:
        raise ValueError(f"{name}: scale must be float32 with E x N = {E * n} values")
    return E


def gmm1_swiglu_quant_pairs(xq, x_scale, topk_ids, weight_nz, weight_scale, n, k, swiglu_limit=0.0):
    """gate_up GEMM + SwiGLU + re-quantisation in pair order: xq int8 [T, K] and x_scale [T] in token order,
    topk_ids [T, top_k] -> (int8 [T*top_k, n/2], fp32 [T*top_k]); row t*top_k + s belongs to slot s of token t."""
    lib = _lib.load()
    T, top_k = topk_ids.shape
    E = _check_pair_operands("gmm1_swiglu_quant_pairs", xq, T, k, T, x_scale, topk_ids, weight_nz, n, weight_scale)
    dev = xq.device
    out = torch.empty((T * top_k, n // 2), dtype=torch.int8, device=dev)
    out_scale = torch.empty((T * top_k,), dtype=torch.float32, device=dev)
    ws = _workspace(lib.moe355_gmm1_swiglu_quant_pairs_workspace(T, top_k, n), dev)
    check(lib.moe355_gmm1_swiglu_quant_pairs(_ptr(xq), _ptr(x_scale), _ptr(topk_ids), T, top_k, _ptr(weight_nz),
                                             _ptr(weight_scale), k, n, E, float(swiglu_limit), _ptr(out),
                                             _ptr(out_scale), _ptr(ws), ws.numel(), _stream(xq)),
          "moe355_gmm1_swiglu_quant_pairs")
    return out, out_scale


def gmm2_dequant_pairs(x, weight_nz, scale, per_token_scale, topk_ids, n, k, out_dtype=torch.bfloat16):
    """down GEMM + dequant in pair order: x int8 [T*top_k, K], per_token_scale [T*top_k] -> [T*top_k, n]."""
    lib = _lib.load()
    T, top_k = topk_ids.shape
    E = _check_pair_operands("gmm2_dequant_pairs", x, T * top_k, k, T * top_k, per_token_scale, topk_ids, weight_nz, n,
                             scale)
    out = torch.empty((T * top_k, n), dtype=_half_dtype(out_dtype), device=x.device)
    check(lib.moe355_gmm2_dequant_pairs(_ptr(x), _ptr(weight_nz), _ptr(scale), _ptr(per_token_scale), _ptr(topk_ids),
                                        T, top_k, k, n, E, _ptr(out), _dt(out, "out"), _stream(x)),
          "moe355_gmm2_dequant_pairs")
    return out


def gmm2_requant_pairs_supported(num_tokens: int, top_k: int, n: int, k: int, num_experts: int) -> bool:
    return bool(_lib.load().moe355_gmm2_requant_pairs_supported(num_tokens, top_k, n, k, num_experts))


def gmm1_swiglu_pairs(xq, x_scale, topk_ids, weight_nz, weight_scale, n, k, swiglu_limit=0.0):
    """gate_up GEMM + SwiGLU in pair order, no re-quantisation: -> fp32 [T*top_k, n/2]."""
    lib = _lib.load()
    T, top_k = topk_ids.shape
    E = _check_pair_operands("gmm1_swiglu_pairs", xq, T, k, T, x_scale, topk_ids, weight_nz, n, weight_scale)
    y = torch.empty((T * top_k, n // 2), dtype=torch.float32, device=xq.device)
    check(lib.moe355_gmm1_swiglu_pairs(_ptr(xq), _ptr(x_scale), _ptr(topk_ids), T, top_k, _ptr(weight_nz),
                                       _ptr(weight_scale), k, n, E, float(swiglu_limit), _ptr(y), _stream(xq)),
          "moe355_gmm1_swiglu_pairs")
    return y


def gmm2_requant_dequant_pairs(y, weight_nz, scale, topk_ids, n, k, out_dtype=torch.bfloat16):
    """Re-quantisation + down GEMM + dequant in pair order: y fp32 [T*top_k, K] -> [T*top_k, n]."""
    lib = _lib.load()
    y = _dev(y, "y")
    T, top_k = topk_ids.shape
    E = weight_nz.shape[0]
    if y.dtype != torch.float32 or tuple(y.shape) != (T * top_k, k):
        raise ValueError(f"gmm2_requant_dequant_pairs: y must be float32 {(T * top_k, k)}, got {y.dtype} "
                         f"{tuple(y.shape)}")
    if _dev(topk_ids, "topk_ids").dtype != torch.int32:
        raise TypeError(f"gmm2_requant_dequant_pairs: topk_ids must be int32, got {topk_ids.dtype}")
    if _dev(weight_nz, "weight").dtype != torch.int8 or weight_nz.numel() != E * n * k:
        raise ValueError(f"gmm2_requant_dequant_pairs: weight must be int8 with E x N x K = {E * n * k} values")
    if _dev(scale, "scale").dtype != torch.float32 or scale.numel() != E * n:
        raise ValueError(f"gmm2_requant_dequant_pairs: scale must be float32 with E x N = {E * n} values")
    out = torch.empty((T * top_k, n), dtype=_half_dtype(out_dtype), device=y.device)
    check(lib.moe355_gmm2_requant_dequant_pairs(_ptr(y), _ptr(weight_nz), _ptr(scale), _ptr(topk_ids), T, top_k, k, n,
                                                E, _ptr(out), _dt(out, "out"), _stream(y)),
          "moe355_gmm2_requant_dequant_pairs")
    return out


def token_unpermute_pairs(rows, probs, topk_ids, num_experts, residual=None):
    """Weighted sum of the top_k rows of every token, rows in pair order.  -> (out [T, H], expert_tokens [E] int64
    counts of the pairs of every expert)."""
    rows = _dev(rows, "rows")
    probs = _dev(probs, "probs")
    topk_ids = _dev(topk_ids, "topk_ids")
    if topk_ids.dtype != torch.int32:
        raise TypeError(f"topk_ids must be int32, got {topk_ids.dtype}")
    if probs.dtype != rows.dtype:
        probs = probs.to(rows.dtype)
    T, k = probs.shape
    H = rows.shape[1]
    if rows.shape[0] != T * k or tuple(topk_ids.shape) != (T, k):
        raise ValueError(f"rows {tuple(rows.shape)} / topk_ids {tuple(topk_ids.shape)} do not match {T} x {k} pairs")
    if residual is not None:
        residual = _dev(residual, "residual")
        if residual.dtype != rows.dtype or tuple(residual.shape) != (T, H):
            raise ValueError(f"residual must be {rows.dtype} of shape {(T, H)}, got {residual.dtype} "
                             f"{tuple(residual.shape)}")
    lib = _lib.load()
    out = torch.empty((T, H), dtype=rows.dtype, device=rows.device)
    tokens = torch.empty((num_experts,), dtype=torch.int64, device=rows.device)
    check(lib.moe355_token_unpermute_pairs(_ptr(rows), _dt(rows, "rows"), _ptr(probs), _ptr(topk_ids), T, k, H,
                                           num_experts, _ptr(residual), _ptr(out), _ptr(tokens), _stream(rows)),
          "moe355_token_unpermute_pairs")
    return out, tokens


# ------------------------------------------------------------------ W4A8 (int4 weights)
def format_cast_nz_int4(w: torch.Tensor, source: int, n: int, k: int) -> torch.Tensor:
    """source 0: int8 [E, N, K] with one int4 value per byte; source 1: packed bytes [E, K, N/2]
    (low nibble = even channel).  Returns the tiled int4 storage as uint8 [E, N*K/2]."""
    w = _dev(w, "weight")
    lib = _lib.load()
    E = w.shape[0]
    out = torch.empty((E, n * k // 2), dtype=torch.uint8, device=w.device)
    check(lib.moe355_format_cast_nz_int4(_ptr(w), source, E, n, k, _ptr(out), _stream(w)),
          "moe355_format_cast_nz_int4")
    return out


def gmm1_swiglu_quant_w4(x, weight_nz4, weight_scale, group_size, x_scale, group_list, group_list_type, n, k,
                         bias=None, swiglu_limit=0.0):
    lib = _lib.load()
    rows = x.shape[0]
    E = weight_nz4.shape[0]
    dev = x.device
    groups = k // group_size if group_size else 1
    _check_gmm_operands("gmm1_swiglu_quant_w4", x, rows, k, n, E, group_list, x_scale, "x_scale", weight_nz4,
                        E * n * k // 2, weight_scale, E * groups * n)
    x = _dev(x, "x")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != E * n or not bias.is_cuda):
        raise ValueError(f"gmm1_swiglu_quant_w4: bias must be a float32 GPU tensor of E x N = {E * n} values")
    out = torch.empty((rows, n // 2), dtype=torch.int8, device=dev)
    out_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    ws = _workspace(rows * (n // 2) * 4 + 256, dev)
    check(lib.moe355_gmm1_swiglu_quant_w4(_ptr(x), _ptr(_dev(weight_nz4, "weight")),
                                          _ptr(_dev(weight_scale, "weight_scale")), group_size,
                                          _ptr(bias), _ptr(_dev(x_scale, "x_scale")), _ptr(_gl(group_list)),
                                          _gl_type(group_list_type), rows, k, n, E, float(swiglu_limit), _ptr(out),
                                          _ptr(out_scale), _ptr(ws), ws.numel(), _stream(x)),
          "moe355_gmm1_swiglu_quant_w4")
    return out, out_scale


def gmm1_swiglu_quant_w4_gather(xq, x_scale, row_token, weight_nz4, weight_scale, group_size, group_list,
                                group_list_type, n, k, bias=None, swiglu_limit=0.0):
    """The W4A8 gate_up op on token rows that were quantised once and are read through the row -> token map."""
    lib = _lib.load()
    rows = row_token.shape[0]
    T = xq.shape[0]
    E = weight_nz4.shape[0]
    dev = xq.device
    groups = k // group_size if group_size else 1
    _check_gmm_operands("gmm1_swiglu_quant_w4_gather", xq, T, k, n, E, group_list, x_scale, "x_scale", weight_nz4,
                        E * n * k // 2, weight_scale, E * groups * n)
    xq = _dev(xq, "x")
    row_token = _dev(row_token, "row_token")
    if row_token.dtype != torch.int32:
        raise ValueError("gmm1_swiglu_quant_w4_gather: row_token must be int32")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != E * n or not bias.is_cuda):
        raise ValueError(f"gmm1_swiglu_quant_w4_gather: bias must be a float32 GPU tensor of E x N = {E * n} values")
    out = torch.empty((rows, n // 2), dtype=torch.int8, device=dev)
    out_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    ws = _workspace(rows * (n // 2) * 4 + 256, dev)
    check(lib.moe355_gmm1_swiglu_quant_w4_gather(_ptr(xq), _ptr(_dev(x_scale, "x_scale")), _ptr(row_token),
                                                 _ptr(_dev(weight_nz4, "weight")),
                                                 _ptr(_dev(weight_scale, "weight_scale")), group_size, _ptr(bias),
                                                 _ptr(_gl(group_list)), _gl_type(group_list_type), rows, k, n, E,
                                                 float(swiglu_limit), _ptr(out), _ptr(out_scale), _ptr(ws), ws.numel(),
                                                 _stream(xq)),
          "moe355_gmm1_swiglu_quant_w4_gather")
    return out, out_scale


def gmm2_dequant_w4(x, weight_nz4, scale, group_size, per_token_scale, group_list, group_list_type, n, k, bias=None,
                    out_dtype=torch.bfloat16):
    lib = _lib.load()
    rows = x.shape[0]
    E = weight_nz4.shape[0]
    groups = k // group_size if group_size else 1
    _check_gmm_operands("gmm2_dequant_w4", x, rows, k, n, E, group_list, per_token_scale, "per_token_scale",
                        weight_nz4, E * n * k // 2, scale, E * groups * n)
    x = _dev(x, "x")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != E * n or not bias.is_cuda):
        raise ValueError(f"gmm2_dequant_w4: bias must be a float32 GPU tensor of E x N = {E * n} values")
    out = torch.empty((rows, n), dtype=_half_dtype(out_dtype), device=x.device)
    check(lib.moe355_gmm2_dequant_w4(_ptr(x), _ptr(_dev(weight_nz4, "weight")), _ptr(_dev(scale, "scale")),
                                     group_size, _ptr(bias), _ptr(_dev(per_token_scale, "per_token_scale")),
                                     _ptr(_gl(group_list)), _gl_type(group_list_type), rows, k, n, E, _ptr(out),
                                     _DT[out.dtype], _stream(x)), "moe355_gmm2_dequant_w4")
    return out


# ------------------------------------------------------------------ per-expert tensor lists
class ExpertTensorList(list):
    """E per-expert tensors of one shape and dtype together with the device array of their addresses that the
    ``*_list`` entry points of the library follow.  The table is built once, when the list is created (after
    weight loading), and lives as long as the list: a HIP graph that captured a launch keeps reading the same
    table.  Replacing an expert (``lst[e] = tensor``, what dynamic expert load balancing does when it cannot
    copy in place) rewrites that one entry of the same table; copying into an expert's tensor in place needs
    nothing."""

    def __init__(self, tensors, name="weight", dtype=None):
        super().__init__(tensors)
        if len(self) == 0:
            raise ValueError(f"{name}: an empty list of per-expert tensors")
        self.name = name
        dtype = dtype or self[0].dtype
        for t in self:
            self._check_one(t, dtype)
        self.table = torch.tensor([t.data_ptr() for t in self], dtype=torch.int64, device=self[0].device)

    def _check_one(self, t, dtype):
        first = self[0]
        if t.dtype != dtype or t.shape != first.shape or t.device != first.device or not t.is_contiguous():
            raise RuntimeError(f"{self.name}: every per-expert tensor must be a contiguous {dtype} tensor of one "
                               "shape on one device")

    def __setitem__(self, e, tensor):
        if not isinstance(e, int):
            raise TypeError("per-expert tensors are replaced one at a time")
        self._check_one(tensor, self[0].dtype)
        super().__setitem__(e, tensor)
        self.table[e] = tensor.data_ptr()  # same table, one entry rewritten

    def _frozen(self, *a, **k):
        raise TypeError("the number of experts of an ExpertTensorList is fixed")

    append = extend = insert = pop = remove = clear = __delitem__ = __iadd__ = __imul__ = sort = reverse = _frozen


def _as_expert_list(tensors, name, dtype) -> ExpertTensorList:
    """A plain list gets a table of its own for this one call (a synchronous host-to-device copy: not usable
    under graph capture); layers hold ExpertTensorList objects, whose table is reused."""
    if isinstance(tensors, ExpertTensorList):
        if tensors[0].dtype != dtype:
            raise RuntimeError(f"{name}: per-expert tensors must be {dtype}, got {tensors[0].dtype}")
        return tensors
    return ExpertTensorList(list(tensors), name, dtype)


def _check_list_operands(op, x, weights, scales, row_scale, row_scale_name, group_list):
    if not weights[0].is_cuda or not scales[0].is_cuda:
        raise RuntimeError(f"{op}: per-expert tensors must live on the GPU")
    if len(weights) != len(scales):
        raise ValueError(f"{op}: {len(weights)} weights but {len(scales)} scales")
    if weights[0].dim() != 2:
        raise ValueError(f"{op}: per-expert weights are [K, N] tiled tensors, got {tuple(weights[0].shape)}")
    k, n = weights[0].shape
    if scales[0].numel() != n:
        raise ValueError(f"{op}: per-expert scales must hold N = {n} values, got {scales[0].numel()}")
    _check_gmm_operands(op, x, x.shape[0], k, n, len(weights), group_list, row_scale, row_scale_name)
    return k, n


def gmm1_swiglu_quant_list(x, weight_list, scale_list, x_scale, group_list, group_list_type, swiglu_limit=0.0):
    """weight_list: E tiled int8 tensors of logical shape [K, N]; scale_list: E fp32 tensors [N]."""
    x = _dev(x, "x")
    lib = _lib.load()
    weight_list = _as_expert_list(weight_list, "weight", torch.int8)
    scale_list = _as_expert_list(scale_list, "weight_scale", torch.float32)
    k, n = _check_list_operands("gmm1_swiglu_quant_list", x, weight_list, scale_list, x_scale, "x_scale", group_list)
    rows, E, dev = x.shape[0], len(weight_list), x.device
    out = torch.empty((rows, n // 2), dtype=torch.int8, device=dev)
    out_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    ws = _workspace(lib.moe355_gmm1_swiglu_quant_workspace(rows, n, k, E), dev)
    check(lib.moe355_gmm1_swiglu_quant_list(_ptr(x), _ptr(weight_list.table), _ptr(scale_list.table),
                                            _ptr(_dev(x_scale, "x_scale")), _ptr(_gl(group_list)),
                                            _gl_type(group_list_type), rows, k, n, E, float(swiglu_limit), _ptr(out),
                                            _ptr(out_scale), _ptr(ws), ws.numel(), _stream(x)),
          "moe355_gmm1_swiglu_quant_list")
    return out, out_scale


def gmm2_dequant_list(x, weight_list, scale_list, per_token_scale, group_list, group_list_type,
                      out_dtype=torch.bfloat16):
    x = _dev(x, "x")
    lib = _lib.load()
    weight_list = _as_expert_list(weight_list, "weight", torch.int8)
    scale_list = _as_expert_list(scale_list, "scale", torch.float32)
    k, n = _check_list_operands("gmm2_dequant_list", x, weight_list, scale_list, per_token_scale, "per_token_scale",
                                group_list)
    rows, E = x.shape[0], len(weight_list)
    out = torch.empty((rows, n), dtype=_half_dtype(out_dtype), device=x.device)
    ws = _workspace(lib.moe355_gmm2_dequant_workspace(rows, n, k, E), x.device)
    check(lib.moe355_gmm2_dequant_list(_ptr(x), _ptr(weight_list.table), _ptr(scale_list.table),
                                       _ptr(_dev(per_token_scale, "per_token_scale")), _ptr(_gl(group_list)),
                                       _gl_type(group_list_type), rows, k, n, E, _ptr(out), _DT[out.dtype], _ptr(ws),
                                       ws.numel(), _stream(x)), "moe355_gmm2_dequant_list")
    return out


def w4_offset_correction(weight_nz4, weight_scale, group_size, n, k):
    """fp32 [E, N]: 8 * sum_k w * scale, the correction term of the reference's int4 op."""
    lib = _lib.load()
    w = _dev(weight_nz4, "weight")
    E = w.shape[0]
    corr = torch.empty((E, n), dtype=torch.float32, device=w.device)
    check(lib.moe355_w4_offset_correction(_ptr(w), _ptr(_dev(weight_scale, "weight_scale")), group_size, E, n, k,
                                          _ptr(corr), _stream(w)), "moe355_w4_offset_correction")
    return corr
