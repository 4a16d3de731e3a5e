"""numpy front end of the C checker in ``moe_oracle.c``.

TEST INFRASTRUCTURE ONLY (see ``moe_oracle.c`` for the arithmetic contract, the
reference citations of every stage and which checks pin each of them).

Conventions: bf16 / fp16 tensors travel as ``uint16`` numpy arrays holding the
raw bits; ``to_np`` / ``to_torch`` convert from and to torch CPU tensors.
Weights are ``[E, N, K]`` int8 (checkpoint order: one row of K per output
channel), scales ``[E, N]`` fp32, group lists are cumulative int64 ``[E]``
unless a function says otherwise.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import subprocess
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``moe_oracle.c`` with gcc (a few seconds)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])
    elif not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s"])
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_expf.restype = ctypes.c_float
        _lib.orc_expf.argtypes = [ctypes.c_float]
        _lib.orc_wave_tree_sum.restype = ctypes.c_float
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return ctypes.c_void_p(a.ctypes.data)


_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float


def num_threads() -> int:
    return int(lib().orc_num_threads())


# ----------------------------------------------------------------- conversions
def to_np(t):
    """torch CPU tensor -> numpy (bf16/fp16 as raw uint16 bits)."""
    import torch

    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def to_torch(a: np.ndarray, dtype=None):
    """numpy -> torch CPU tensor; ``dtype`` bf16/fp16 reinterprets uint16 bits."""
    import torch

    if dtype in (torch.bfloat16, torch.float16):
        return torch.from_numpy(a.view(np.int16).copy()).view(dtype)
    return torch.from_numpy(a.copy())


@contextlib.contextmanager
def half_kind(kind: str):
    """Hidden states in ``'bf16'`` (default) or ``'f16'`` while the block runs: the functions whose arguments are
    called ``*_bf16`` then take and return fp16 bit patterns."""
    if kind not in ("bf16", "f16"):
        raise ValueError(kind)
    before = lib().orc_get_half_kind()
    lib().orc_set_half_kind(ctypes.c_int(int(kind == "f16")))
    try:
        yield
    finally:
        lib().orc_set_half_kind(ctypes.c_int(before))


def f32_to_half(a: np.ndarray) -> np.ndarray:
    """fp32 -> the current kind of 16-bit float (see half_kind)."""
    return f32_to_f16(a) if lib().orc_get_half_kind() else f32_to_bf16(a)


def half_to_f32(a: np.ndarray) -> np.ndarray:
    return f16_to_f32(a) if lib().orc_get_half_kind() else bf16_to_f32(a)


def f32_to_bf16(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16(_p(a), _i64(a.size), _p(out))
    return out


def bf16_to_f32(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.float32)
    lib().orc_bf16_to_f32(_p(a), _i64(a.size), _p(out))
    return out


def f32_to_f16(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_f32_to_f16(_p(a), _i64(a.size), _p(out))
    return out


def f16_to_f32(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.float32)
    lib().orc_f16_to_f32(_p(a), _i64(a.size), _p(out))
    return out


def expf(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    f = lib().orc_expf
    return np.array([f(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def wave_tree_sum(v: np.ndarray) -> np.float32:
    v = np.ascontiguousarray(v, dtype=np.float32)
    return np.float32(lib().orc_wave_tree_sum(_p(v), _i32(v.size)))


# ----------------------------------------------------------------- stages
def gating_top_k(x, k, *, bias=None, k_group=1, group_count=1, group_select_mode=1, renorm=0, norm_type=0,
                 routed_scaling_factor=1.0, eps=1e-20, x_dtype="f32", want_norm=False):
    """Group-limited top-k routing.  ``x_dtype``: 'f32' | 'bf16' | 'f16' (x and bias
    given as raw bits for the 16-bit types).  Returns (y in x_dtype, idx int32, norm|None)."""
    widen = {"f32": lambda a: np.ascontiguousarray(a, dtype=np.float32), "bf16": bf16_to_f32, "f16": f16_to_f32}[x_dtype]
    narrow = {"f32": lambda a: a, "bf16": f32_to_bf16, "f16": f32_to_f16}[x_dtype]
    xf = widen(x)
    bf = widen(bias) if bias is not None else None
    T, E = xf.shape
    y = np.empty((T, k), dtype=np.float32)
    idx = np.empty((T, k), dtype=np.int32)
    norm = np.empty((T, E), dtype=np.float32) if want_norm else None
    rc = lib().orc_gating_top_k(_p(xf), _p(bf), _i64(T), _i32(E), _i32(k), _i32(k_group), _i32(group_count),
                                _i32(group_select_mode), _i32(renorm), _i32(norm_type), _f32(routed_scaling_factor),
                                _f32(eps), _p(y), _p(idx), _p(norm))
    if rc != 0:
        raise ValueError(f"orc_gating_top_k rejected the arguments (rc={rc})")
    return narrow(y), idx, norm


def router_gate(x, w, bias=None) -> np.ndarray:
    """x [T, H] bf16 bit patterns (uint16) or float32, w [E, H] float32 -> logits [T, E] float32."""
    is_bf16 = x.dtype == np.uint16
    x = np.ascontiguousarray(x, dtype=np.uint16 if is_bf16 else np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    T, H = x.shape
    E = w.shape[0]
    assert w.shape[1] == H
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((T, E), dtype=np.float32)
    lib().orc_router_gate(_p(x), ctypes.c_int(int(is_bf16)), _p(w), _p(b), _i64(T), _i64(H), _i64(E), _p(out))
    return out


def dynamic_quant(x_bf16: np.ndarray):
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    rows, cols = x.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty((rows,), dtype=np.float32)
    lib().orc_dynamic_quant_bf16(_p(x), _i64(rows), _i64(cols), _p(q), _p(s))
    return q, s


def init_routing(x_bf16, topk_ids, num_experts, quant=True):
    """Returns (expanded_x, expanded_row_idx[R] int32, expert_tokens[E] int64 counts, dynamic_scale[R]|None).
    Pairs whose expert id lies outside [0, num_experts) are dropped: destination R, rows past the last valid one
    are left zero."""
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
    T, k = ids.shape
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    H = x.shape[1]
    R = T * k
    dst = np.empty((R,), dtype=np.int32)
    cnt = np.empty((num_experts,), dtype=np.int64)
    if quant:
        xs = np.zeros((R, H), dtype=np.int8)
        sx = np.zeros((R,), dtype=np.float32)
        rc = lib().orc_init_routing(_p(ids), _i64(T), _i32(k), _i32(num_experts), _p(x), _i64(H), _p(dst), _p(cnt),
                                    _p(xs), _p(sx))
        if rc != 0:
            raise ValueError(f"orc_init_routing failed (rc={rc})")
        return xs, dst, cnt, sx
    rc = lib().orc_init_routing(_p(ids), _i64(T), _i32(k), _i32(num_experts), None, _i64(H), _p(dst), _p(cnt), None,
                                None)
    if rc != 0:
        raise ValueError(f"orc_init_routing failed (rc={rc})")
    xp = np.zeros((R, H), dtype=np.uint16)
    lib().orc_permute_rows_bf16(_p(dst), _i64(T), _i32(k), _p(x), _i64(H), _p(xp))
    return xp, dst, cnt, None


def gmm_i32(x_i8, w_enk, cum):
    x = np.ascontiguousarray(x_i8, dtype=np.int8)
    w = np.ascontiguousarray(w_enk, dtype=np.int8)
    cum = np.ascontiguousarray(cum, dtype=np.int64)
    R, K = x.shape
    E, N, K2 = w.shape
    assert K == K2 and cum.shape == (E,)
    acc = np.zeros((R, N), dtype=np.int32)
    lib().orc_gmm_i32(_p(x), _p(w), _p(cum), _i64(R), _i64(K), _i64(N), _i32(E), _p(acc))
    return acc


def gmm_w4_grouped(x_i8, w_enk_int4vals, sg, cum, group_size):
    x = np.ascontiguousarray(x_i8, dtype=np.int8)
    w = np.ascontiguousarray(w_enk_int4vals, dtype=np.int8)
    sg = np.ascontiguousarray(sg, dtype=np.float32)
    cum = np.ascontiguousarray(cum, dtype=np.int64)
    R, K = x.shape
    E, N, _ = w.shape
    assert sg.shape == (E, K // group_size, N)
    f = np.zeros((R, N), dtype=np.float32)
    rc = lib().orc_gmm_w4_grouped(_p(x), _p(w), _p(sg), _p(cum), _i64(R), _i64(K), _i64(N), _i32(E), _i64(group_size),
                                  _p(f))
    assert rc == 0
    return f


def dequant_acc(acc, sx, sw, cum):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sx = np.ascontiguousarray(sx, dtype=np.float32)
    sw = np.ascontiguousarray(sw, dtype=np.float32)
    cum = np.ascontiguousarray(cum, dtype=np.int64)
    R, N = acc.shape
    f = np.zeros((R, N), dtype=np.float32)
    lib().orc_dequant_acc(_p(acc), _p(sx), _p(sw), _p(cum), _i64(R), _i64(N), _i32(cum.size), _p(f))
    return f


def scale_rows(f, sx):
    f = np.ascontiguousarray(f, dtype=np.float32).copy()
    sx = np.ascontiguousarray(sx, dtype=np.float32)
    lib().orc_scale_rows(_p(f), _p(sx), _i64(f.shape[0]), _i64(f.shape[1]))
    return f


def w4_rows_to_bf16(f, s1):
    f = np.ascontiguousarray(f, dtype=np.float32)
    s1 = np.ascontiguousarray(s1, dtype=np.float32)
    o = np.zeros(f.shape, dtype=np.uint16)
    lib().orc_w4_rows_to_bf16(_p(f), _p(s1), _i64(f.shape[0]), _i64(f.shape[1]), _p(o))
    return o


def w4a8_experts_forward(x_bf16, topk_w_bf16, topk_ids, w13_i4, sg13, w2_i4, sg2, group_size) -> LayerTrace:
    """W4A8 twin of experts_forward: int4 weight values (one per int8) [E,N,K], group scales [E,K/g,N]."""
    E = w13_i4.shape[0]
    tr = LayerTrace(topk_weights=topk_w_bf16, topk_ids=topk_ids)
    tr.xs, tr.expanded_row_idx, tr.expert_tokens, tr.sx = init_routing(x_bf16, topk_ids, E)
    cum = np.cumsum(tr.expert_tokens)
    g1 = group_size if group_size > 0 else w13_i4.shape[2]
    g2 = group_size if group_size > 0 else w2_i4.shape[2]
    f = scale_rows(gmm_w4_grouped(tr.xs, w13_i4, sg13, cum, g1), tr.sx)
    tr.q1, tr.s1 = swiglu_quant(f)
    f2 = gmm_w4_grouped(tr.q1, w2_i4, sg2, cum, g2)
    tr.o = w4_rows_to_bf16(f2, tr.s1)
    tr.out = unpermute(tr.o, tr.expanded_row_idx, topk_w_bf16)
    return tr


def swiglu_quant(f, swiglu_limit=0.0, want_y=False):
    f = np.ascontiguousarray(f, dtype=np.float32)
    rows, N = f.shape
    q = np.zeros((rows, N // 2), dtype=np.int8)
    qs = np.zeros((rows,), dtype=np.float32)
    y = np.zeros((rows, N // 2), dtype=np.float32) if want_y else None
    lib().orc_swiglu_quant(_p(f), _i64(rows), _i64(N), _f32(swiglu_limit), _p(q), _p(qs), _p(y))
    return (q, qs, y) if want_y else (q, qs)


def silu(g):
    """g / (1 + exp(-g)) element by element in binary32 (the gate function of the SwiGLU)."""
    g = np.ascontiguousarray(g, dtype=np.float32)
    out = np.empty_like(g)
    lib().orc_silu(_p(g), _i64(g.size), _p(out))
    return out


def gmm2_dequant(acc, s1, s2, cum):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    s1 = np.ascontiguousarray(s1, dtype=np.float32)
    s2 = np.ascontiguousarray(s2, dtype=np.float32)
    cum = np.ascontiguousarray(cum, dtype=np.int64)
    R, N = acc.shape
    o = np.zeros((R, N), dtype=np.uint16)
    lib().orc_gmm2_dequant(_p(acc), _p(s1), _p(s2), _p(cum), _i64(R), _i64(N), _i32(cum.size), _p(o))
    return o


def unpermute(o_bf16, dst, w_bf16, add_bf16=None):
    o = np.ascontiguousarray(o_bf16, dtype=np.uint16)
    w = np.ascontiguousarray(w_bf16, dtype=np.uint16)
    T, k = w.shape
    dst = np.ascontiguousarray(dst, dtype=np.int32).reshape(-1)
    H = o.shape[1]
    add = np.ascontiguousarray(add_bf16, dtype=np.uint16) if add_bf16 is not None else None
    out = np.empty((T, H), dtype=np.uint16)
    lib().orc_unpermute(_p(o), _i64(o.shape[0]), _p(dst), _p(w), _i64(T), _i32(k), _i64(H), _p(add), _p(out))
    return out


def dequant_swiglu_quant(x_i32, w_scale, a_scale, activate_left=True, clamp_limit=0.0):
    x = np.ascontiguousarray(x_i32, dtype=np.int32)
    rows, N = x.shape
    ws = np.ascontiguousarray(w_scale, dtype=np.float32).reshape(-1)
    as_ = np.ascontiguousarray(a_scale, dtype=np.float32).reshape(-1)
    q = np.zeros((rows, N // 2), dtype=np.int8)
    qs = np.zeros((rows,), dtype=np.float32)
    lib().orc_dequant_swiglu_quant(_p(x), _p(ws), _p(as_), _i64(rows), _i64(N), _i32(int(activate_left)),
                                   _f32(clamp_limit), _p(q), _p(qs))
    return q, qs


def dequant_swiglu_quant_grouped(x_i32, w_scale, a_scale=None, group_index=None, bias=None, activate_left=True,
                                 swiglu_mode=0, clamp_limit=0.0, glu_alpha=1.0, glu_bias=0.0, quant_mode=1,
                                 quant_scale=None, quant_offset=None):
    """The grouped form: w_scale [G, N] (or [N]), group_index [G] row counts or None, bias [G, N] int32 or float.
    -> (q int8 [rows, N/2], scale [rows] float32; zeros in static mode)."""
    x = np.ascontiguousarray(x_i32, dtype=np.int32)
    rows, N = x.shape
    ws = np.ascontiguousarray(w_scale, dtype=np.float32).reshape(-1, N)
    G = ws.shape[0]
    as_ = None if a_scale is None else np.ascontiguousarray(a_scale, dtype=np.float32).reshape(-1)
    gi = None if group_index is None else np.ascontiguousarray(group_index, dtype=np.int64).reshape(-1)
    assert gi is None or gi.size == G
    kind, b = 0, None
    if bias is not None:
        kind = 1 if np.asarray(bias).dtype == np.int32 else 2
        b = np.ascontiguousarray(bias, dtype=np.int32 if kind == 1 else np.float32).reshape(G, N)
    qsc = qof = None
    per_channel = 0
    if quant_mode == 0:
        qsc = np.ascontiguousarray(quant_scale, dtype=np.float32).reshape(-1)
        per_channel = int(qsc.size == G * (N // 2) and N // 2 != 1)
        assert per_channel or qsc.size == G
        if quant_offset is not None:
            qof = np.ascontiguousarray(quant_offset, dtype=np.float32).reshape(-1)
            assert qof.size == qsc.size
    q = np.zeros((rows, N // 2), dtype=np.int8)
    qs = np.zeros((rows,), dtype=np.float32)
    lib().orc_dequant_swiglu_quant_grouped(_p(x), _p(ws), _p(as_), _p(b), _i32(kind), _p(gi), _i64(G), _i64(rows),
                                           _i64(N), _i32(int(activate_left)), _i32(swiglu_mode), _f32(clamp_limit),
                                           _f32(glu_alpha), _f32(glu_bias), _i32(quant_mode), _p(qsc),
                                           _i32(per_channel), _p(qof), _p(q), _p(qs))
    return q, qs


def dequant_swiglu_quant_static(x_i32, w_scale, a_scale, quant_scale, quant_offset=None, activate_left=True,
                                clamp_limit=0.0):
    x = np.ascontiguousarray(x_i32, dtype=np.int32)
    rows, N = x.shape
    ws = np.ascontiguousarray(w_scale, dtype=np.float32)
    as_ = np.ascontiguousarray(a_scale, dtype=np.float32).reshape(-1)
    qsc = np.ascontiguousarray(quant_scale, dtype=np.float32).reshape(-1)
    qof = None if quant_offset is None else np.ascontiguousarray(quant_offset, dtype=np.float32).reshape(-1)
    q = np.zeros((rows, N // 2), dtype=np.int8)
    lib().orc_dequant_swiglu_quant_static(_p(x), _p(ws), _p(as_), _p(qsc), _i64(qsc.size), _p(qof), _i64(rows), _i64(N),
                                          _i32(int(activate_left)), _f32(clamp_limit), _p(q))
    return q


ACTIVATIONS = {"gelu": 1, "gelu_tanh": 2, "swiglustep": 3, "swigluoai": 4}


def erff(x):
    f = lib().orc_erff
    f.restype, f.argtypes = ctypes.c_float, [ctypes.c_float]
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).reshape(-1)], dtype=np.float32)


def tanhf(x):
    f = lib().orc_tanhf
    f.restype, f.argtypes = ctypes.c_float, [ctypes.c_float]
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).reshape(-1)], dtype=np.float32)


def act_mul_quant(h_bits, activation: str, limit=0.0, alpha=1.0, beta=0.0):
    """h_bits [rows, 2I] 16-bit floats as uint16 (gate first) -> int8 [rows, I], fp32 scale [rows]."""
    h = np.ascontiguousarray(h_bits, dtype=np.uint16)
    rows, N = h.shape
    q = np.zeros((rows, N // 2), dtype=np.int8)
    qs = np.zeros((rows,), dtype=np.float32)
    rc = lib().orc_act_mul_quant(_p(h), _i64(rows), _i64(N), _i32(ACTIVATIONS[activation]), _f32(limit), _f32(alpha),
                                 _f32(beta), _p(q), _p(qs))
    if rc != 0:
        raise ValueError(f"orc_act_mul_quant rejected the arguments (rc={rc})")
    return q, qs


def cumsum_group_list(group_list: np.ndarray, src_list_type: int, dst_list_type: int) -> np.ndarray:
    """count <-> cumulative conversion; restates vllm_ascend/ops/fused_moe/moe_mlp.py:54-83 (types 0 and 1)."""
    if src_list_type not in (0, 1, 2):
        raise ValueError(f"group_list_type should be in [0, 1, 2], but received {src_list_type}")
    if src_list_type == dst_list_type:
        return group_list
    if src_list_type == 1 and dst_list_type == 0:
        return np.cumsum(group_list)
    if src_list_type == 0 and dst_list_type == 1:
        return np.concatenate([group_list[:1], np.diff(group_list)])
    raise NotImplementedError("conversion not restated in the checker")


# ----------------------------------------------------------------- whole layer
@dataclass
class LayerTrace:
    """Every intermediate of one routed-experts pass (names follow the layer's stages)."""

    topk_weights: np.ndarray = None  # [T,k] bf16 bits
    topk_ids: np.ndarray = None  # [T,k] int32
    expanded_row_idx: np.ndarray = None  # [R] int32
    expert_tokens: np.ndarray = None  # [E] int64 counts
    xs: np.ndarray = None  # [R,H] int8
    sx: np.ndarray = None  # [R] fp32
    acc1: np.ndarray = None  # [R,2I] int32
    q1: np.ndarray = None  # [R,I] int8
    s1: np.ndarray = None  # [R] fp32
    acc2: np.ndarray = None  # [R,H] int32
    o: np.ndarray = None  # [R,H] bf16 bits
    out: np.ndarray = None  # [T,H] bf16 bits
    extra: dict = field(default_factory=dict)


def experts_forward(x_bf16, topk_w_bf16, topk_ids, w13, s13, w2, s2, *, keep_acc=True, add_bf16=None,
                    activation="silu", swiglu_limit=0.0, swiglu_alpha=1.0, swiglu_beta=0.0) -> LayerTrace:
    """dispatch -> gate_up GEMM + SwiGLU/re-quant -> down GEMM + dequant -> combine.
    Stage order restates vllm_ascend/ops/fused_moe/moe_comm_method.py:117-162.  An activation other than SiLU takes
    the unfused form of vllm_ascend/ops/fused_moe/moe_mlp.py:484-549: gate_up product dequantised to 16 bits,
    activation, dynamic quantisation."""
    E = w13.shape[0]
    tr = LayerTrace(topk_weights=topk_w_bf16, topk_ids=topk_ids)
    tr.xs, tr.expanded_row_idx, tr.expert_tokens, tr.sx = init_routing(x_bf16, topk_ids, E)
    cum = np.cumsum(tr.expert_tokens)
    acc1 = gmm_i32(tr.xs, w13, cum)
    if activation == "silu":
        f = dequant_acc(acc1, tr.sx, s13, cum)
        tr.q1, tr.s1 = swiglu_quant(f, swiglu_limit)
    else:
        h = gmm2_dequant(acc1, tr.sx, s13, cum)
        limit = (swiglu_limit or 7.0) if activation == "swiglustep" else swiglu_limit
        tr.q1, tr.s1 = act_mul_quant(h, activation, limit, swiglu_alpha, swiglu_beta)
    acc2 = gmm_i32(tr.q1, w2, cum)
    tr.o = gmm2_dequant(acc2, tr.s1, s2, cum)
    tr.out = unpermute(tr.o, tr.expanded_row_idx, topk_w_bf16, add_bf16)
    if keep_acc:
        tr.acc1, tr.acc2 = acc1, acc2
    return tr


def shared_expert_forward(x_bf16, w13, s13, w2, s2, swiglu_limit=0.0, swiglu_alpha=1.0, swiglu_beta=0.0) -> np.ndarray:
    """Dense W8A8 MLP every token goes through, op for op as the reference's shared expert
    (vllm_ascend/ops/fused_moe/shared_experts.py:254-301): dynamic quant -> int32 matmul ->
    dequant_swiglu_quant (weight scale first, then activation scale; called with swiglu_mode=1 on int32 x,
    :272-289, which the reference's tiling sends to its grouped kernel class) -> matmul with per-token
    scale -> bf16.  w13 [2I,H], s13 [2I], w2 [H,I], s2 [H]."""
    T = x_bf16.shape[0]
    one = np.array([T], dtype=np.int64)
    xq, sx = dynamic_quant(x_bf16)
    acc1 = gmm_i32(xq, w13[None], one)
    q1, s1 = dequant_swiglu_quant_grouped(acc1, s13, sx, activate_left=True, swiglu_mode=1, clamp_limit=swiglu_limit,
                                          glu_alpha=swiglu_alpha, glu_bias=swiglu_beta)
    acc2 = gmm_i32(q1, w2[None], one)
    return gmm2_dequant(acc2, s1, s2[None], one)


def moe_layer(x_bf16, logits_f32, w13, s13, w2, s2, *, top_k, bias=None, k_group=1, group_count=1, renorm=1,
              norm_type=0, routed_scaling_factor=1.0, keep_acc=True, shared=None) -> LayerTrace:
    """router logits -> final bf16, all stages.  ``shared`` = (w13s[1,2I,H], s13s[1,2I], w2s[1,H,I], s2s[1,H]):
    a dense W8A8 expert every token goes through, added to the routed output in fp32."""
    y, ids, _ = gating_top_k(logits_f32, top_k, bias=bias, k_group=k_group, group_count=group_count,
                             group_select_mode=1, renorm=renorm, norm_type=norm_type,
                             routed_scaling_factor=routed_scaling_factor, x_dtype="f32")
    w_bf16 = f32_to_half(y)
    add = None
    extra = {}
    if shared is not None:
        sw13, ss13, sw2, ss2 = shared
        add = shared_expert_forward(x_bf16, sw13[0], ss13[0], sw2[0], ss2[0])
        extra["shared_out"] = add
    tr = experts_forward(x_bf16, w_bf16, ids, w13, s13, w2, s2, keep_acc=keep_acc, add_bf16=add)
    tr.extra.update(extra)
    return tr


def fp32_dequant_reference(x_bf16, topk_w_bf16, topk_ids, w13, s13, w2, s2) -> np.ndarray:
    """Dense fp32 rendering without any activation quantisation (weights * scale in
    fp32), the tolerance reference for the bf16 output.  Restates torch_moe of
    tests/e2e/nightly/single_node/ops/singlecard_ops/test_fused_moe.py:85-97."""
    x = half_to_f32(x_bf16).astype(np.float64)
    w = half_to_f32(topk_w_bf16).astype(np.float64)
    T, k = topk_ids.shape
    H = x.shape[1]
    I = w2.shape[2]
    out = np.zeros((T, H), dtype=np.float64)
    for e in np.unique(topk_ids):
        tok, slot = np.nonzero(topk_ids == e)
        if tok.size == 0:
            continue
        w1 = w13[e].astype(np.float64) * s13[e].astype(np.float64)[:, None]
        wd = w2[e].astype(np.float64) * s2[e].astype(np.float64)[:, None]
        gu = x[tok] @ w1.T
        g, u = gu[:, :I], gu[:, I:]
        act = g / (1.0 + np.exp(-g)) * u
        o = act @ wd.T
        np.add.at(out, tok, o * w[tok, slot][:, None])
    return out.astype(np.float32)


def quantized_fp64_reference(tr: LayerTrace, s2) -> np.ndarray:
    """The same quantised pipeline (identical int8 activations and int32 accumulators) with the
    final dequantisation and the weighted combine evaluated in float64 and no bf16 rounding:
    isolates the rounding error of the floating-point tail from the quantisation noise."""
    E = tr.expert_tokens.size
    cum = np.cumsum(tr.expert_tokens)
    row_expert = np.searchsorted(cum, np.arange(tr.acc2.shape[0]), side="right")
    o = tr.acc2.astype(np.float64) * tr.s1.astype(np.float64)[:, None] * s2.astype(np.float64)[row_expert]
    w = half_to_f32(tr.topk_weights).astype(np.float64)
    T, k = w.shape
    dst = tr.expanded_row_idx.reshape(T, k)
    return (o[dst] * w[:, :, None]).sum(axis=1).astype(np.float32)
