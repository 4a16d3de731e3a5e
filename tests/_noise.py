"""Where the relative error of the 16-bit layer output against an fp32-dequant reference comes from.

A numpy rendering of the reference's own golden math, with nothing from the CPU checker in it: the gate_up stage
follows ``gmm_swiglu_quant`` of tests/e2e/nightly/single_node/ops/singlecard_ops/
test_gmm_swiglu_quant_weight_nz_tensor_list.py:14-55 (int matmul, channel scale, token scale, x * sigmoid(x) * up,
scale = 127 / max, round), the token quantiser is the closed form ``scale = absmax / 127, q = round(x / scale)`` of
the public dynamic quantiser, the rest is float64.  Either activation quantisation can be switched off, which
splits the error of the quantised layer into the share of the first quantiser (hidden states) and the share of the
second (SwiGLU output).  Used by tests/test_tolerance_floor.py and by the parity block of the benchmark.
"""
from __future__ import annotations

import numpy as np


def quantise_rows(v: np.ndarray):
    """Per-row symmetric int8: scale = absmax / 127, q = round-half-even(v / scale); all-zero rows stay zero."""
    v = np.asarray(v, dtype=np.float64)
    a = np.abs(v).max(axis=-1)
    s = np.where(a > 0, a / 127.0, 1.0)
    q = np.clip(np.rint(v / s[:, None]), -128, 127)
    return q, np.where(a > 0, s, 0.0)


def expert_mlp_variants(x_rows, w_up, s_up, w_down, s_down, variants) -> list:
    """One expert on a few rows in float64, once per (first, second) pair in `variants`.
    w_up [2I, H] int8 with scales s_up [2I], w_down [H, I] with s_down [H].  first / second: apply the quantiser
    in front of the gate_up product / in front of the down product."""
    x_rows = np.asarray(x_rows, dtype=np.float64)
    wu = w_up.astype(np.float64)
    wd = w_down.astype(np.float64)
    su = s_up.astype(np.float64)[None, :]
    sd = s_down.astype(np.float64)[None, :]
    q, s = quantise_rows(x_rows)
    c_by_first = {True: ((q @ wu.T) * su) * s[:, None],  # golden order: channel scale, then token scale
                  False: (x_rows @ wu.T) * su}
    outs = []
    for first, second in variants:
        c = c_by_first[first]
        half = c.shape[1] // 2
        a, up = c[:, :half], c[:, half:]
        y = a * (1.0 / (1.0 + np.exp(-a))) * up
        if second:
            q1, s1 = quantise_rows(y)
            outs.append((q1 @ wd.T) * s1[:, None] * sd)
        else:
            outs.append((y @ wd.T) * sd)
    return outs


VARIANTS = ((False, False), (True, False), (False, True), (True, True))


def layer_tokens_variants(x_tok, w_tok, ids_tok, w13, s13, w2, s2, variants=VARIANTS) -> list:
    """The routed layer for a few tokens, once per variant: x_tok [n, H] and w_tok [n, k] as float values,
    ids_tok [n, k]; int8 weights w13 [E, 2I, H], w2 [E, H, I] with per-channel scales.  No 16-bit rounding."""
    n = ids_tok.shape[0]
    outs = [np.zeros((n, w2.shape[1]), dtype=np.float64) for _ in variants]
    wt = np.asarray(w_tok, dtype=np.float64)
    for e in np.unique(ids_tok):
        tok, slot = np.nonzero(ids_tok == e)
        for out, o in zip(outs, expert_mlp_variants(x_tok[tok], w13[e], s13[e], w2[e], s2[e], variants)):
            np.add.at(out, tok, o * wt[tok, slot][:, None])
    return outs


def _rel(a, b) -> float:
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def error_split(x_tok, w_tok, ids_tok, w13, s13, w2, s2) -> dict:
    """Relative error against the layer without activation quantisation, with only the first quantiser, only the
    second, and both (int8 per-channel weights)."""
    ref, first, second, both = layer_tokens_variants(x_tok, w_tok, ids_tok, w13, s13, w2, s2)
    return {
        "first_quant_only": _rel(first, ref),
        "second_quant_only": _rel(second, ref),
        "both": _rel(both, ref),
        "_both_output": both,
        "_reference": ref,
    }
