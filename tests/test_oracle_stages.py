"""Pins for the checker's permutation, quantiser, grouped GEMM, epilogues and combine (CPU only).
Each check compares the C checker with something that is not its own code: the reference's
known-answer vectors, numpy renderings of the reference's golden functions, library routines
(stable argsort, bincount, integer matmul) or closed forms."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as orc

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def bf16(a):
    return orc.f32_to_bf16(np.asarray(a, dtype=np.float32))


# ------------------------------------------------------------------ conversions
def test_bf16_rounding_closed_forms():
    # exactly representable values survive; ties go to even; NaN stays NaN
    v = np.array([1.0, -2.5, 0.0, 3.140625], dtype=np.float32)
    assert np.array_equal(orc.bf16_to_f32(bf16(v)), v)
    one_plus_half_ulp = np.float32(1.0 + 2.0 ** -8)  # halfway between 1.0 and the next bf16
    assert orc.bf16_to_f32(bf16([one_plus_half_ulp]))[0] == 1.0  # tie -> even mantissa
    three_halves_ulp = np.float32(1.0 + 3 * 2.0 ** -8)
    assert orc.bf16_to_f32(bf16([three_halves_ulp]))[0] == np.float32(1.0 + 2.0 ** -6)
    assert np.isnan(orc.bf16_to_f32(bf16([np.nan]))[0])
    import torch

    x = torch.randn(4096, dtype=torch.float32)
    assert np.array_equal(bf16(x.numpy()), orc.to_np(x.to(torch.bfloat16)))
    assert np.array_equal(orc.f32_to_f16(x.numpy()), x.numpy().astype(np.float16).view(np.uint16))
    big = np.array([65504.0, 65519.9, 65520.0, 1e-8, 6e-8, -1e-5], dtype=np.float32)
    assert np.array_equal(orc.f32_to_f16(big), big.astype(np.float16).view(np.uint16))
    h = np.arange(0, 65536, 7, dtype=np.uint16)
    ref = h.view(np.float16).astype(np.float32)
    got = orc.f16_to_f32(h)
    assert np.array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])


# ------------------------------------------------------------------ permutation
def test_permutation_known_answer_of_the_reference():
    k = KATS["permutation"]
    ids = np.array(k["topk_ids"], dtype=np.int32)
    x = np.zeros((3, 8), dtype=np.uint16)
    _, dst, cnt, _ = orc.init_routing(x, ids, 2)
    assert dst.tolist() == k["expanded_row_idx"]
    # the reference recovers the expert of each sorted row through the inverse permutation
    inv = np.argsort(dst)
    assert ids.reshape(-1)[inv].tolist() == k["expert_of_sorted_row"]
    assert cnt.tolist() == [2, 4]


@pytest.mark.parametrize("T,k,E", [(1, 1, 4), (64, 8, 128), (333, 6, 64), (40, 2, 2048)])
def test_permutation_is_the_inverse_of_a_stable_argsort(T, k, E):
    rng = np.random.RandomState(T + E)
    ids = rng.randint(0, E, size=(T, k)).astype(np.int32)
    x = orc.f32_to_bf16(rng.normal(size=(T, 16)).astype(np.float32))
    xp, dst, cnt, _ = orc.init_routing(x, ids, E, quant=False)
    order = np.argsort(ids.reshape(-1), kind="stable")  # sorted position -> flat index
    assert np.array_equal(dst[order], np.arange(T * k))
    assert np.array_equal(cnt, np.bincount(ids.reshape(-1), minlength=E))
    assert np.array_equal(xp, x[order // k])  # sorted row i holds the token of flat pair order[i]


def test_pairs_with_out_of_range_experts_are_dropped():
    """Ids outside [0, E) take no row: the other pairs keep the stable order among themselves, the histogram
    only counts them, and the dropped pairs point one past the last row (the index the combine skips, as the
    reference kernel skips indices >= num_out_tokens, moe_token_unpermute.h:250-275)."""
    rng = np.random.RandomState(77)
    T, k, E, H = 50, 4, 16, 32
    ids = rng.randint(0, E, size=(T, k)).astype(np.int32)
    flat = ids.reshape(-1)
    bad = rng.choice(T * k, size=23, replace=False)
    flat[bad[:10]] = E + rng.randint(0, 5, size=10)
    flat[bad[10:]] = -1 - rng.randint(0, 5, size=13)
    x = orc.f32_to_bf16(rng.normal(size=(T, H)).astype(np.float32))
    xs, dst, cnt, sx = orc.init_routing(x, ids, E)
    R = T * k
    valid = (flat >= 0) & (flat < E)
    assert np.all(dst[~valid] == R)
    keep = np.nonzero(valid)[0]
    order = keep[np.argsort(flat[keep], kind="stable")]  # sorted position -> flat index, valid pairs only
    assert np.array_equal(dst[order], np.arange(order.size))
    assert np.array_equal(cnt, np.bincount(flat[keep], minlength=E))
    q, s = orc.dynamic_quant(x)
    assert np.array_equal(xs[: order.size], q[order // k]) and np.array_equal(sx[: order.size], s[order // k])
    assert not xs[order.size:].any()  # rows past the last valid pair are not written
    # ... and the combine leaves them out: the same result as a combine over the valid pairs with the others' weights at 0
    o = bf16(rng.normal(size=(R, H)).astype(np.float32))
    w = bf16(rng.rand(T, k).astype(np.float32))
    w0 = w.copy().reshape(-1)
    w0[~valid] = 0
    dst0 = np.where(valid, dst, 0).astype(np.int32)
    assert np.array_equal(orc.unpermute(o, dst, w), orc.unpermute(o, dst0, w0.reshape(T, k)))


def test_cumsum_group_list_vectors():
    k = KATS["cumsum_group_list"]
    c0, c1 = np.array(k["type0_cumsum"]), np.array(k["type1_count"])
    assert np.array_equal(orc.cumsum_group_list(c1, 1, 0), c0)
    assert np.array_equal(orc.cumsum_group_list(c0, 0, 1), c1)
    assert orc.cumsum_group_list(c0, 0, 0) is c0


# ------------------------------------------------------------------ quantiser
def test_quantiser_closed_forms():
    # a row of -127..127 times c quantises to itself with scale c (c a power of two: exact)
    c = np.float32(0.25)
    row = (np.arange(-127, 128, dtype=np.float32) * c)[None, :]
    row = np.concatenate([row, np.zeros((1, 1), np.float32)], axis=1)  # 256 columns
    q, s = orc.dynamic_quant(bf16(row))
    assert s[0] == c and np.array_equal(q[0, :255], np.arange(-127, 128))
    # all-zero row -> zeros, scale 0
    q, s = orc.dynamic_quant(bf16(np.zeros((2, 64))))
    assert s.tolist() == [0.0, 0.0] and not q.any()
    # single non-zero element is the absmax -> +-127
    z = np.zeros((1, 64), np.float32)
    z[0, 5] = -3.0
    q, s = orc.dynamic_quant(bf16(z))
    assert q[0, 5] == -127 and s[0] == np.float32(3.0) / np.float32(127.0)
    # halves round to even: scale 1 (absmax 127), values k + 0.5
    v = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 3.5, 0.0]], dtype=np.float32)
    q, s = orc.dynamic_quant(bf16(v))
    assert s[0] == 1.0 and q[0].tolist() == [127, 0, 2, 2, 0, -2, 4, 0]
    # invariants on random rows
    rng = np.random.RandomState(0)
    x = bf16(rng.normal(size=(50, 512)).astype(np.float32))
    q, s = orc.dynamic_quant(x)
    assert np.all(np.abs(q.astype(np.int32)).max(axis=1) == 127)
    xf = orc.bf16_to_f32(x)
    assert np.allclose(s, np.abs(xf).max(axis=1) / 127.0, rtol=1e-7)
    assert np.max(np.abs(q * s[:, None] - xf)) <= 0.5001 * s.max()


def test_fused_quant_in_the_gather_equals_the_standalone_quantiser():
    rng = np.random.RandomState(1)
    T, k, E, H = 20, 4, 16, 64
    x = bf16(rng.normal(size=(T, H)).astype(np.float32))
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    xs, dst, _, sx = orc.init_routing(x, ids, E)
    q, s = orc.dynamic_quant(x)
    for t in range(T):
        for j in range(k):
            assert np.array_equal(xs[dst[t * k + j]], q[t]) and sx[dst[t * k + j]] == s[t]


# ------------------------------------------------------------------ integer GEMM
@pytest.mark.parametrize("R,E,K,N", [(17, 3, 64, 32), (100, 8, 256, 96), (5, 4, 7168, 64)])
def test_grouped_gemm_is_an_exact_integer_matmul(R, E, K, N):
    rng = np.random.RandomState(R)
    x = rng.randint(-128, 128, size=(R, K)).astype(np.int8)
    w = rng.randint(-128, 128, size=(E, N, K)).astype(np.int8)
    cnt = np.bincount(rng.randint(0, E, size=R - 2), minlength=E)  # two trailing rows belong to no expert
    cum = np.cumsum(cnt)
    acc = orc.gmm_i32(x, w, cum)
    ref = np.zeros((R, N), dtype=np.int64)
    r = 0
    for e in range(E):
        ref[r:r + cnt[e]] = x[r:r + cnt[e]].astype(np.int64) @ w[e].astype(np.int64).T
        r += cnt[e]
    assert np.array_equal(acc.astype(np.int64), ref)
    assert not acc[cum[-1]:].any()
    # worst case magnitude stays inside int32: 7168 * 128 * 128 < 2^31
    assert 7168 * 128 * 128 < 2 ** 31


# ------------------------------------------------------------------ gate_up epilogue
def golden_gmm_swiglu_quant(x, w_kn, per_channel, per_token):
    """numpy rendering of gmm_swiglu_quant, tests/e2e/nightly/single_node/ops/singlecard_ops/
    test_gmm_swiglu_quant_weight_nz_tensor_list.py:14-55 (channel scale first, sigmoid form, 127/max)."""
    c = (x.astype(np.int64) @ w_kn.astype(np.int64)).astype(np.float32)
    c = c * per_channel[None, :]
    c = c * per_token[:, None]
    a, gate = np.split(c, 2, axis=-1)
    a = a * (1.0 / (1.0 + np.exp(-a.astype(np.float64)))).astype(np.float32)
    y = a * gate
    mx = np.abs(y).max(axis=-1)
    qscale = 127.0 / mx
    q = np.round(y * qscale[:, None]).astype(np.int8)
    return q, (1.0 / qscale).astype(np.float32)


def test_gate_up_epilogue_against_the_reference_golden():
    """Shapes scaled down from the reference case (M=8192,K=7168,E=4,N=4096); same value ranges and the
    reference's tolerances: int8 +-1, scale rtol 1e-6 (test file :135-136)."""
    c = KATS["gmm_swiglu_quant_case"]
    rng = np.random.RandomState(0)
    M, K, E, N = 256, 512, 4, 256
    x = rng.randint(-128, 127, size=(M, K)).astype(np.int8)
    w = rng.randint(-128, 127, size=(E, K, N)).astype(np.int8)  # reference layout [E,K,N]
    ws = (rng.rand(E, N) * 0.9 + 0.1).astype(np.float32)
    xs = (rng.rand(M) * 0.9 + 0.1).astype(np.float32)
    cum = np.array([64, 128, 192, 256], dtype=np.int64)
    acc = orc.gmm_i32(x, np.ascontiguousarray(w.transpose(0, 2, 1)), cum)
    q, s = orc.swiglu_quant(orc.dequant_acc(acc, xs, ws, cum))
    for e in range(E):
        lo, hi = e * 64, (e + 1) * 64
        qg, sg = golden_gmm_swiglu_quant(x[lo:hi], w[e], ws[e], xs[lo:hi])
        assert np.max(np.abs(q[lo:hi].astype(np.int32) - qg.astype(np.int32))) <= c["int8_atol"]
        assert np.allclose(s[lo:hi], sg, rtol=c["scale_rtol"], atol=1e-9)


def test_swiglu_quant_closed_forms():
    # gate 0 -> silu 0 -> y 0 ; large gate -> silu(g) = g ; clamp
    f = np.array([[0.0, 100.0, -100.0, 2.0, 3.0, 5.0, 7.0, 11.0]], dtype=np.float32)  # I = 4
    q, s, y = orc.swiglu_quant(f, want_y=True)
    assert y[0, 0] == 0.0 and y[0, 1] == 500.0 and abs(y[0, 2]) < 1e-35  # exp argument clamps at 88.7
    assert np.isclose(y[0, 3], 2.0 / (1.0 + np.exp(-2.0)) * 11.0, rtol=1e-6)
    assert s[0] == np.float32(500.0) / np.float32(127.0) and q[0, 1] == 127
    q2, s2, y2 = orc.swiglu_quant(f, swiglu_limit=4.0, want_y=True)
    # gate 100 clamped to 4, up 5 clamped to 4: silu(4) * 4
    assert np.isclose(y2[0, 1], 4.0 / (1.0 + np.exp(-4.0)) * 4.0, rtol=1e-6)
    assert np.isclose(y2[0, 3], 2.0 / (1.0 + np.exp(-2.0)) * 4.0, rtol=1e-6)  # up 11 clamped to 4
    # all-zero row
    q3, s3 = orc.swiglu_quant(np.zeros((1, 8), np.float32))
    assert s3[0] == 0 and not q3.any()


def test_silu_against_float64_and_closed_forms():
    """orc_silu pinned outside itself: the float64 quotient on a dense grid, the exact regions, the SwiGLU stage."""
    g = np.concatenate([np.linspace(-87.0, 20.0, 200001), np.linspace(-1e-3, 1e-3, 2001)]).astype(np.float32)
    got = orc.silu(g).astype(np.float64)
    g64 = g.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64))
    ulp = np.spacing(np.abs(want).astype(np.float32)).astype(np.float64)
    # exp() is within 2 units (its own pin), 1 + E and the quotient add half a unit each
    assert np.all(np.abs(got - want) <= 3.0 * ulp)
    # 1 + exp(-g) rounds to 1 from g = 17.33 on (exp(-g) < 2^-25): the quotient is g itself
    big = np.array([17.4, 18.0, 100.0, 1e10, 3e38], dtype=np.float32)
    assert np.array_equal(orc.silu(big), big)
    z = orc.silu(np.array([0.0, -0.0], dtype=np.float32))
    assert z[0] == 0.0 and z[1] == 0.0 and not np.signbit(z[0]) and np.signbit(z[1])
    # far negative: the divisor stays finite (the exponential's argument is clamped at 88.72283)
    far = orc.silu(np.array([-90.0, -1e30], dtype=np.float32))
    assert np.all(np.isfinite(far)) and np.all(far < 0)
    # the SwiGLU stage with up = 1 returns exactly these values
    gates = np.linspace(-30.0, 30.0, 64).astype(np.float32)
    f = np.concatenate([gates, np.ones_like(gates)])[None, :]
    _, _, y = orc.swiglu_quant(f, want_y=True)
    assert np.array_equal(y[0], orc.silu(gates))


def test_token_scale_is_applied_before_the_channel_scale():
    """csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:387-399 then :448-459.
    Chosen so that the two orders differ in the last bit."""
    acc = np.array([[16777217]], dtype=np.int32)  # 2^24 + 1: float(acc) rounds to 2^24 (RNE)
    sx = np.array([np.float32(1.0 / 3.0)])
    sw = np.array([[np.float32(3.0)]])
    f = orc.dequant_acc(acc, sx, sw, np.array([1], dtype=np.int64))
    a = np.float32(16777216.0)
    assert f[0, 0] == np.float32(np.float32(a * sx[0]) * sw[0, 0])


# ------------------------------------------------------------------ down GEMM dequant, combine
def test_gmm2_dequant_against_float64():
    rng = np.random.RandomState(4)
    R, E, N = 40, 4, 64
    acc = rng.randint(-2 ** 22, 2 ** 22, size=(R, N)).astype(np.int32)
    s1 = (rng.rand(R) * 0.05).astype(np.float32)
    s2 = (rng.rand(E, N) * 0.01).astype(np.float32)
    cum = np.array([10, 10, 25, 40], dtype=np.int64)
    o = orc.bf16_to_f32(orc.gmm2_dequant(acc, s1, s2, cum))
    e_of = np.searchsorted(cum, np.arange(R), side="right")
    ref = acc.astype(np.float64) * s1[:, None].astype(np.float64) * s2[e_of].astype(np.float64)
    assert np.allclose(o, ref, rtol=2 ** -8, atol=0)


def test_unpermute_against_a_dense_reference():
    """Restates torch_moe (tests/e2e/nightly/single_node/ops/singlecard_ops/test_fused_moe.py:85-97):
    out[t] = sum_j w[t,j] * expert_out(t, j)."""
    rng = np.random.RandomState(5)
    T, k, H = 12, 4, 32
    R = T * k
    o = bf16(rng.normal(size=(R, H)).astype(np.float32))
    w = bf16(rng.rand(T, k).astype(np.float32))
    dst = rng.permutation(R).astype(np.int32)
    out = orc.bf16_to_f32(orc.unpermute(o, dst, w))
    of, wf = orc.bf16_to_f32(o).astype(np.float64), orc.bf16_to_f32(w).astype(np.float64)
    ref = (of[dst.reshape(T, k)] * wf[:, :, None]).sum(axis=1)
    assert np.allclose(out, ref, rtol=2 ** -7, atol=1e-6)
    # weight 1, k = 1 is a pure gather; negative indices are taken by magnitude
    ones = bf16(np.ones((R, 1), np.float32))
    g = orc.unpermute(o, -dst, ones)
    assert np.array_equal(g, o[dst])
    # exact small case: slot order matters in fp32
    o2 = bf16(np.array([[2.0 ** 24], [1.0], [-(2.0 ** 24)]], dtype=np.float32))
    w2 = bf16(np.ones((1, 3), np.float32))
    assert orc.bf16_to_f32(orc.unpermute(o2, np.array([0, 1, 2], np.int32), w2))[0, 0] == 0.0  # (2^24+1)-2^24 -> 0
    assert orc.bf16_to_f32(orc.unpermute(o2, np.array([0, 2, 1], np.int32), w2))[0, 0] == 1.0


def test_unpermute_residual_is_added_last_in_fp32():
    """The shared-expert output joins the sum after the k routed rows and before the one rounding to bf16."""
    one = bf16(np.ones((1, 2), np.float32))
    idx = np.array([0, 1], np.int32)

    def run(o_vals, add_val, w=one, index=idx):
        o = bf16(np.array(o_vals, np.float32).reshape(-1, 1))
        add = bf16(np.array([[add_val]], np.float32))
        return float(orc.bf16_to_f32(orc.unpermute(o, index, w, add))[0, 0])

    # exact small integers
    assert run([3.0, 4.0], 5.0) == 12.0
    # one rounding at the end: 1 + 2^-8 is a bf16 tie (-> 1.0); with the residual 2^-8 the fp32 sum 1 + 2^-7 is
    # representable.  Rounding before the add would give bf16(1 + 2^-8) + 2^-8 -> 1.0
    assert run([1.0, 2.0 ** -8], 2.0 ** -8) == 1.0 + 2.0 ** -7
    # added last: (2^24 - 2^24) + 1 = 1; added first, 1 + 2^24 rounds to 2^24 in fp32 and the result is 0
    assert run([2.0 ** 24, -(2.0 ** 24)], 1.0) == 1.0
    # the residual is not scaled by a routing weight
    half = bf16(np.full((1, 2), 0.5, np.float32))
    assert run([2.0, 4.0], 7.0, w=half) == 10.0
    # a skipped row (index one past the end) leaves only the others and the residual
    assert run([2.0, 4.0], 7.0, index=np.array([1, 2], np.int32)) == 11.0


def test_dequant_swiglu_quant_activates_the_right_half_when_asked():
    """activate_left = False: the SiLU goes on the right half, the left half is the linear factor
    (csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant_dynamic_base.hpp:86-91 swaps the two offsets)."""
    rng = np.random.RandomState(8)
    rows, n = 7, 192
    x = rng.randint(-100, 100, size=(rows, n)).astype(np.int32)
    ws = (rng.normal(size=n) * 0.1).astype(np.float32)
    a = (rng.normal(size=rows) * 0.5).astype(np.float32)
    q, s = orc.dequant_swiglu_quant(x, ws, a, activate_left=False)
    # numpy rendering of the golden with the halves exchanged
    gu = x.astype(np.float32) * ws[None, :] * a[:, None]
    u, g = gu[:, : n // 2].astype(np.float64), gu[:, n // 2:].astype(np.float64)
    y = (g / (1 + np.exp(-g)) * u).astype(np.float32)
    assert np.allclose(s, np.abs(y).max(axis=1) / 127.0, rtol=1e-5)
    assert np.max(np.abs(q - np.round(y / s[:, None]))) <= 1
    # identity: exchanging the halves of x and of the weight scale turns it into the default op, bit for bit
    swap = np.concatenate([np.arange(n // 2, n), np.arange(n // 2)])
    q2, s2 = orc.dequant_swiglu_quant(np.ascontiguousarray(x[:, swap]), ws[swap], a, activate_left=True)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    # and it is not the default op
    q3, _ = orc.dequant_swiglu_quant(x, ws, a, activate_left=True)
    assert not np.array_equal(q, q3)


def test_shared_expert_against_a_dense_float64_mlp():
    """The dense W8A8 MLP of the shared expert (op order of vllm_ascend/ops/fused_moe/shared_experts.py:254-301)
    against silu(x W1^T) * (x W3^T) W2^T on the dequantised weights in float64: they differ by the noise of the two
    activation quantisations only.  With power-of-two weight scales the order of the two scale multiplications
    cannot matter, and the result must equal the routed path run with one expert that owns every token."""
    rng = np.random.RandomState(21)
    T, H, I = 24, 256, 128
    x = bf16(rng.normal(size=(T, H)).astype(np.float32))
    w13 = rng.randint(-127, 128, size=(2 * I, H)).astype(np.int8)
    w2 = rng.randint(-127, 128, size=(H, I)).astype(np.int8)
    s13 = (rng.rand(2 * I) * 0.009 + 0.001).astype(np.float32)
    s2 = (rng.rand(H) * 0.009 + 0.001).astype(np.float32)
    got = orc.bf16_to_f32(orc.shared_expert_forward(x, w13, s13, w2, s2)).astype(np.float64)
    xf = orc.bf16_to_f32(x).astype(np.float64)
    gu = xf @ (w13.astype(np.float64) * s13[:, None].astype(np.float64)).T
    g, u = gu[:, :I], gu[:, I:]
    ref = (g / (1 + np.exp(-g)) * u) @ (w2.astype(np.float64) * s2[:, None].astype(np.float64)).T
    err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    assert err <= 5e-2, err
    # a dropped term, a transposed weight or a missing scale is far outside that: e.g. without the SiLU
    wrong = (g * u) @ (w2.astype(np.float64) * s2[:, None].astype(np.float64)).T
    assert np.linalg.norm(got - wrong) / np.linalg.norm(wrong) > 0.3
    # one expert, top-1, weight 1: the routed path is the same MLP
    p13 = (2.0 ** rng.randint(-10, -6, size=2 * I)).astype(np.float32)
    p2 = (2.0 ** rng.randint(-10, -6, size=H)).astype(np.float32)
    sh = orc.shared_expert_forward(x, w13, p13, w2, p2)
    ids = np.zeros((T, 1), np.int32)
    tr = orc.experts_forward(x, bf16(np.ones((T, 1), np.float32)), ids, w13[None], p13[None], w2[None], p2[None])
    assert np.array_equal(tr.o, sh) and np.array_equal(tr.out, sh)


def golden_dequant_swiglu_quant(x, w_scale, a_scale):
    """numpy rendering of _shared_dequant_swiglu_quant (test_dequant_swiglu_quant.py:16-45) up to the
    SwiGLU values (the golden then calls the closed npu_dynamic_quant on a bf16 copy)."""
    gu = x.astype(np.float32) * w_scale[None, :] * a_scale[:, None]
    half = gu.shape[-1] // 2
    g, u = gu[:, :half].astype(np.float64), gu[:, half:].astype(np.float64)
    return (g / (1 + np.exp(-g)) * u).astype(np.float32)


@pytest.mark.parametrize("shape", KATS["dequant_swiglu_quant_shapes"]["shapes"][1:])
def test_dequant_swiglu_quant_against_the_reference_golden(shape):
    rng = np.random.RandomState(shape[0])
    x = rng.randint(-100, 100, size=shape).astype(np.int32)
    ws = (rng.normal(size=shape[1]) * 0.1).astype(np.float32)
    a = (rng.normal(size=shape[0]) * 0.5).astype(np.float32)
    q, s = orc.dequant_swiglu_quant(x, ws, a)
    y = golden_dequant_swiglu_quant(x, ws, a)
    assert np.allclose(s, np.abs(y).max(axis=1) / 127.0, rtol=1e-5)
    assert np.max(np.abs(q - np.round(y / s[:, None]))) <= 1


# ------------------------------------------------------------------ W4A8 integer stage
def test_w4_grouped_against_the_reference_golden():
    """custom_mm per-group branch of test_grouped_matmul_swiglu_quant.py:22-55, in fp32."""
    rng = np.random.RandomState(6)
    M, K, N, E, g = 16, 512, 32, 2, 256
    x = rng.randint(-128, 128, size=(M, K)).astype(np.int8)
    w = rng.randint(-8, 8, size=(E, N, K)).astype(np.int8)
    sg = rng.normal(size=(E, K // g, N)).astype(np.float32)
    cum = np.array([10, 16], dtype=np.int64)
    f = orc.gmm_w4_grouped(x, w, sg, cum, g)
    for e, (lo, hi) in enumerate([(0, 10), (10, 16)]):
        xg = x[lo:hi].reshape(hi - lo, K // g, g).astype(np.int64)
        wg = w[e].reshape(N, K // g, g).astype(np.int64)
        part = np.einsum("mgk,ngk->gmn", xg, wg).astype(np.float64)
        ref = (part * sg[e][:, None, :].astype(np.float64)).sum(axis=0)
        assert np.allclose(f[lo:hi], ref, rtol=1e-5, atol=1e-3)


# ------------------------------------------------------------------ whole layer
def test_layer_matches_the_dense_reference_within_quantisation_noise():
    import sys

    sys.path.insert(0, os.path.dirname(__file__))
    from _inputs import CONFIGS, bits, make_layer
    from _layer_utils import oracle_layer, rel_err

    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=0)
    tr = oracle_layer(cfg, d)
    got = orc.bf16_to_f32(tr.out)
    ref = orc.fp32_dequant_reference(bits(d["x"]), tr.topk_weights, tr.topk_ids, d["w13"].numpy(), d["s13"].numpy(),
                                     d["w2"].numpy(), d["s2"].numpy())
    assert rel_err(got, ref) <= 5e-2
    assert rel_err(got, orc.quantized_fp64_reference(tr, d["s2"].numpy())) <= 1e-2
    # linearity of the combine in the routing weights: doubling every weight doubles the output exactly
    w2 = orc.f32_to_bf16(orc.bf16_to_f32(tr.topk_weights) * 2)
    out2 = orc.unpermute(tr.o, tr.expanded_row_idx, w2)
    assert np.array_equal(orc.bf16_to_f32(out2), orc.bf16_to_f32(tr.out) * 2)


def test_w4_sum_over_groups_runs_in_ascending_group_order():
    """f = ((0 + t_0) + t_1) + t_2 in fp32.  With t = (2^24, 1, 1) the ascending order loses both ones
    (2^24 + 1 ties back to 2^24, twice); any order that adds the ones first gives 2^24 + 2.  Pins the order
    that the int4 kernel must reproduce."""
    K, g, N = 192, 64, 32
    x = np.zeros((1, K), dtype=np.int8)
    w = np.zeros((1, N, K), dtype=np.int8)
    for grp in range(3):
        x[0, 64 * grp] = 1
        w[0, :, 64 * grp] = 1   # every group's integer sum is 1
    one = np.array([1], dtype=np.int64)
    sg = np.zeros((1, 3, N), dtype=np.float32)
    sg[0, :, :] = np.array([2.0 ** 24, 1.0, 1.0], dtype=np.float32)[:, None]
    assert np.all(orc.gmm_w4_grouped(x, w, sg, one, g) == np.float32(2.0 ** 24))
    sg[0, :, :] = np.array([1.0, 1.0, 2.0 ** 24], dtype=np.float32)[:, None]
    assert np.all(orc.gmm_w4_grouped(x, w, sg, one, g) == np.float32(2.0 ** 24 + 2))
    sg[0, :, :] = np.array([3.0, 0.0, 2.0 ** 24], dtype=np.float32)[:, None]
    assert np.all(orc.gmm_w4_grouped(x, w, sg, one, g) == np.float32(2.0 ** 24 + 4))  # 2^24 + 3 rounds to even


def test_w4_stage_extremes_and_empty_groups():
    """Largest magnitudes (x = -128, w = -8 everywhere) stay exact integers in the int32 group sums; rows past
    the last group stay zero; an empty expert changes nothing."""
    K, g, N = 256, 128, 32
    x = np.full((3, K), -128, dtype=np.int8)
    w = np.full((2, N, K), -8, dtype=np.int8)
    sg = np.ones((2, K // g, N), dtype=np.float32)
    f = orc.gmm_w4_grouped(x, w, sg, np.array([0, 2], dtype=np.int64), g)   # expert 0 empty, row 2 unowned
    assert np.all(f[:2] == np.float32(128 * 8 * K)) and np.all(f[2] == 0)
    o = orc.w4_rows_to_bf16(f, np.array([0.5, 0.0, 1.0], dtype=np.float32))
    assert np.all(orc.bf16_to_f32(o[0]) == 128 * 8 * K / 2) and np.all(o[1] == 0) and np.all(o[2] == 0)


def test_w4_layer_matches_a_dense_float64_rendering():
    import sys

    sys.path.insert(0, os.path.dirname(__file__))
    from _inputs import CONFIGS, bits, make_layer
    from _layer_utils import oracle_layer, rel_err

    cfg = CONFIGS["c5_small"]
    d = make_layer(cfg, seed=0)
    tr = oracle_layer(cfg, d)
    # the same quantised pipeline in float64 from the traced int8 activations: no fp32 or bf16 rounding
    g = cfg.w4_group
    sg2 = d["s2"].numpy().transpose(0, 2, 1)   # [E, G, N]
    cum = np.cumsum(tr.expert_tokens)
    o = np.zeros((tr.q1.shape[0], cfg.H), dtype=np.float64)
    lo = 0
    for e, hi in enumerate(cum):
        if hi > lo:
            q = tr.q1[lo:hi].astype(np.float64).reshape(hi - lo, -1, g)
            w = d["w2"].numpy()[e].astype(np.float64).reshape(cfg.H, -1, g)
            part = np.einsum("mgk,ngk->gmn", q, w)
            o[lo:hi] = (part * sg2[e][:, None, :]).sum(axis=0) * tr.s1[lo:hi, None].astype(np.float64)
        lo = hi
    assert rel_err(orc.bf16_to_f32(tr.o), o) <= 1e-2


# ------------------------------------------------------------------ static quantisation mode, other activations
def test_dequant_swiglu_quant_static_against_numpy():
    """quant_mode 0 (dequant_swiglu_quant_static_base.hpp:266-305): y / scale[c] + offset[c] per channel,
    y * (1 / scale) + offset per tensor, one rounding, saturation."""
    rng = np.random.RandomState(3)
    rows, N = 6, 192
    x = rng.randint(-100, 100, size=(rows, N)).astype(np.int32)
    ws = (rng.randn(N) * 0.1).astype(np.float32)
    as_ = (rng.randn(rows) * 0.5).astype(np.float32)
    # the SwiGLU values of the dynamic mode are the ones that get quantised
    f = (x.astype(np.float32) * ws[None, :]) * as_[:, None]
    _, _, y = orc.swiglu_quant(f, want_y=True)
    qs = (rng.rand(N // 2) * 0.05 + 0.01).astype(np.float32)
    qo = (rng.randn(N // 2) * 3).astype(np.float32)
    for scale, off in ((qs, qo), (qs, None), (qs[:1], qo[:1]), (qs[:1], None)):
        got = orc.dequant_swiglu_quant_static(x, ws, as_, scale, off)
        o = np.float32(0) if off is None else off
        if scale.size == 1:
            v = y * (np.float32(1.0) / scale[0]) + (o if off is None else o[0])
        else:
            v = y / scale[None, :] + (o if off is None else o[None, :])
        want = np.clip(np.rint(v.astype(np.float32)), -128, 127).astype(np.int8)
        assert np.array_equal(got, want)
    # saturation both ways
    big = orc.dequant_swiglu_quant_static(x, ws, as_, np.array([1e-6], dtype=np.float32))
    assert big.max() == 127 and big.min() == -128
    # activate_left = False: the halves swap roles
    swapped = np.concatenate([x[:, N // 2:], x[:, :N // 2]], axis=1)
    ws_sw = np.concatenate([ws[N // 2:], ws[:N // 2]])
    assert np.array_equal(orc.dequant_swiglu_quant_static(swapped, ws_sw, as_, qs, qo, activate_left=False),
                          orc.dequant_swiglu_quant_static(x, ws, as_, qs, qo))


def test_erf_and_tanh_against_libm():
    import math

    xs = np.linspace(-6.0, 6.0, 4801).astype(np.float32)
    e = orc.erff(xs).astype(np.float64)
    t = orc.tanhf(xs).astype(np.float64)
    assert np.max(np.abs(e - np.array([math.erf(float(v)) for v in xs]))) <= 5e-7
    assert np.max(np.abs(t - np.tanh(xs.astype(np.float64)))) <= 3e-7
    assert np.array_equal(orc.erff(-xs), -orc.erff(xs))          # odd by construction (copysign)
    assert orc.erff(np.array([0.0, 10.0, -10.0], dtype=np.float32)).tolist() == [0.0, 1.0, -1.0]
    assert orc.tanhf(np.array([50.0, -50.0], dtype=np.float32)).tolist() == [1.0, -1.0]


@pytest.mark.parametrize("act", ["gelu", "gelu_tanh", "swiglustep", "swigluoai"])
@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_activation_and_quantisation_against_float64(act, kind):
    """The unfused activations (moe_mlp.py:484-549) against their float64 formulas: values within the rounding of
    the 16-bit result, then exactly the dynamic quantiser's rule on those rounded values."""
    import math

    rng = np.random.RandomState(11)
    rows, I = 5, 96
    limit, alpha, beta = (7.0, 1.0, 0.0) if act == "swiglustep" else ((3.0, 1.702, 1.0) if act == "swigluoai" else (0.0, 1.0, 0.0))
    with orc.half_kind(kind):
        h = orc.f32_to_half((rng.randn(rows, 2 * I) * 4).astype(np.float32))
        hf = orc.half_to_f32(h).astype(np.float64)
        q, s = orc.act_mul_quant(h, act, limit, alpha, beta)
        g, u = hf[:, :I], hf[:, I:]
        if act == "gelu":
            y = 0.5 * g * (1 + np.vectorize(math.erf)(g / math.sqrt(2))) * u
        elif act == "gelu_tanh":
            y = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))) * u
        elif act == "swiglustep":
            y = np.minimum(g / (1 + np.exp(-g)), limit) * np.clip(u, -limit, limit)
        else:
            gc, uc = np.minimum(g, limit), np.clip(u, -limit, limit)
            y = gc / (1 + np.exp(-alpha * gc)) * (uc + beta)
        y16 = orc.half_to_f32(orc.f32_to_half(y.astype(np.float32))).astype(np.float64)
        # rebuild what the checker quantised: q * s must be within half a step of a 16-bit value near y
        amax = np.abs(y16).max(axis=1)
        assert np.allclose(s, amax / 127.0, rtol=2e-2)  # the row maximum may round to a neighbouring 16-bit value
        ulp16 = 2.0 ** (-7 if kind == "bf16" else -10)
        assert np.all(np.abs(q.astype(np.float64) * s[:, None] - y) <= 0.5 * s[:, None] + np.abs(y) * ulp16 + 2e-6)
        assert np.abs(q).max(axis=1).tolist() == [127] * rows
    # an all-zero row: zeros and a zero scale
    with orc.half_kind(kind):
        qz, sz = orc.act_mul_quant(np.zeros((1, 8), dtype=np.uint16), act, limit, alpha, beta)
        assert not qz.any() and sz[0] == 0.0


def test_layer_with_other_activations_matches_a_dense_float64_rendering():
    """experts_forward(activation=...) end to end against the dense float64 layer with that activation, within the
    quantisation noise (the same bound as the SiLU layer)."""
    import math

    from _inputs import CONFIGS, bits, make_layer

    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=0)
    y, ids, _ = orc.gating_top_k(d["logits"].numpy(), cfg.k, renorm=1, norm_type=0, x_dtype="f32")
    w = orc.f32_to_half(y)
    for act in ("gelu", "gelu_tanh", "swiglustep", "swigluoai"):
        limit, alpha, beta = (7.0, 1.0, 0.0) if act == "swiglustep" else ((7.0, 1.702, 1.0) if act == "swigluoai" else (0.0, 1.0, 0.0))
        tr = orc.experts_forward(bits(d["x"]), w, ids, d["w13"].numpy(), d["s13"].numpy(), d["w2"].numpy(),
                                 d["s2"].numpy(), activation=act, swiglu_limit=limit, swiglu_alpha=alpha,
                                 swiglu_beta=beta)
        x = orc.half_to_f32(bits(d["x"])).astype(np.float64)
        wf = orc.half_to_f32(w).astype(np.float64)
        ref = np.zeros((cfg.T, cfg.H))
        for e in np.unique(ids):
            tok, slot = np.nonzero(ids == e)
            gu = x[tok] @ (d["w13"][e].numpy().astype(np.float64) * d["s13"][e].numpy().astype(np.float64)[:, None]).T
            g, u = gu[:, :cfg.I], gu[:, cfg.I:]
            if act == "gelu":
                a = 0.5 * g * (1 + np.vectorize(math.erf)(g / math.sqrt(2))) * u
            elif act == "gelu_tanh":
                a = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))) * u
            elif act == "swiglustep":
                a = np.minimum(g / (1 + np.exp(-g)), limit) * np.clip(u, -limit, limit)
            else:
                gc, uc = np.minimum(g, limit), np.clip(u, -limit, limit)
                a = gc / (1 + np.exp(-alpha * gc)) * (uc + beta)
            o = a @ (d["w2"][e].numpy().astype(np.float64) * d["s2"][e].numpy().astype(np.float64)[:, None]).T
            np.add.at(ref, tok, o * wf[tok, slot][:, None])
        got = orc.half_to_f32(tr.out).astype(np.float64)
        err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
        assert err <= 5e-2, (act, err)


# ---- the grouped / swiglu_mode 1 form of dequant_swiglu_quant (csrc/moe/dequant_swiglu_quant/op_kernel/
# dequant_swiglu_quant.h): pinned from outside the C restatement
def _dsq_inputs(rows, n, groups, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(-2000, 2000, (rows, n), dtype=np.int32)
    ws = (rng.uniform(0.2, 2.0, (groups, n)) * 1e-3).astype(np.float32)
    a = rng.uniform(0.5, 2.0, rows).astype(np.float32)
    return rng, x, ws, a


def _np_dynamic_quant_of_the_grouped_kernel(v):
    """scale = max * float32(1 / 127); q = rint(v / scale), every step rounded to float32 (numpy)."""
    v = v.astype(np.float32)
    amax = np.abs(v).max(axis=1)
    s = (amax * np.float32(1.0 / 127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint((v / s[:, None]).astype(np.float32))
    q = np.where(amax[:, None] == 0, 0, np.clip(q, -128, 127)).astype(np.int8)
    return q, np.where(amax == 0, np.float32(0), s)


def test_grouped_dsq_with_one_group_is_the_plain_swiglu_through_its_own_quantiser():
    rng, x, ws, a = _dsq_inputs(400, 256, 1, 1)
    q, s = orc.dequant_swiglu_quant_grouped(x, ws, a)
    # the SwiGLU values of the plain op: same dequant order, same gate function (want_y of the fused epilogue's
    # restatement takes the dequantised fp32 values)
    f = ((x.astype(np.float32) * ws[0]).astype(np.float32) * a[:, None]).astype(np.float32)
    _, _, y = orc.swiglu_quant(f, 0.0, want_y=True)
    q_np, s_np = _np_dynamic_quant_of_the_grouped_kernel(y)
    assert np.array_equal(q, q_np) and np.array_equal(s.view(np.uint32), s_np.view(np.uint32))
    # no activation scale = a scale of ones
    q1, s1 = orc.dequant_swiglu_quant_grouped(x, ws, None)
    q2, s2 = orc.dequant_swiglu_quant_grouped(x, ws, np.ones(400, dtype=np.float32))
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)
    # the scale is max * (1/127), not max / 127: a row maximum where the two differ
    amax = np.abs(y).max(axis=1)
    differs = (amax * np.float32(1.0 / 127.0)).astype(np.float32) != (amax / np.float32(127.0)).astype(np.float32)
    assert differs.any()
    assert np.array_equal(s[differs], (amax * np.float32(1.0 / 127.0)).astype(np.float32)[differs])
    # right half activated = halves swapped
    swap = np.r_[128:256, 0:128]
    q3, s3 = orc.dequant_swiglu_quant_grouped(np.ascontiguousarray(x[:, swap]), ws[:, swap], a, activate_left=False)
    assert np.array_equal(q3, q) and np.array_equal(s3, s)


def test_grouped_dsq_groups_are_row_ranges_with_their_own_scales():
    counts = np.array([3, 0, 5, -2, 1, 0, 7], dtype=np.int64)     # negative counts are empty groups
    rows, n = 20, 192                                             # 16 rows in groups, 4 past the last group
    rng, x, ws, a = _dsq_inputs(rows, n, len(counts), 2)
    bias_i = rng.integers(-50, 50, (len(counts), n), dtype=np.int32)
    for kw in ({}, {"swiglu_mode": 1, "clamp_limit": 1.5, "glu_alpha": 1.702, "glu_bias": 1.0}):
        q, s = orc.dequant_swiglu_quant_grouped(x, ws, a, counts, **kw)
        qb, sb = orc.dequant_swiglu_quant_grouped(x, ws, a, counts, bias=bias_i, **kw)
        start = 0
        for g, c in enumerate(np.maximum(counts, 0)):
            sl = slice(start, start + c)
            q1, s1 = orc.dequant_swiglu_quant_grouped(x[sl], ws[g], a[sl], **kw)
            assert np.array_equal(q[sl], q1) and np.array_equal(s[sl], s1), g
            # an int32 bias is added to x before anything else
            q2, s2 = orc.dequant_swiglu_quant_grouped(x[sl] + bias_i[g], ws[g], a[sl], **kw)
            assert np.array_equal(qb[sl], q2) and np.array_equal(sb[sl], s2), g
            start += c
        assert start == 16 and not q[16:].any() and not s[16:].any()


def test_grouped_dsq_mode_one_formula_against_float64():
    rows, n = 64, 128
    rng, x, ws, a = _dsq_inputs(rows, n, 1, 3)
    bias_f = rng.standard_normal((1, n)).astype(np.float32)
    for limit, alpha, beta, bias in ((0.0, 1.0, 0.0, None), (1.25, 1.702, 1.0, None), (0.0, 0.5, -0.75, bias_f),
                                     (2.0, 1.0, 0.0, bias_f)):
        q, s = orc.dequant_swiglu_quant_grouped(x, ws, a, bias=bias, swiglu_mode=1, clamp_limit=limit,
                                                glu_alpha=alpha, glu_bias=beta)
        f = x.astype(np.float64) * ws[0].astype(np.float64) * a[:, None].astype(np.float64)
        if bias is not None:
            f = f + bias[0]
        act, lin = f[:, :64], f[:, 64:]
        if limit > 0:
            act = np.minimum(act, limit)
            lin = np.clip(lin, -limit, limit)
        v = (lin + beta) * act / (1.0 + np.exp(-alpha * act))
        amax = np.abs(v).max(axis=1)
        assert np.allclose(s, amax / 127.0, rtol=1e-5)
        assert np.abs(q.astype(np.float64) * s[:, None] - v).max() <= 0.5001 * s.max() + 1e-6, (limit, alpha, beta)
    # swiglu_mode 1 with alpha 1, beta 0 and no clamp is swiglu_mode 0; swiglu_mode 0 ignores all three
    base = orc.dequant_swiglu_quant_grouped(x, ws, a)
    same = orc.dequant_swiglu_quant_grouped(x, ws, a, swiglu_mode=1)
    ignored = orc.dequant_swiglu_quant_grouped(x, ws, a, swiglu_mode=0, clamp_limit=0.01, glu_alpha=3.0, glu_bias=5.0)
    for other in (same, ignored):
        assert np.array_equal(base[0], other[0]) and np.array_equal(base[1], other[1])


def test_grouped_dsq_static_mode_per_group_scales():
    counts = np.array([4, 2, 0, 6], dtype=np.int64)
    rows, n = 12, 64
    rng, x, ws, a = _dsq_inputs(rows, n, 4, 4)
    qs_g = rng.uniform(0.01, 0.05, 4).astype(np.float32)
    qo_g = rng.standard_normal(4).astype(np.float32)
    qs_c = rng.uniform(0.01, 0.05, (4, 32)).astype(np.float32)
    qo_c = rng.standard_normal((4, 32)).astype(np.float32)
    group_of_row = np.repeat(np.arange(4), counts)
    f = ((x.astype(np.float32) * ws[group_of_row]).astype(np.float32) * a[:, None]).astype(np.float32)
    _, _, y = orc.swiglu_quant(f, 0.0, want_y=True)
    got, _ = orc.dequant_swiglu_quant_grouped(x, ws, a, counts, quant_mode=0, quant_scale=qs_g, quant_offset=qo_g)
    inv = (np.float32(1.0) / qs_g).astype(np.float32)
    want = np.clip(np.rint((y * inv[group_of_row][:, None]).astype(np.float32) + qo_g[group_of_row][:, None]), -128, 127)
    assert np.array_equal(got, want.astype(np.int8))
    got, _ = orc.dequant_swiglu_quant_grouped(x, ws, a, counts, quant_mode=0, quant_scale=qs_c, quant_offset=qo_c)
    want = np.clip(np.rint((y / qs_c[group_of_row]).astype(np.float32) + qo_c[group_of_row]), -128, 127)
    assert np.array_equal(got, want.astype(np.int8))
    got, _ = orc.dequant_swiglu_quant_grouped(x, ws, a, counts, quant_mode=0, quant_scale=qs_c)
    assert np.array_equal(got, np.clip(np.rint((y / qs_c[group_of_row]).astype(np.float32)), -128, 127).astype(np.int8))
