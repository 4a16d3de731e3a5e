"""Pins for the checker's routing stage (CPU only).

The checker is compared with (1) a numpy rendering of the reference's golden
function over the reference's own parameter grid, (2) brute-force enumeration
on tiny inputs, (3) closed forms and tie cases.  None of these re-uses the
checker's code."""
import itertools
import json
import os

import numpy as np
import pytest

from oracle import oracle as orc

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def golden_numpy(x, k, bias, k_group, group_count, group_select_mode, renorm, norm_type, rsf=1.0, eps=1e-20):
    """numpy rendering of moe_gating_top_k_numpy_ref
    (tests/e2e/nightly/single_node/ops/singlecard_ops/test_npu_moe_gating_top_k.py:33-112)."""
    x = x.astype(np.float32)
    if norm_type == 0:
        e = np.exp(x - x.max(axis=-1, keepdims=True))
        x = e / e.sum(axis=-1, keepdims=True)
    else:
        x = 1 / (1 + np.exp(-x))
    original = x
    if bias is not None:
        x = x + bias.astype(np.float32)
    if group_count > 1:
        xg = x.reshape(x.shape[0], group_count, -1)
        if group_select_mode == 0:
            gx = np.amax(xg, axis=-1)
        else:
            gx = np.partition(xg, -2, axis=-1)[..., -2:].sum(axis=-1)
        gi = np.argsort(-gx, axis=-1, kind="stable")[:, :k_group]
        mask = np.ones((x.shape[0], group_count), dtype=bool)
        mask[np.arange(x.shape[0])[:, None], gi] = False
        x = np.where(mask[..., None], -np.inf, xg).reshape(x.shape[0], -1)
    idx = np.argsort(-x, axis=-1, kind="stable")[:, :k]
    y = np.take_along_axis(original, idx, axis=1)
    if norm_type == 1 or renorm == 1:
        y = y / (y.sum(axis=-1, keepdims=True) + eps)
    y = y * rsf
    return y.astype(np.float32), idx.astype(np.int32)


def _grid():
    g = KATS["gating_grid"]
    for mode, norm_type, G, k, T, E in itertools.product(g["group_select_mode"], g["norm_type"], g["group_count"],
                                                         g["k"], g["rows"], g["experts"]):
        if k > E // G:
            continue  # the reference test skips these
        yield mode, norm_type, G, k, T, E


def test_reference_grid():
    g = KATS["gating_grid"]
    rng = np.random.RandomState(g["seed"])
    n = 0
    for mode, norm_type, G, k, T, E in _grid():
        x = rng.uniform(-2, 2, (T, E)).astype(np.float32)
        bias = rng.uniform(-2, 2, (E,)).astype(np.float32)
        k_group = min(1, G)
        y_ref, idx_ref = golden_numpy(x, k, bias, k_group, G, mode, 1, norm_type)
        y, idx, _ = orc.gating_top_k(x, k, bias=bias, k_group=k_group, group_count=G, group_select_mode=mode,
                                     renorm=1, norm_type=norm_type)
        assert np.array_equal(idx, idx_ref), (mode, norm_type, G, k, T, E)
        assert np.allclose(y, y_ref, rtol=g["rtol"], atol=g["atol"])
        n += 1
    assert n > 50


@pytest.mark.parametrize("norm_type", [0, 1])
@pytest.mark.parametrize("mode", [0, 1])
def test_multi_group_grid(norm_type, mode):
    """k_group > 1 (the reference grid fixes k_group = 1; DeepSeek-V3 uses 4 of 8)."""
    rng = np.random.RandomState(7)
    for T, E, G, k_group, k in [(9, 256, 8, 4, 8), (4, 64, 4, 2, 6), (3, 128, 16, 5, 8)]:
        x = rng.uniform(-2, 2, (T, E)).astype(np.float32)
        bias = rng.normal(0, 0.01, (E,)).astype(np.float32)
        y_ref, idx_ref = golden_numpy(x, k, bias, k_group, G, mode, 0, norm_type, rsf=2.5)
        y, idx, _ = orc.gating_top_k(x, k, bias=bias, k_group=k_group, group_count=G, group_select_mode=mode,
                                     renorm=0, norm_type=norm_type, routed_scaling_factor=2.5)
        assert np.array_equal(idx, idx_ref)
        assert np.allclose(y, y_ref, rtol=1e-5, atol=1e-8)


def test_brute_force_tiny():
    """Enumerate every admissible choice on tiny inputs: the selected groups maximise
    the total group score, the selected experts maximise the total biased score."""
    rng = np.random.RandomState(3)
    E, G, k_group, k = 8, 4, 2, 3
    gs = E // G
    for trial in range(40):
        x = rng.uniform(-2, 2, (1, E)).astype(np.float32)
        bias = rng.uniform(-1, 1, (E,)).astype(np.float32)
        y, idx, norm = orc.gating_top_k(x, k, bias=bias, k_group=k_group, group_count=G, group_select_mode=1,
                                        renorm=0, norm_type=1, want_norm=True)
        sel = (norm[0] + bias).astype(np.float64)
        gscore = np.sort(sel.reshape(G, gs), axis=1)[:, -2:].sum(axis=1)
        best_groups = max(itertools.combinations(range(G), k_group), key=lambda c: sum(gscore[list(c)]))
        allowed = [g * gs + j for g in best_groups for j in range(gs)]
        best = max(itertools.combinations(allowed, k), key=lambda c: sum(sel[list(c)]))
        assert sorted(idx[0].tolist()) == sorted(best)
        # descending biased score, weights are the UNBIASED sigmoid scores
        assert all(sel[idx[0][i]] >= sel[idx[0][i + 1]] for i in range(k - 1))
        ysum = norm[0][idx[0]].sum()
        assert np.allclose(y[0], norm[0][idx[0]] / (ysum + 1e-20), rtol=1e-6)


def test_closed_forms():
    rng = np.random.RandomState(11)
    x = rng.normal(0, 1, (5, 128)).astype(np.float32)
    y, idx, norm = orc.gating_top_k(x, 8, renorm=1, norm_type=0, want_norm=True)
    assert np.allclose(norm.sum(axis=1), 1.0, atol=1e-6)  # softmax rows sum to one
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-6)  # renormalised weights sum to one
    y2, idx2, _ = orc.gating_top_k(x, 8, renorm=0, norm_type=0, routed_scaling_factor=3.0)
    assert np.array_equal(idx, idx2)
    assert np.allclose(y2, 3.0 * np.take_along_axis(norm, idx, 1), rtol=1e-6)
    # sigmoid(0) = 1/2 exactly; all-equal scores -> lowest indices, equal weights
    z = np.zeros((2, 64), dtype=np.float32)
    y3, idx3, n3 = orc.gating_top_k(z, 4, renorm=0, norm_type=1, want_norm=True)
    assert np.all(n3 == 0.5)
    assert idx3.tolist() == [[0, 1, 2, 3]] * 2
    assert np.all(y3 == 0.25)
    # softmax of equal logits: 1/E each; ties go to the lower index
    y4, idx4, n4 = orc.gating_top_k(z, 4, renorm=1, norm_type=0, want_norm=True)
    assert np.allclose(n4, 1 / 64, rtol=1e-6) and idx4.tolist() == [[0, 1, 2, 3]] * 2
    # bias changes the selection but not the weights
    b = np.zeros(64, dtype=np.float32)
    b[[60, 61]] = 1.0
    y5, idx5, _ = orc.gating_top_k(z, 2, bias=b, renorm=0, norm_type=1)
    assert idx5.tolist() == [[60, 61]] * 2 and np.all(y5 == 0.5)  # sigmoid always divides by the sum: 0.5/(1+eps)


def test_group_mask_ties_and_order():
    # two groups with equal scores: the lower group index wins
    x = np.array([[1, 0, 1, 0, 0.5, 0.5, 0.2, 0.1]], dtype=np.float32)
    _, idx, _ = orc.gating_top_k(x, 2, k_group=1, group_count=4, group_select_mode=0, renorm=1, norm_type=1)
    assert idx.tolist() == [[0, 1]]
    # sum-of-top-2 prefers group 2 (0.5+0.5 in sigmoid space beats 1+0)
    _, idx, norm = orc.gating_top_k(x * 4, 2, k_group=1, group_count=4, group_select_mode=1, renorm=1, norm_type=1,
                                    want_norm=True)
    assert idx.tolist() == [[4, 5]]


def test_low_precision_inputs():
    rng = np.random.RandomState(5)
    x = rng.uniform(-2, 2, (6, 128)).astype(np.float32)
    xb = orc.f32_to_bf16(x)
    y, idx, _ = orc.gating_top_k(xb, 8, renorm=1, norm_type=0, x_dtype="bf16")
    y_ref, idx_ref = golden_numpy(orc.bf16_to_f32(xb), 8, None, 1, 1, 1, 1, 0)
    assert np.array_equal(idx, idx_ref)
    assert np.allclose(orc.bf16_to_f32(y), y_ref, rtol=2 ** -8)
    xh = x.astype(np.float16)
    y, idx, _ = orc.gating_top_k(xh.view(np.uint16), 8, renorm=1, norm_type=0, x_dtype="f16")
    y_ref, idx_ref = golden_numpy(xh.astype(np.float32), 8, None, 1, 1, 1, 1, 0)
    assert np.array_equal(idx, idx_ref)
    assert np.array_equal(y.view(np.float16), y_ref.astype(np.float16)) or np.allclose(
        y.view(np.float16).astype(np.float32), y_ref, rtol=2 ** -10)


def test_argument_errors():
    x = np.zeros((1, 8), dtype=np.float32)
    with pytest.raises(ValueError):
        orc.gating_top_k(x, 9)
    with pytest.raises(ValueError):
        orc.gating_top_k(x, 2, group_count=3)


def test_expf_against_libm():
    xs = np.concatenate([np.linspace(-87, 88.7, 20001), np.linspace(-1, 1, 4001), [0.0, -0.0, 1e-10, -1e-10]]).astype(
        np.float32)
    got = orc.expf(xs).astype(np.float64)
    ref = np.exp(xs.astype(np.float64))
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - ref) / ulp) <= 2.0
    assert orc.expf(np.array([0.0], np.float32))[0] == 1.0
    # the argument is clamped to [-87, 88.72283]; NaN counts as the lower clamp
    lo = orc.expf(np.array([-87.0], np.float32))[0]
    hi = orc.expf(np.array([88.72283], np.float32))[0]
    assert lo > 0 and np.isclose(lo, np.exp(-87.0), rtol=1e-6) and lo >= np.finfo(np.float32).tiny
    assert orc.expf(np.array([-200.0, -np.inf, np.nan], np.float32)).tolist() == [lo, lo, lo]
    assert orc.expf(np.array([100.0, np.inf], np.float32)).tolist() == [hi, hi] and hi > 3.4e38


def test_wave_tree_sum_is_a_sum():
    rng = np.random.RandomState(2)
    for n in (1, 7, 64, 65, 128, 256, 1000):
        v = rng.uniform(0, 1, n).astype(np.float32)
        assert abs(float(orc.wave_tree_sum(v)) - float(v.astype(np.float64).sum())) <= 1e-6 * n
    # integers sum exactly in any order
    assert orc.wave_tree_sum(np.arange(300, dtype=np.float32)) == 300 * 299 / 2
