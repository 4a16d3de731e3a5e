"""Pins of the checker's router gate (oracle.router_gate): the value against float64, and the summation order
(chunks of 128, fused multiply-add, ascending k, ascending chunks, bias last) through cases in which every
other plausible order gives a different float."""
import numpy as np

from oracle import oracle as orc

F = np.float32
BIG = F(2.0 ** 24)


def _one_row(pairs, H=256):
    """x [1, H], w [1, H] with x[k] * w[k] = given products (x carries the value, w is 1)."""
    x = np.zeros((1, H), dtype=F)
    w = np.ones((1, H), dtype=F)
    for k, v in pairs.items():
        x[0, k] = v
    return x, w


def test_value_against_float64():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((37, 320)).astype(F)
    w = (rng.standard_normal((24, 320)) * 0.05).astype(F)
    b = rng.standard_normal(24).astype(F)
    got = orc.router_gate(x, w, b)
    want = x.astype(np.float64) @ w.astype(np.float64).T + b
    scale = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T + np.abs(b)
    assert np.all(np.abs(got - want) <= 1e-6 * scale)
    assert got.dtype == F and got.shape == (37, 24)


def test_small_integers_are_exact():
    rng = np.random.default_rng(1)
    x = rng.integers(-8, 9, (9, 192)).astype(F)
    w = rng.integers(-8, 9, (5, 192)).astype(F)
    assert np.array_equal(orc.router_gate(x, w), (x.astype(np.int64) @ w.astype(np.int64).T).astype(F))


def test_fused_multiply_add_not_multiply_then_add():
    # (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24: the product rounds to 1 + 2^-11, the fused form keeps the 2^-24
    a = F(1.0) + F(2.0 ** -12)
    x = np.zeros((1, 64), dtype=F)
    w = np.zeros((1, 64), dtype=F)
    x[0, 0], w[0, 0] = F(1.0), -(F(1.0) + F(2.0 ** -11))
    x[0, 1], w[0, 1] = a, a
    assert orc.router_gate(x, w)[0, 0] == F(2.0 ** -24)


def test_chunks_of_128_in_ascending_order():
    # 2^24 + 1 rounds back to 2^24; 2^24 + 2 is representable
    x, w = _one_row({0: BIG, 128: 1, 129: 1})          # the two ones meet in the second chunk first
    assert orc.router_gate(x, w)[0, 0] == BIG + F(2)
    x, w = _one_row({0: BIG, 64: 1, 65: 1})            # same chunk as 2^24: each one is lost (chunks are not 64 long)
    assert orc.router_gate(x, w)[0, 0] == BIG
    x, w = _one_row({0: 1, 1: 1, 2: BIG})              # ascending k inside a chunk
    assert orc.router_gate(x, w)[0, 0] == BIG + F(2)
    x, w = _one_row({5: 1, 130: 1, 260: BIG}, H=320)   # ascending chunks: (1 + 1) + 2^24; the tail chunk is 64 long
    assert orc.router_gate(x, w)[0, 0] == BIG + F(2)
    x, w = _one_row({5: BIG, 130: 1, 260: 1}, H=320)   # the other way round both ones are lost
    assert orc.router_gate(x, w)[0, 0] == BIG


def test_bias_is_added_last():
    x, w = _one_row({0: 1, 128: BIG})
    assert orc.router_gate(x, w, np.array([1], dtype=F))[0, 0] == BIG      # (1 + 2^24) + 1, not (1 + 1) + 2^24


def test_bf16_input_is_widened_exactly():
    rng = np.random.default_rng(2)
    xb = orc.f32_to_bf16(rng.standard_normal((6, 128)).astype(F))
    w = rng.standard_normal((4, 128)).astype(F)
    assert np.array_equal(orc.router_gate(xb, w), orc.router_gate(orc.bf16_to_f32(xb), w))
