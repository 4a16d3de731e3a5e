"""The tolerance of the 16-bit output, pinned outside the CPU checker.

The relative error of the layer against an fp32-dequant reference (weights * scale, no activation quantisation) is
about 2e-2 on the benchmark's synthetic data, above the 1e-2 one would like to state.  This test shows with the
reference's own golden math in numpy (tests/_noise.py; nothing of the checker in it) that the figure is the noise
of the two 8-bit activation quantisers, which any bit-faithful W8A8-dynamic implementation carries: the golden
pipeline has the same error as the checker's bit-exact pipeline, the two quantisers' shares add up in quadrature,
and the checker's output agrees with the golden pipeline an order of magnitude better than either agrees with the
unquantised reference.  That is what the 5e-2 gate of the GPU tests stands on.
"""
import numpy as np

from _inputs import CONFIGS, bits, make_layer
from _layer_utils import oracle_layer
from _noise import error_split
from oracle import oracle as orc


def test_the_error_against_the_fp32_dequant_reference_is_the_noise_of_the_two_quantisers():
    cfg = CONFIGS["c1_tiny"]
    d = make_layer(cfg, seed=0)
    tr = oracle_layer(cfg, d, keep_acc=False)
    x = orc.half_to_f32(bits(d["x"]))
    w = orc.half_to_f32(tr.topk_weights)
    sp = error_split(x, w, tr.topk_ids, d["w13"].numpy(), d["s13"].numpy(), d["w2"].numpy(), d["s2"].numpy())
    ref = sp["_reference"]
    got = orc.half_to_f32(tr.out).astype(np.float64)  # the checker's 16-bit output == the GPU's, bit for bit
    err_checker = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
    first, second, both = sp["first_quant_only"], sp["second_quant_only"], sp["both"]
    print(f"first {first:.4e} second {second:.4e} both {both:.4e} checker {err_checker:.4e}")
    # the golden pipeline carries the same error as the checker's: the figure does not come from the checker
    assert abs(err_checker - both) <= 0.1 * both
    # and it is above 1e-2 and inside the 5e-2 gate
    assert 1e-2 < both < 5e-2 and 1e-2 < err_checker < 5e-2
    # two independent noise sources: shares add in quadrature
    assert abs(np.hypot(first, second) - both) <= 0.1 * both
    # neither share is negligible and neither is the whole of it
    assert 2e-3 < first < both and 2e-3 < second < both
    # the checker against the golden pipeline: 16-bit rounding and the golden's +-1 steps, far below the noise
    err_vs_golden = float(np.linalg.norm(got - sp["_both_output"]) / np.linalg.norm(sp["_both_output"]))
    assert err_vs_golden <= 0.25 * both


def test_the_quantiser_noise_follows_the_step_size():
    """Closed form behind the first share: a row quantised with step s = absmax / 127 carries uniform rounding
    noise of rms s / sqrt(12); for N(0,1) rows of 1024 values (absmax about 3.4) that is 0.77 % of the row's rms."""
    from _noise import quantise_rows

    rng = np.random.default_rng(0)
    v = rng.standard_normal((256, 1024))
    q, s = quantise_rows(v)
    err = q * s[:, None] - v
    rms = np.sqrt((err ** 2).mean(axis=1))
    assert np.allclose(rms, s / np.sqrt(12.0), rtol=0.1)
    rel = float(np.linalg.norm(err) / np.linalg.norm(v))
    assert 6e-3 < rel < 1e-2
