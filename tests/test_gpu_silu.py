"""The SwiGLU gate function of the kernels against its definition, on every binary32 input.

The kernels compute ``g / (1 + exp(-g))`` with a division specialised to divisors in [1, 2^128) (seven
instructions where a general IEEE division takes twelve).  The function has one fp32 argument, so "the same
result bit for bit" can be checked exhaustively: all 2^32 patterns go through both forms on the GPU
(``moe355_silu_f32`` form 0 = the kernels' sequence, form 1 = the IEEE quotient), and a sample that covers
every exponent goes through the CPU checker as well (reference formula:
csrc/gmm/grouped_matmul_swiglu_quant/README.md:63-67).
"""
import numpy as np
import pytest
import torch

from oracle import oracle
from vllm_ascend_amd import _lib

pytestmark = pytest.mark.gpu


def _silu(g: torch.Tensor, form: int) -> torch.Tensor:
    out = torch.empty_like(g)
    lib = _lib.load()
    _lib.check(lib.moe355_silu_f32(g.data_ptr(), out.data_ptr(), g.numel(), form,
                                   torch.cuda.current_stream().cuda_stream), "moe355_silu_f32")
    return out


def test_silu_sequence_equals_the_ieee_quotient_on_all_inputs():
    chunk = 1 << 26
    base = torch.arange(chunk, dtype=torch.int64, device="cuda")
    bad = 0
    first_bad = None
    for c in range((1 << 32) // chunk):
        bits = (base + c * chunk).to(torch.int32)  # wraps into the negative patterns, which is the point
        g = bits.view(torch.float32)
        a = _silu(g, 0)
        b = _silu(g, 1)
        same = (a.view(torch.int32) == b.view(torch.int32)) | (torch.isnan(a) & torch.isnan(b))
        n = int((~same).sum())
        if n and first_bad is None:
            i = int(torch.nonzero(~same)[0])
            first_bad = (hex(int(bits[i]) & 0xFFFFFFFF), float(g[i]), float(a[i]), float(b[i]))
        bad += n
    assert bad == 0, f"{bad} inputs differ; first: {first_bad}"


def test_silu_sequence_equals_the_cpu_checker_on_a_sample_of_every_exponent():
    rng = np.random.default_rng(5)
    # every sign and exponent with 4096 random mantissas each, plus the edges of every binade
    exps = np.arange(512, dtype=np.uint32)  # sign + exponent
    mant = rng.integers(0, 1 << 23, size=(512, 4096), dtype=np.uint32)
    mant[:, 0] = 0
    mant[:, 1] = (1 << 23) - 1
    mant[:, 2] = 1
    bits = ((exps[:, None] << 23) | mant).reshape(-1)
    # and a dense sweep of the range where the exponential is neither 0 nor huge
    sweep = np.linspace(-90.0, 20.0, 1 << 20).astype(np.float32).view(np.uint32)
    bits = np.concatenate([bits, sweep])
    g = bits.view(np.float32)
    want = oracle.silu(g)
    got = _silu(torch.from_numpy(g).cuda(), 0).cpu().numpy()
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), f"{(~same).sum()} differ, first at g = {g[~same][0]!r}"
