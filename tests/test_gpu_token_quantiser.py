"""The token quantiser of the kernels against its definition, on every pair a 16-bit row can hold.

The definition divides every value by the row's scale (torch_npu.npu_dynamic_quant as called from
vllm_ascend/device/device_op.py:192-206: ``rint(x / (max|row| / 127))``).  The kernels take the scale's
reciprocal once per row and correct the product once.  A row of bf16 or fp16 values offers 2^15 finite maxima
and, below each, at most 2^16 values: every such pair goes through the shipped sequence
(``moe355_dynamic_quant``, form 0) and through the IEEE division (form 1 of ``moe355_dynamic_quant_form``) and
must give the same int8 and the same scale; the fused gating-and-quantisation launch, which carries its own
copy of the row loop, is run on the same rows, and a sample is checked against the CPU checker.
"""
import numpy as np
import pytest
import torch

from oracle import oracle
from vllm_ascend_amd import _lib
from vllm_ascend_amd import kernels as K

pytestmark = pytest.mark.gpu

DT = {torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16}


def _quant(x: torch.Tensor, form: int):
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    s = torch.empty((rows,), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.moe355_dynamic_quant_form(x.data_ptr(), DT[x.dtype], rows, cols, q.data_ptr(), s.data_ptr(), form,
                                             torch.cuda.current_stream().cuda_stream), "moe355_dynamic_quant_form")
    return q, s


def _rows(dtype, maxima: torch.Tensor, lo: int, hi: int) -> torch.Tensor:
    """One row per maximum pattern: eight copies of the maximum, then the patterns lo..hi-1 of both signs' worth
    of 16-bit values, with everything that is larger than the maximum (or not a number) replaced by zero."""
    pats = torch.arange(lo, hi, dtype=torch.int32, device="cuda").to(torch.int16).view(dtype)
    amax = maxima.to(torch.int16).view(dtype)
    body = pats[None, :].expand(amax.numel(), -1)
    keep = body.float().abs() <= amax.float()[:, None]
    body = torch.where(keep, body, torch.zeros((), dtype=dtype, device="cuda"))
    return torch.cat([amax[:, None].expand(-1, 8), body], dim=1).contiguous()


def _finite_maxima(dtype) -> torch.Tensor:
    p = torch.arange(1, 1 << 15, dtype=torch.int32, device="cuda")
    return p[torch.isfinite(p.to(torch.int16).view(dtype).float())]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_row_reciprocal_equals_the_division_on_every_pair(dtype):
    maxima = _finite_maxima(dtype)
    pairs = 0
    # rows of 8 + 4096 values take the kernel form that keeps a row in registers
    for c0 in range(0, maxima.numel(), 2048):
        m = maxima[c0:c0 + 2048]
        for lo in range(0, 1 << 16, 4096):
            x = _rows(dtype, m, lo, lo + 4096)
            q0, s0 = _quant(x, 0)
            q1, s1 = _quant(x, 1)
            assert torch.equal(s0.view(torch.int32), s1.view(torch.int32))
            if not torch.equal(q0, q1):
                r, c = [int(v[0]) for v in torch.nonzero(q0 != q1, as_tuple=True)]
                raise AssertionError(f"max {float(x[r, 0])!r} value {float(x[r, c])!r}: {int(q0[r, c])} != {int(q1[r, c])}")
            pairs += int((x[:, 8:] != 0).sum())
    assert pairs > 900_000_000  # about half of 2^15 x 2^16: the values at or below each maximum


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("cols", [1 << 16, (1 << 16) - 3])
def test_the_other_row_loops_on_a_sweep_of_maxima(dtype, cols):
    """Long rows (the loop that reads the row twice) and rows that are not a multiple of eight (the scalar loop);
    every 61st maximum with all its values in one row."""
    maxima = _finite_maxima(dtype)[::61]
    for c0 in range(0, maxima.numel(), 128):
        x = _rows(dtype, maxima[c0:c0 + 128], 0, 1 << 16)[:, :cols + 8].contiguous()
        q0, s0 = _quant(x, 0)
        q1, s1 = _quant(x, 1)
        assert torch.equal(s0.view(torch.int32), s1.view(torch.int32))
        assert torch.equal(q0, q1)
        # the entry point without a form argument is form 0
        q2, s2 = K.dynamic_quant(x)
        assert torch.equal(q2, q0) and torch.equal(s2.view(torch.int32), s0.view(torch.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_gating_launch_quantises_like_the_division(dtype):
    maxima = _finite_maxima(dtype)[::7]
    g = torch.Generator(device="cuda").manual_seed(3)
    for c0 in range(0, maxima.numel(), 1024):
        m = maxima[c0:c0 + 1024]
        for lo in (0, 1 << 15):  # half of the patterns per row: 8 + 32768 values
            x = _rows(dtype, m, lo, lo + (1 << 15))
            logits = torch.randn((x.shape[0], 16), device="cuda", generator=g)
            _, _, xq, xs = K.gate_quant(x, logits, 2, 1, 1, 0, 1, 0, 1.0, 1e-20, None)
            q1, s1 = _quant(x, 1)
            assert torch.equal(xs.view(torch.int32), s1.view(torch.int32))
            assert torch.equal(xq, q1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sample_of_maxima_against_the_cpu_checker(dtype):
    maxima = _finite_maxima(dtype)
    pick = torch.cat([maxima[:4], maxima[-4:], maxima[torch.randperm(maxima.numel(), device="cuda",
                                                                     generator=torch.Generator(device="cuda").manual_seed(1))[:24]]])
    x = _rows(dtype, pick, 0, 1 << 16)
    q0, s0 = _quant(x, 0)
    with oracle.half_kind("bf16" if dtype == torch.bfloat16 else "f16"):
        want_q, want_s = oracle.dynamic_quant(x.view(torch.int16).cpu().numpy().view(np.uint16))
    assert np.array_equal(s0.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(q0.cpu().numpy(), want_q)
