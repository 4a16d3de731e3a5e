"""Router gate kernel against the checker, bit for bit (fp32 logits), every launch form (one workgroup per K
chunk for few tokens; two or four wavefronts sharing an output tile and taking its chunks in turn; one wavefront
per tile over all chunks), ragged token and expert counts, the order-pin cases of the CPU suite, and the layer
computing its own logits."""
import numpy as np
import pytest
import torch

from _inputs import CONFIGS, bits, make_layer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = np.float32


@pytest.fixture(scope="module")
def K():
    from vllm_ascend_amd import kernels

    return kernels


@pytest.fixture(scope="module")
def orc():
    from oracle import oracle

    return oracle


def _same_bits(a: torch.Tensor, b: np.ndarray):
    return np.array_equal(a.cpu().numpy().view(np.uint32), b.view(np.uint32))


# (T, H, E): decode (split over chunks), ragged everything, tail chunk of 64, more than 128 experts per row of
# workgroups, enough tiles for the single-pass form, DeepSeek-V3's K; then the forms in which the wavefronts of a
# workgroup share a tile: four per tile (256 tiles; fp32 tokens: two), two per tile with a last group of one
# chunk that is 64 long, at most 32 experts with two and with four per tile; more than one round of workgroups,
# the rest of the tokens in a launch of their own (two and four wavefronts per tile)
@pytest.mark.parametrize("T,H,E", [(64, 2048, 128), (5, 192, 40), (1, 64, 8), (33, 320, 288), (4200, 256, 256),
                                   (4100, 192, 130), (96, 7168, 256), (1000, 2112, 256), (2000, 1088, 250),
                                   (16001, 1088, 24), (9000, 2112, 20), (5000, 1088, 256), (4600, 2112, 256)])
@pytest.mark.parametrize("x_dtype", ["bf16", "f32", "f16"])
def test_router_gate_matches_the_checker(K, orc, T, H, E, x_dtype):
    print(f"router gate T={T} H={H} E={E} x={x_dtype}", flush=True)
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g)
    w = torch.randn(E, H, generator=g) * 0.05
    b = torch.randn(E, generator=g)
    if x_dtype in ("bf16", "f16"):
        xb = x.to(torch.bfloat16 if x_dtype == "bf16" else torch.float16)
        x_np = bits(xb) if x_dtype == "bf16" else xb.float().numpy()  # fp16 -> fp32 is exact
        x_dev = xb.to(DEV)
    else:
        x_np = x.numpy()
        x_dev = x.to(DEV)
    got = K.router_gate(x_dev, w.to(DEV))
    got_b = K.router_gate(x_dev, w.to(DEV), b.to(DEV))
    torch.cuda.synchronize()
    assert got.dtype == torch.float32 and tuple(got.shape) == (T, E)
    assert _same_bits(got, orc.router_gate(x_np, w.numpy()))
    assert _same_bits(got_b, orc.router_gate(x_np, w.numpy(), b.numpy()))
    # and the value: float64 dot products within a few ulps of the magnitude sum
    want = x_dev.double().cpu().numpy() @ w.double().numpy().T
    mag = np.abs(x_dev.double().cpu().numpy()) @ np.abs(w.double().numpy()).T
    assert np.all(np.abs(got.cpu().numpy() - want) <= 1e-6 * mag + 1e-30)


def test_router_gate_order_cases_on_the_gpu(K, orc):
    """The cases that tell the summation order apart, on every launch form: with 32 experts, 5 tokens run one
    workgroup per chunk (8 at the longer K), 4200 one wavefront per tile; at 17 chunks (the last 64 long) 9000 tokens run four
    wavefronts per tile, 16000 two and 30000 one."""
    big = F(2.0 ** 24)
    for H, T in ((320, 5), (320, 4200), (2112, 8), (2112, 9000), (2112, 16000), (2112, 30000)):
        rows = []
        cases = [({0: big, 128: 1, 129: 1}, big + 2), ({0: big, 64: 1, 65: 1}, big), ({0: 1, 1: 1, 2: big}, big + 2),
                 ({5: 1, 130: 1, 260: big}, big + 2), ({5: big, 130: 1, 260: 1}, big)]
        if H > 2100:  # chunks of different groups of two and of four, and the short last chunk
            cases += [({0: big, 517: 1, 1027: 1}, big), ({517: 1, 1027: 1, 2100: big}, big + 2),
                      ({700: big, 2050: 1, 2111: 1}, big + 2)]
        for pairs, _ in cases:
            r = np.zeros(H, dtype=F)
            for k, v in pairs.items():
                r[k] = v
            rows.append(r)
        n = len(rows)
        want_col = np.array([v for _, v in cases], dtype=F)
        a = F(1.0) + F(2.0 ** -12)
        fma_row = np.zeros(H, dtype=F)
        fma_w = np.ones(H, dtype=F)
        fma_row[0], fma_w[0] = 1.0, -(F(1.0) + F(2.0 ** -11))
        fma_row[1], fma_w[1] = a, a
        print(f"gate order cases H={H} T={T}", flush=True)
        x = np.zeros((T, H), dtype=F)
        x[:n] = np.stack(rows)
        w = np.ones((32, H), dtype=F)
        got = K.router_gate(torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV))
        torch.cuda.synchronize()
        assert np.array_equal(got[:n, 0].cpu().numpy(), want_col), (H, T)
        assert _same_bits(got, orc.router_gate(x, w))
        x[0] = fma_row
        w[3] = fma_w
        got = K.router_gate(torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV))
        assert got[0, 3].item() == 2.0 ** -24, (H, T)
        # bias last: (1 + 2^24) + 1
        x[1] = 0
        x[1, 0], x[1, 128] = 1, big
        w[3] = 1
        got = K.router_gate(torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV), torch.ones(32, device=DEV))
        assert got[1, 3].item() == float(big), (H, T)


def test_router_gate_argument_checks(K):
    w = torch.zeros(8, 64, device=DEV)
    assert tuple(K.router_gate(torch.zeros(0, 64, device=DEV), w).shape) == (0, 8)
    assert tuple(K.router_gate(torch.zeros(2, 3, 64, device=DEV, dtype=torch.bfloat16), w).shape) == (2, 3, 8)
    with pytest.raises(ValueError, match="features"):
        K.router_gate(torch.zeros(4, 128, device=DEV), w)
    with pytest.raises(TypeError, match="float32"):
        K.router_gate(torch.zeros(4, 64, device=DEV), w.to(torch.bfloat16))
    with pytest.raises(TypeError):
        K.router_gate(torch.zeros(4, 64, device=DEV, dtype=torch.float64), w)
    with pytest.raises(RuntimeError, match="GPU"):
        K.router_gate(torch.zeros(4, 64), w)
    with pytest.raises(RuntimeError):   # hidden not a multiple of 64
        K.router_gate(torch.zeros(4, 32, device=DEV), torch.zeros(8, 32, device=DEV))


def test_gate_linear_module_and_internal_router(K, orc):
    from _layer_utils import build_layer
    from vllm_ascend_amd.fused_moe.gate_linear import AscendGateLinear

    cfg = CONFIGS["c1_tiny"]
    d = make_layer(cfg, seed=7)
    g = torch.Generator().manual_seed(11)
    gate = AscendGateLinear(cfg.H, cfg.E, params_dtype=torch.bfloat16, device=DEV)
    assert gate.weight.dtype == torch.float32 and gate.bias is None
    w = torch.randn(cfg.E, cfg.H, generator=g) * 0.05
    gate.weight_loader(gate.weight, w.to(torch.bfloat16))            # checkpoints may hold the gate in bf16
    with pytest.raises(ValueError, match="does not fit"):
        gate.weight_loader(gate.weight, torch.zeros(cfg.E, cfg.H + 1))
    x = d["x"].to(DEV)
    logits, second = gate(x)
    assert second is None and logits.dtype == torch.float32
    assert _same_bits(logits, orc.router_gate(bits(d["x"]), w.to(torch.bfloat16).float().numpy()))
    half, _ = gate(x.to(torch.float16))                              # other dtypes are widened on the host side
    assert _same_bits(half, orc.router_gate(x.to(torch.float16).float().cpu().numpy(),
                                            w.to(torch.bfloat16).float().numpy()))
    layer = build_layer(cfg, d)
    with pytest.raises(ValueError, match="router_logits is required"):
        layer(x)
    layer.gate = gate
    assert torch.equal(layer(x), layer(x, logits))
