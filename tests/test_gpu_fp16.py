"""fp16 hidden states (the reference follows the model dtype: bf16 or fp16): the per-token quantiser, the fused
gather, the down projection's output, the combine and the whole layer, bit for bit against the checker with its
16-bit kind switched to fp16."""
import dataclasses

import numpy as np
import pytest
import torch

from _inputs import CONFIGS, bits, gating_kwargs, make_layer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def K():
    from vllm_ascend_amd import kernels

    return kernels


@pytest.fixture(scope="module")
def orc():
    from oracle import oracle

    return oracle


def test_checker_fp16_conversions_match_numpy(orc):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * s for s in (1e-6, 1e-3, 1.0, 300.0, 7e4)])
    x = np.concatenate([x, np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6.1e-5, 5.96e-8, 2.98e-8], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(orc.f32_to_f16(x), want.view(np.uint16))
    assert np.array_equal(orc.f16_to_f32(want.view(np.uint16)), want.astype(np.float32))


@pytest.mark.parametrize("rows,cols", [(37, 2048), (5, 100), (1, 8)])
def test_dynamic_quant_fp16(K, orc, rows, cols):
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, cols, generator=g) * 3).to(torch.float16)
    x[0] = 0
    q, s = K.dynamic_quant(x.to(DEV))
    torch.cuda.synchronize()
    with orc.half_kind("f16"):
        q_want, s_want = orc.dynamic_quant(bits(x))
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


def test_fp16_stages_match_the_checker(K, orc):
    """init_routing (fused quant and plain copy), down projection to fp16 on all three GEMM kernels, combine."""
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(3)
    T, k, E, H = 70, 4, 12, 256
    x = torch.randn(T, H, generator=g).to(torch.float16)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    with orc.half_kind("f16"):
        xs_w, dst_w, cnt_w, sx_w = orc.init_routing(bits(x), ids.numpy(), E)
        xp_w, _, _, _ = orc.init_routing(bits(x), ids.numpy(), E, quant=False)
    xs, dst, cnt, sx = K.init_routing(x.to(DEV), ids.to(DEV), E, 1, 1)
    xp, _, _, _ = K.init_routing(x.to(DEV), ids.to(DEV), E, -1, 1)
    torch.cuda.synchronize()
    assert np.array_equal(xs.cpu().numpy(), xs_w) and np.array_equal(dst.cpu().numpy(), dst_w)
    assert np.array_equal(sx.cpu().numpy().view(np.uint32), sx_w.view(np.uint32))
    assert xp.dtype == torch.float16 and np.array_equal(bits(xp.cpu()), xp_w)

    # down projection: streaming kernel (few rows), 128-row tiles, 256-row weight-streaming tiles
    for counts, Kd, N in (([3, 0, 9, 1], 256, 128), ([128, 64, 65, 129, 1, 0], 256, 256), ([128, 300, 0, 64], 4096, 128)):
        cnt_t = torch.tensor(counts, dtype=torch.int64)
        R, Ee = int(cnt_t.sum()), len(counts)
        cum = torch.cumsum(cnt_t, 0)
        a = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
        w = torch.randint(-128, 128, (Ee, N, Kd), generator=g, dtype=torch.int8)
        sw = torch.rand(Ee, N, generator=g) * 0.009 + 0.001
        sa = torch.rand(R, generator=g) * 0.05 + 0.001
        wnz = K.format_cast_nz(w.to(DEV), W_ENK)
        acc = orc.gmm_i32(a.numpy(), w.numpy(), cum.numpy())
        with orc.half_kind("f16"):
            want = orc.gmm2_dequant(acc, sa.numpy(), sw.numpy(), cum.numpy())
        got = K.gmm2_dequant(a.to(DEV), wnz, sw.to(DEV), sa.to(DEV), cnt_t.to(DEV), 1, N, Kd, out_dtype=torch.float16)
        torch.cuda.synchronize()
        assert got.dtype == torch.float16
        assert np.array_equal(bits(got.cpu()), want), (counts, Kd, N)

    # combine
    o = torch.randn(T * k, H, generator=g).to(torch.float16)
    wts = torch.rand(T, k, generator=g).to(torch.float16)
    res = torch.randn(T, H, generator=g).to(torch.float16)
    with orc.half_kind("f16"):
        want = orc.unpermute(bits(o), dst_w, bits(wts))
        want_r = orc.unpermute(bits(o), dst_w, bits(wts), bits(res))
    got = K.token_unpermute(o.to(DEV), dst, wts.to(DEV))
    got_r = K.token_unpermute(o.to(DEV), dst, wts.to(DEV), res.to(DEV))
    torch.cuda.synchronize()
    assert got.dtype == torch.float16
    assert np.array_equal(bits(got.cpu()), want) and np.array_equal(bits(got_r.cpu()), want_r)


@pytest.mark.parametrize("name", ["c1_tiny", "c2_small", "w4a8_small"])
def test_fp16_layer_matches_the_checker(orc, name):
    from _layer_utils import build_layer, oracle_layer

    if name == "w4a8_small":
        cfg = dataclasses.replace(CONFIGS["c5_w4a8_zipf"], name=name, T=48, E=8, H=512, I=256, n_group=1, topk_group=1)
    else:
        cfg = CONFIGS[name]
    print(f"fp16 layer {name}", flush=True)
    d = make_layer(cfg, seed=9)
    d["x"] = d["x"].to(torch.float16)
    if cfg.w4_group >= 0:
        layer = build_layer(cfg, d)
    else:
        from vllm_ascend_amd.quantization import get_scheme_class

        layer = build_layer(cfg, d)
        layer.quant_method.in_dtype = torch.float16
    out = layer(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    with orc.half_kind("f16"):
        want = oracle_layer(cfg, d, keep_acc=False)
    want_out = want.out if hasattr(want, "out") else want
    assert np.array_equal(bits(out.cpu()), want_out)


def test_router_gate_fp16_input(K, orc):
    g = torch.Generator().manual_seed(5)
    for T in (6, 4200):
        x = torch.randn(T, 320, generator=g).to(torch.float16)
        w = torch.randn(40, 320, generator=g) * 0.05
        got = K.router_gate(x.to(DEV), w.to(DEV))
        torch.cuda.synchronize()
        want = orc.router_gate(x.float().numpy(), w.numpy())   # the widening is exact
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_fp16_output_rounds_the_fp32_product_not_the_exact_one(K, orc):
    """(acc * s_token) * s_channel is rounded to fp32 and then to fp16.  Channels are chosen so that the fp32
    product is an exact fp16 tie while the exact product is not: a multiply fused into the conversion (one
    rounding) gives the odd neighbour there."""
    from vllm_ascend_amd._lib import W_ENK

    rng = np.random.default_rng(0)
    n_try = 1 << 21
    acc = rng.integers(-127, 128, n_try).astype(np.float32)
    cs = (rng.random(n_try, dtype=np.float32) * np.float32(3.0) + np.float32(0.5))
    rs = np.float32(0.37109375)
    t = (acc * rs).astype(np.float32)
    v = (t * cs).astype(np.float32)
    exact = t.astype(np.float64) * cs.astype(np.float64)
    is_tie = ((v.view(np.uint32) & 0x1FFF) == 0x1000) & (np.abs(v) > 1.0) & (exact != v.astype(np.float64))
    pick = np.flatnonzero(is_tie)[:64]
    assert len(pick) == 64
    N, Kd = 64, 64
    w = np.zeros((1, N, Kd), dtype=np.int8)
    w[0, :, 0] = acc[pick].astype(np.int8)
    x = np.zeros((2, Kd), dtype=np.int8)
    x[:, 0] = 1
    sw = cs[pick].reshape(1, N)
    sa = np.array([rs, rs], dtype=np.float32)
    cum = np.array([2], dtype=np.int64)
    with orc.half_kind("f16"):
        want = orc.gmm2_dequant(orc.gmm_i32(x, w, cum), sa, sw, cum)
    with np.errstate(over="ignore"):
        assert np.array_equal(want[0], v[pick].astype(np.float16).view(np.uint16))      # the checker rounds twice
    wnz = K.format_cast_nz(torch.from_numpy(w).to(DEV), W_ENK)
    got = K.gmm2_dequant(torch.from_numpy(x).to(DEV), wnz, torch.from_numpy(sw).to(DEV), torch.from_numpy(sa).to(DEV),
                         torch.from_numpy(cum).to(DEV), 0, N, Kd, out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)


@pytest.mark.parametrize("variant", ["shared", "shared_overlap", "weight_lists"])
def test_fp16_layer_with_shared_expert_and_weight_lists(orc, variant):
    from _layer_utils import build_layer, oracle_layer

    shared = variant.startswith("shared")
    cfg = CONFIGS["c4_small"] if shared else CONFIGS["c2_small"]
    print(f"fp16 layer variant {variant}", flush=True)
    d = make_layer(cfg, seed=2)
    d["x"] = d["x"].to(torch.float16)
    layer = build_layer(cfg, d, DEV, shared=shared, overlap=variant == "shared_overlap",
                        dynamic_eplb=variant == "weight_lists")
    layer.quant_method.in_dtype = torch.float16
    res = layer.forward_impl(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    with orc.half_kind("f16"):
        tr = oracle_layer(cfg, d, shared=shared)
    assert res.routed_out.dtype == torch.float16
    if shared:
        assert np.array_equal(bits(res.shared_out), tr.extra["shared_out"])
    assert np.array_equal(bits(res.routed_out), tr.out)
