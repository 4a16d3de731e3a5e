"""GPU parity: every entry point of libmoe355.so against the CPU checker, bit for bit."""
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


@pytest.mark.parametrize("rows,cols", [(1, 8), (3, 1024), (64, 2048), (17, 7168), (5, 200), (2, 30), (9, 4096), (4, 3080),
                                       (3, 8192), (2, 8200), (2, 12288)])
def test_dynamic_quant(K, orc, rows, cols):
    print(f"dynamic_quant rows={rows} cols={cols}", flush=True)
    g = torch.Generator().manual_seed(rows * 1000 + cols)
    x = torch.randn(rows, cols, generator=g).to(torch.bfloat16)
    x[0, :] = 0  # an all-zero row
    q, s = K.dynamic_quant(x.to(DEV))
    torch.cuda.synchronize()
    qo, so = orc.dynamic_quant(bits(x))
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))


GATING_CASES = [
    # (T, E, k, k_group, G, mode, renorm, norm_type, rsf, bias, dtype)
    (64, 128, 8, 1, 1, 1, 1, 0, 1.0, False, torch.float32),
    (64, 8, 2, 1, 1, 1, 1, 0, 1.0, False, torch.float32),
    (33, 256, 8, 4, 8, 1, 0, 1, 2.5, True, torch.float32),
    (33, 256, 8, 4, 8, 0, 1, 1, 2.5, True, torch.float32),
    (16, 64, 4, 1, 8, 1, 1, 0, 1.0, True, torch.float32),
    (16, 256, 32, 1, 8, 0, 1, 1, 1.0, True, torch.float32),
    (7, 128, 16, 2, 4, 1, 1, 0, 1.0, False, torch.bfloat16),
    (7, 128, 16, 2, 4, 1, 1, 1, 1.0, True, torch.float16),
    (5, 384, 6, 3, 6, 1, 1, 1, 1.0, True, torch.float32),
    (3, 2048, 8, 1, 1, 1, 1, 0, 1.0, False, torch.float32),
    (4097, 128, 8, 1, 1, 1, 1, 0, 1.0, False, torch.float32),
]


@pytest.mark.parametrize("case", GATING_CASES, ids=[str(i) for i in range(len(GATING_CASES))])
def test_gating_top_k(K, orc, case):
    T, E, k, k_group, G, mode, renorm, norm_type, rsf, use_bias, dtype = case
    print(f"gating {case}", flush=True)
    g = torch.Generator().manual_seed(45)
    x = (torch.rand(T, E, generator=g) * 4 - 2).to(dtype)
    bias = (torch.rand(E, generator=g) * 4 - 2).to(dtype) if use_bias else None
    y, idx, out = K.gating_top_k(x.to(DEV), k, k_group, G, mode, renorm, norm_type, True, rsf, 1e-20,
                                 bias.to(DEV) if use_bias else None)
    torch.cuda.synchronize()
    name = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}[dtype]
    yo, io, no = orc.gating_top_k(bits(x), k, bias=bits(bias) if use_bias else None, k_group=k_group, group_count=G,
                                  group_select_mode=mode, renorm=renorm, norm_type=norm_type,
                                  routed_scaling_factor=rsf, eps=1e-20, x_dtype=name, want_norm=True)
    assert np.array_equal(idx.cpu().numpy(), io)
    assert np.array_equal(bits(y).view(np.uint16 if dtype != torch.float32 else np.uint32),
                          yo.view(np.uint16 if dtype != torch.float32 else np.uint32))
    assert np.array_equal(out.cpu().numpy().view(np.uint32), no.view(np.uint32))


# Group-limited routing over every group length: powers of two up to 64 (the group scores come from a butterfly
# over the lanes of a group), others (one lane per group walks its experts), with logits from a set of five values
# so that ties inside and between groups are the rule, and with zeros of both signs.
@pytest.mark.parametrize("E,G,k_group,k", [(8, 8, 3, 2), (16, 8, 4, 4), (64, 16, 5, 6), (128, 8, 3, 8), (256, 16, 4, 8),
                                           (256, 8, 4, 8), (512, 8, 2, 8), (96, 4, 2, 6), (160, 5, 3, 8), (384, 2, 1, 4),
                                           (256, 64, 9, 8)])
@pytest.mark.parametrize("mode,norm_type", [(1, 1), (0, 0)])
def test_gating_groups_with_ties(K, orc, E, G, k_group, k, mode, norm_type):
    print(f"gating groups with ties E={E} G={G} k_group={k_group} k={k} mode={mode} norm={norm_type}", flush=True)
    T = 37
    g = torch.Generator().manual_seed(E * 31 + G)
    levels = torch.tensor([-1.5, -0.0, 0.0, 0.75, 2.0])
    x = levels[torch.randint(0, 5, (T, E), generator=g)]
    x[1::3] = (torch.rand(T, E, generator=g) * 4 - 2)[1::3]   # some rows without ties
    bias = levels[torch.randint(0, 5, (E,), generator=g)] * 0.5
    y, idx, out = K.gating_top_k(x.to(DEV), k, k_group, G, mode, 1, norm_type, True, 1.0, 1e-20, bias.to(DEV))
    torch.cuda.synchronize()
    yo, io, no = orc.gating_top_k(bits(x), k, bias=bits(bias), k_group=k_group, group_count=G, group_select_mode=mode,
                                  renorm=1, norm_type=norm_type, routed_scaling_factor=1.0, eps=1e-20, x_dtype="f32",
                                  want_norm=True)
    assert np.array_equal(idx.cpu().numpy(), io)
    assert np.array_equal(bits(y).view(np.uint32), yo.view(np.uint32))
    assert np.array_equal(out.cpu().numpy().view(np.uint32), no.view(np.uint32))


@pytest.mark.parametrize("T,k,E,H", [(3, 2, 2, 64), (64, 8, 128, 2048), (1, 1, 8, 64), (700, 8, 256, 512),
                                     (2000, 4, 16, 128), (40, 6, 2048, 64),
                                     # the single-launch path ends at 2048 rows; 64 slots per token is its widest
                                     (256, 8, 128, 256), (257, 8, 128, 256), (4, 64, 128, 64), (32, 64, 64, 64),
                                     # more than 2048 rows: the chunked path, whose scan splits the chunks into
                                     # 1024 / E partitions (E not a power of two, E above the thread count)
                                     (500, 6, 2048, 64), (3000, 3, 1000, 64), (1500, 2, 100, 64)])
@pytest.mark.parametrize("quant", [True, False])
def test_init_routing(K, orc, T, k, E, H, quant):
    print(f"init_routing T={T} k={k} E={E} H={H} quant={quant}", flush=True)
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    # distinct experts per token, like a real top-k
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    xs, dst, cnt, sx = K.init_routing(x.to(DEV), ids.to(DEV), E, 1 if quant else -1, 1)
    torch.cuda.synchronize()
    xo, do, co, so = orc.init_routing(bits(x), ids.numpy(), E, quant=quant)
    assert np.array_equal(dst.cpu().numpy(), do)
    assert np.array_equal(cnt.cpu().numpy(), co)
    assert np.array_equal(bits(xs), xo)
    if quant:
        assert np.array_equal(sx.cpu().numpy().view(np.uint32), so.view(np.uint32))
    # cumulative form of the token counts
    _, _, cum, _ = K.init_routing(x.to(DEV), ids.to(DEV), E, 1 if quant else -1, 0)
    assert np.array_equal(cum.cpu().numpy(), np.cumsum(co))


@pytest.mark.parametrize("T,k,E,H", [(60, 4, 16, 64), (900, 6, 100, 64), (3, 2, 8, 128)])
@pytest.mark.parametrize("quant", [True, False])
def test_init_routing_drops_out_of_range_experts(K, orc, T, k, E, H, quant):
    """Ids outside [0, E) take no row; their destination is one past the last row, which the combine skips (both the
    single-launch and the chunked form)."""
    print(f"init_routing with dropped pairs T={T} k={k} E={E} quant={quant}", flush=True)
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    bad = torch.rand(T, k, generator=g) < 0.15
    bad[0, 0] = True
    ids[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, E + 3, -2).to(torch.int32)
    R = T * k
    xs = torch.zeros(R, H, dtype=torch.int8 if quant else torch.bfloat16, device=DEV)
    xs_got, dst, cnt, sx = K.init_routing(x.to(DEV), ids.to(DEV), E, 1 if quant else -1, 1)
    torch.cuda.synchronize()
    xo, do, co, so = orc.init_routing(bits(x), ids.numpy(), E, quant=quant)
    valid = int(co.sum())
    assert valid < R and np.all(do[bad.reshape(-1).numpy()] == R)
    assert np.array_equal(dst.cpu().numpy(), do)
    assert np.array_equal(cnt.cpu().numpy(), co)
    assert np.array_equal(bits(xs_got[:valid]), xo[:valid])      # rows past the last valid pair are not written
    if quant:
        assert np.array_equal(sx[:valid].cpu().numpy().view(np.uint32), so[:valid].view(np.uint32))
    # the combine leaves the dropped pairs out (k rows of bf16 expert outputs per token, weights all non-zero)
    o = torch.randn(R, H, generator=g).to(torch.bfloat16)
    p = (torch.rand(T, k, generator=g) + 0.5).to(torch.bfloat16)
    out = K.token_unpermute(o.to(DEV), dst, p.to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), orc.unpermute(bits(o), do, bits(p)))
    # ... also when the caller has taken abs() of the indices first, as the reference's caller does
    out_abs = K.token_unpermute(o.to(DEV), dst.abs(), p.to(DEV))
    assert torch.equal(out_abs, out)


@pytest.mark.parametrize("T,k,E,H", [(64, 8, 128, 2048), (700, 8, 256, 512), (1, 1, 8, 64)])
def test_init_routing_of_prequantised_activations(K, orc, T, k, E, H):
    """int8 rows with their per-token scales are only moved: the result is what the quantising gather produces
    from the unquantised rows (the identity the checker's tests pin on the CPU)."""
    g = torch.Generator().manual_seed(T + E + 5)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    xq, s = K.dynamic_quant(x.to(DEV))
    xs, dst, cnt, sx = K.init_routing_prequant(xq, s, ids.to(DEV), E, 1)
    torch.cuda.synchronize()
    xo, do, co, so = orc.init_routing(bits(x), ids.numpy(), E, quant=True)
    assert np.array_equal(dst.cpu().numpy(), do) and np.array_equal(cnt.cpu().numpy(), co)
    assert np.array_equal(xs.cpu().numpy(), xo)
    assert np.array_equal(sx.cpu().numpy().view(np.uint32), so.view(np.uint32))


SMALL_ROUTE_CASES = [
    # T, k, E, H, norm_type, renorm, bias, G, k_group, rsf, logits dtype, hidden dtype
    (64, 8, 128, 2048, 0, 1, False, 1, 1, 1.0, torch.float32, torch.bfloat16),
    (64, 8, 256, 7168, 1, 1, True, 8, 4, 2.5, torch.float32, torch.bfloat16),
    (1, 1, 8, 64, 0, 0, False, 1, 1, 1.0, torch.float32, torch.bfloat16),
    (128, 8, 64, 512, 0, 1, False, 1, 1, 1.0, torch.bfloat16, torch.bfloat16),   # 1024 pairs: the limit
    (33, 6, 96, 9216, 1, 0, True, 4, 2, 1.5, torch.float16, torch.float16),      # rows longer than one pass
    (17, 2, 3, 72, 0, 1, False, 1, 1, 1.0, torch.float32, torch.float16),
    (100, 4, 256, 128, 0, 1, False, 1, 1, 1.0, torch.float32, torch.bfloat16),
    # a handful of tokens: fewer gating workgroups than wavefronts in one, groups that do not divide 64
    (16, 8, 256, 7168, 1, 1, True, 8, 4, 2.5, torch.float32, torch.bfloat16),
    (8, 8, 128, 2048, 0, 1, False, 1, 1, 1.0, torch.float32, torch.bfloat16),
    (5, 4, 64, 256, 1, 0, True, 4, 2, 1.0, torch.bfloat16, torch.bfloat16),
    (13, 6, 160, 512, 0, 1, False, 5, 3, 1.0, torch.float16, torch.float16),
    (2, 2, 2, 64, 0, 1, False, 1, 1, 1.0, torch.float32, torch.bfloat16),
]


@pytest.mark.parametrize("case", SMALL_ROUTE_CASES)
def test_route_quant_small_equals_gating_plus_init_routing(K, orc, case):
    """The one-launch form for small batches against the checker's gating and dispatch: ids, weights (rounded to
    the logits dtype, then to the hidden dtype), permutation, histogram; and, through the row -> token map, the
    int8 rows and scales of the expert-sorted activation."""
    T, k, E, H, norm_type, renorm, use_bias, G, k_group, rsf, ldt, xdt = case
    print(f"route_quant_small {case}", flush=True)
    assert K.route_quant_small_supported(T, k, E)
    g = torch.Generator().manual_seed(T * 31 + E)
    x = torch.randn(T, H, generator=g).to(xdt)
    logits = (torch.rand(T, E, generator=g) * 4 - 2).to(ldt)
    bias = (torch.rand(E, generator=g) * 0.4 - 0.2).to(ldt) if use_bias else None
    counter = torch.zeros(1, dtype=torch.int32, device=DEV)
    for _ in range(3):  # the arrival counter is left at zero: calls in a row share it
        tw, ids, xq, xs, dst, row_token, cnt = K.route_quant_small(
            x.to(DEV), logits.to(DEV), k, k_group, G, 1, renorm, norm_type, rsf, 1e-20,
            bias.to(DEV) if use_bias else None, sync_counter=counter)
    torch.cuda.synchronize()
    lname = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}[ldt]
    with orc.half_kind("f16" if xdt == torch.float16 else "bf16"):
        y, ids_want, _ = orc.gating_top_k(bits(logits), k, bias=bits(bias) if use_bias else None, k_group=k_group,
                                          group_count=G, group_select_mode=1, renorm=renorm, norm_type=norm_type,
                                          routed_scaling_factor=rsf, eps=1e-20, x_dtype=lname)
        # the reference's caller casts the gate's weights (logits dtype) to the hidden dtype
        yf = y if lname == "f32" else (orc.bf16_to_f32(y) if lname == "bf16" else orc.f16_to_f32(y))
        tw_want = orc.f32_to_half(yf)
        xs_want, dst_want, cnt_want, sx_want = orc.init_routing(bits(x), ids_want, E, quant=True)
    assert np.array_equal(ids.cpu().numpy(), ids_want)
    assert np.array_equal(bits(tw), tw_want)
    assert np.array_equal(dst.cpu().numpy(), dst_want)
    assert np.array_equal(cnt.cpu().numpy(), cnt_want)
    rt = row_token.cpu().numpy()
    assert np.array_equal(rt[dst_want], np.arange(T * k) // k)            # row -> token is the inverse map
    assert np.array_equal(xq.cpu().numpy()[rt], xs_want)                   # the expert-sorted rows, read through it
    assert np.array_equal(xs.cpu().numpy()[rt].view(np.uint32), sx_want.view(np.uint32))
    assert int(counter.item()) == 0
    assert not K.route_quant_small_supported(129, 8, 128) and not K.route_quant_small_supported(8, 8, 257)


@pytest.mark.parametrize("case", SMALL_ROUTE_CASES + [(3000, 8, 128, 512, 0, 1, False, 1, 1, 1.0, torch.float32,
                                                       torch.bfloat16),
                                                      (1500, 6, 256, 7168, 1, 1, True, 8, 4, 2.5, torch.bfloat16,
                                                       torch.bfloat16),
                                                      (700, 2, 40, 200, 1, 0, True, 4, 2, 1.0, torch.float16,
                                                       torch.float16),
                                                      # long rows (several passes of the workgroup over a row) and
                                                      # a row shorter than a wavefront, on more than a thousand tokens
                                                      (1100, 2, 16, 8192, 0, 1, False, 1, 1, 1.0, torch.float32,
                                                       torch.bfloat16),
                                                      (1030, 2, 16, 8200, 0, 1, False, 1, 1, 1.0, torch.float32,
                                                       torch.float16),
                                                      (2049, 4, 64, 72, 1, 1, False, 1, 1, 1.0, torch.bfloat16,
                                                       torch.bfloat16)])
def test_gate_quant_equals_gating_plus_dynamic_quant(K, orc, case):
    """Gating and token quantisation in one launch (any number of tokens) against the two separate kernels."""
    T, k, E, H, norm_type, renorm, use_bias, G, k_group, rsf, ldt, xdt = case
    print(f"gate_quant {case}", flush=True)
    assert K.gate_quant_supported(T, k, E)
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g).to(xdt).to(DEV)
    logits = (torch.rand(T, E, generator=g) * 4 - 2).to(ldt).to(DEV)
    bias = (torch.rand(E, generator=g) * 0.4 - 0.2).to(ldt).to(DEV) if use_bias else None
    tw, ids, xq, xs = K.gate_quant(x, logits, k, k_group, G, 1, renorm, norm_type, rsf, 1e-20, bias)
    y, ids_want, _, y_alt = K.gating_top_k(logits, k, k_group, G, 1, renorm, norm_type, False, rsf, 1e-20, bias,
                                           alt_dtype=xdt)
    xq_want, xs_want = K.dynamic_quant(x)
    torch.cuda.synchronize()
    assert torch.equal(ids, ids_want)
    assert torch.equal(tw.view(torch.int16), y_alt.view(torch.int16))
    assert torch.equal(xq, xq_want) and torch.equal(xs.view(torch.int32), xs_want.view(torch.int32))


@pytest.mark.parametrize("R,E,Kd,N,T", [(512, 128, 2048, 1536, 64), (40, 4, 64, 128, 40), (300, 16, 768, 256, 75),
                                        (512, 256, 1024, 4096, 64), (100, 8, 64, 4160, 25),
                                        # many rows per expert: the LDS-tiled kernel (128- and 64-row tiles) and the
                                        # weight-streaming tiles (wide and tall) read through the map as well
                                        (4096, 8, 512, 256, 700), (1300, 16, 192, 128, 400), (1100, 8, 1024, 256, 300),
                                        (700, 4, 4096, 128, 200), (1500, 6, 4096, 192, 1500),
                                        # one expert: the dense kernel
                                        (3100, 1, 128, 4096, 900)])
def test_gmm1_swiglu_quant_gather(K, orc, R, E, Kd, N, T):
    """Rows read through the row -> token map give what the gathered copy gives."""
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(R + E + 9)
    xq = torch.randint(-128, 128, (T, Kd), generator=g, dtype=torch.int8)
    sx = torch.rand(T, generator=g) * 0.05 + 0.001
    row_token = torch.randint(0, T, (R,), generator=g, dtype=torch.int32)
    w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    cnt = _rand_groups(g, E, R)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    q, qs = K.gmm1_swiglu_quant_gather(xq.to(DEV), sx.to(DEV), row_token.to(DEV), wnz, sw.to(DEV), cnt.to(DEV), 1, N,
                                       Kd)
    idx = row_token.long()
    q2, qs2 = K.gmm1_swiglu_quant(xq[idx].contiguous().to(DEV), wnz, sw.to(DEV), sx[idx].contiguous().to(DEV),
                                  cnt.to(DEV), 1, N, Kd)
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(qs, qs2)
    cum = torch.cumsum(cnt, 0)
    acc = orc.gmm_i32(xq[idx].numpy(), w.numpy(), cum.numpy())
    qo, so = orc.swiglu_quant(orc.dequant_acc(acc, sx[idx].numpy(), sw.numpy(), cum.numpy()))
    assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(qs.cpu().numpy().view(np.uint32), so.view(np.uint32))


# up to 4096 pairs of at most 1024 tokens: one launch; beyond: histogram, scan, scatter
@pytest.mark.parametrize("T,k,E,bad", [(3, 2, 2, False), (64, 8, 128, False), (300, 8, 256, True), (4096, 8, 256, False),
                                       (1000, 6, 40, True), (2500, 1, 7, False), (512, 8, 256, True), (513, 8, 256, False),
                                       (1024, 4, 2048, False), (64, 64, 64, False)])
def test_route_map_equals_init_routing_maps(K, T, k, E, bad):
    """The maps alone (nothing moved) against the ones of the init-routing op; row -> token inverts pair -> row."""
    g = torch.Generator().manual_seed(T + 5 * k + E)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if bad:
        drop = torch.rand(T, k, generator=g) < 0.1
        drop[0, 0] = True
        ids[drop] = E + 3
    x = torch.randn(T, 64, generator=g).to(torch.bfloat16)
    _, dst_want, cnt_want, _ = K.init_routing(x.to(DEV), ids.to(DEV), E, 1, 1)
    dst, row_token, cnt = K.route_map(ids.to(DEV), E, 1)
    _, _, cum = K.route_map(ids.to(DEV), E, 0)
    torch.cuda.synchronize()
    assert torch.equal(dst, dst_want) and torch.equal(cnt, cnt_want)
    assert torch.equal(cum, torch.cumsum(cnt_want, 0))
    d = dst.cpu().numpy()
    kept = d < T * k
    assert int(kept.sum()) == int(cnt.sum())
    assert np.array_equal(row_token.cpu().numpy()[d[kept]], (np.arange(T * k) // k)[kept])


def test_init_routing_known_answer(K):
    """Permutation known-answer vector of the reference (tests/ut/lora/test_lora.py:151-165)."""
    ids = torch.tensor([[1, 0], [0, 1], [1, 1]], dtype=torch.int32)
    x = torch.zeros(3, 64, dtype=torch.bfloat16)
    _, dst, cnt, _ = K.init_routing(x.to(DEV), ids.to(DEV), 2, 1, 1)
    assert dst.cpu().tolist() == [2, 0, 1, 3, 4, 5]
    assert cnt.cpu().tolist() == [2, 4]


def _rand_groups(g, E, R, empty_some=True):
    w = torch.rand(E, generator=g)
    if empty_some and E > 2:
        w[torch.randperm(E, generator=g)[: E // 4]] = 0
    cnt = torch.floor(w / w.sum() * R).to(torch.int64)
    cnt[int(torch.argmax(w))] += R - int(cnt.sum())
    return cnt


# (rows, experts, K, N).  rows/experts picks the kernel: < 48 weight streaming, >= 48 LDS-tiled with
# 128-row tiles, 48..256 with K >= 4096 (96..192 from K = 1024) the weight-streaming tiles; K % 64 != 0 always streams.
GMM_CASES = [(8, 128, 256, 128), (128, 2, 1024, 2816), (500, 32, 512, 512), (100, 16, 768, 2048),
             (1, 4, 32, 64), (300, 3, 7168, 256), (2100, 8, 256, 256), (3000, 4, 768, 2048),
             (1000, 16, 2048, 1536), (700, 2, 128, 320), (900, 3, 96, 192), (4100, 16, 512, 4096),
             # long rows of the SwiGLU re-quantisation: 2112 values (held in registers), 4160 (two passes)
             (40, 4, 64, 4224), (24, 2, 64, 8320),
             # many experts (a lane of the tile map / a thread of the scans owns more than one expert from 257
             # on): weight streaming, 128-row tiles and the weight-streaming tiles, each with 256 and with more
             (2000, 256, 128, 128), (1500, 320, 64, 64), (16000, 256, 128, 256), (20000, 320, 192, 128),
             (32000, 256, 1024, 128), (40000, 320, 1024, 64),
             # one expert with at most 64 rows and a long K (the shared expert of a decode batch): the int32 product
             # cuts K into slabs and adds the partial sums into the zeroed result
             (64, 1, 7168, 256), (33, 1, 2048, 1024), (1, 1, 4096, 128),
             # one expert with thousands of rows (the shared expert of a prefill batch): the dense kernel's 256 x 256
             # tiles, with a ragged last row tile and a last column block of 64 channels
             # (K of one to seven blocks of 64: fewer than, as many as and more than the closing steps of its K loop)
             (3000, 1, 128, 4096), (2049, 1, 192, 6464), (2100, 1, 64, 4096), (2050, 1, 384, 4096),
             (2300, 1, 448, 4096)]


@pytest.mark.parametrize("R,E,Kd,N", GMM_CASES)
@pytest.mark.parametrize("layout", ["enk", "ekn"])
def test_gmm_i32(K, orc, R, E, Kd, N, layout):
    print(f"gmm_i32 R={R} E={E} K={Kd} N={N} {layout}", flush=True)
    from vllm_ascend_amd._lib import W_EKN, W_ENK

    g = torch.Generator().manual_seed(R + E + Kd)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    cnt = _rand_groups(g, E, R)
    cum = torch.cumsum(cnt, 0)
    if layout == "enk":
        wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    else:
        wnz = K.format_cast_nz(w.transpose(1, 2).contiguous().to(DEV), W_EKN)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    acc = K.gmm_i32(x.to(DEV), wnz, cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)
    acc2 = K.gmm_i32(x.to(DEV), wnz, cnt.to(DEV), 1, N, Kd)
    assert np.array_equal(acc2.cpu().numpy(), ref)


@pytest.mark.parametrize("R,Kd,N,rows", [(64, 7168, 256, 64), (33, 2048, 1024, 20), (1, 4096, 128, 1), (48, 2048, 128, 0)])
def test_gmm_i32_dense_few_rows_with_and_without_scratch(K, orc, R, Kd, N, rows):
    """One expert, at most 64 rows, long K: K is cut into slabs.  With the scratch of moe355_gmm_i32_workspace() the
    slabs' partial sums are stored and added up, without any scratch they are added with atomics; both are the
    checker's sums, and the rows behind the expert's last one are zero."""
    from vllm_ascend_amd import _lib
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(R + Kd + N)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (1, N, Kd), generator=g, dtype=torch.int8)
    cnt = torch.tensor([rows], dtype=torch.int64)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cnt.numpy())
    ref[rows:] = 0
    acc = K.gmm_i32(x.to(DEV), wnz, cnt.to(DEV), 1, N, Kd)
    lib = _lib.load()
    xd, cd = x.to(DEV), cnt.to(DEV)
    acc2 = torch.full((R, N), 7, dtype=torch.int32, device=DEV)
    rc = lib.moe355_gmm_i32(xd.data_ptr(), wnz.data_ptr(), cd.data_ptr(), 1, R, Kd, N, 1, acc2.data_ptr(), None, 0,
                            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert np.array_equal(acc.cpu().numpy(), ref)
    got2 = acc2.cpu().numpy()
    assert np.array_equal(got2[:rows], ref[:rows])


def test_gmm_i32_dense_group_shorter_than_the_buffer(K, orc):
    """The dense kernel takes the row count from the group list on the device, not from the buffer's size: rows
    behind the group's last one stay as the caller's fill left them."""
    from vllm_ascend_amd._lib import W_ENK

    R, Kd, N, rows = 3200, 64, 4096, 2450
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (1, N, Kd), generator=g, dtype=torch.int8)
    cnt = torch.tensor([rows], dtype=torch.int64)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cnt.numpy())
    ref[rows:] = 0
    for glt in (0, 1):
        acc = K.gmm_i32(x.to(DEV), wnz, cnt.to(DEV), glt, N, Kd)
        assert np.array_equal(acc.cpu().numpy(), ref)


@pytest.mark.parametrize("R,E,Kd,N", GMM_CASES)
def test_gmm1_swiglu_quant(K, orc, R, E, Kd, N):
    print(f"gmm1 R={R} E={E} K={Kd} N={N}", flush=True)
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(R + E + Kd + 1)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    cnt = _rand_groups(g, E, R)
    covered = int(cnt.sum())
    cum = torch.cumsum(cnt, 0)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    q = torch.full((R, N // 2), 77, dtype=torch.int8, device=DEV)
    qs = torch.full((R,), -1.0, dtype=torch.float32, device=DEV)
    K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd, out=q, out_scale=qs)
    torch.cuda.synchronize()
    acc = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    f = orc.dequant_acc(acc, sx.numpy(), sw.numpy(), cum.numpy())
    qo, so = orc.swiglu_quant(f)
    assert covered == R
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(qs.cpu().numpy().view(np.uint32), so.view(np.uint32))


def test_gmm1_rows_beyond_groups_untouched(K):
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(3)
    R, E, Kd, N = 40, 4, 64, 128
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    cum = torch.tensor([5, 5, 20, 33], dtype=torch.int64)
    q = torch.full((R, N // 2), 77, dtype=torch.int8, device=DEV)
    qs = torch.full((R,), -1.0, dtype=torch.float32, device=DEV)
    K.gmm1_swiglu_quant(x.to(DEV), K.format_cast_nz(w.to(DEV), W_ENK), torch.ones(E, N, device=DEV),
                        torch.ones(R, device=DEV), cum.to(DEV), 0, N, Kd, out=q, out_scale=qs)
    assert bool((q[33:] == 77).all()) and bool((qs[33:] == -1.0).all())
    assert bool((qs[:33] >= 0).all())


@pytest.mark.parametrize("R,E,Kd,N", GMM_CASES)
def test_gmm2_dequant(K, orc, R, E, Kd, N):
    print(f"gmm2 R={R} E={E} K={Kd} N={N}", flush=True)
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(R + E + Kd + 2)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    cnt = _rand_groups(g, E, R)
    cum = torch.cumsum(cnt, 0)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    o = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt.to(DEV), 1, N, Kd)
    torch.cuda.synchronize()
    acc = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    oo = orc.gmm2_dequant(acc, sx.numpy(), sw.numpy(), cum.numpy())
    assert np.array_equal(bits(o), oo)


@pytest.mark.parametrize("T,k,H", [(64, 8, 2048), (5, 2, 1024), (33, 1, 64), (100, 8, 7168)])
@pytest.mark.parametrize("residual", [False, True])
def test_token_unpermute(K, orc, T, k, H, residual):
    print(f"unpermute T={T} k={k} H={H} residual={residual}", flush=True)
    g = torch.Generator().manual_seed(T + H)
    R = T * k
    o = torch.randn(R, H, generator=g).to(torch.bfloat16)
    idx = torch.randperm(R, generator=g).to(torch.int32)
    p = torch.rand(T, k, generator=g).to(torch.bfloat16)
    res = torch.randn(T, H, generator=g).to(torch.bfloat16) if residual else None
    out = K.token_unpermute(o.to(DEV), idx.to(DEV), p.to(DEV), res.to(DEV) if residual else None)
    torch.cuda.synchronize()
    ref = orc.unpermute(bits(o), idx.numpy(), bits(p), bits(res) if residual else None)
    assert np.array_equal(bits(out), ref)


# n / 2 up to 1024 and up to 4096 are held in registers between the passes, longer rows are computed twice
@pytest.mark.parametrize("rows,n", [(2, 192), (4, 192), (8, 384), (1, 256), (300, 2048), (3, 4096), (2, 8448)])
@pytest.mark.parametrize("left", [True, False])
def test_dequant_swiglu_quant(K, orc, rows, n, left):
    g = torch.Generator().manual_seed(rows + n)
    x = torch.randint(-100, 100, (rows, n), generator=g, dtype=torch.int32)
    ws = torch.randn(n, generator=g) * 0.1
    a = torch.randn(rows, generator=g) * 0.5
    y, s = K.dequant_swiglu_quant(x.to(DEV), ws.to(DEV), a.to(DEV), left, 0.0)
    torch.cuda.synchronize()
    yo, so = orc.dequant_swiglu_quant(x.numpy(), ws.numpy(), a.numpy(), left, 0.0)
    assert np.array_equal(y.cpu().numpy(), yo)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))


@pytest.mark.parametrize("rows,n", [(3, 192), (8, 384), (2, 8448)])
@pytest.mark.parametrize("left", [True, False])
def test_dequant_swiglu_quant_static_mode(K, orc, rows, n, left):
    """quant_mode 0 through the operator (torch.ops._C_ascend.npu_dequant_swiglu_quant) and the launcher."""
    from vllm_ascend_amd import custom_ops

    custom_ops.enable_custom_op()
    g = torch.Generator().manual_seed(rows * 31 + n)
    x = torch.randint(-100, 100, (rows, n), generator=g, dtype=torch.int32)
    ws = torch.randn(n, generator=g) * 0.1
    as_ = torch.randn(rows, generator=g) * 0.5
    qs = torch.rand(n // 2, generator=g) * 0.05 + 0.01
    qo = torch.randn(n // 2, generator=g) * 3
    for scale, off in ((qs, qo), (qs, None), (qs[:1], qo[:1]), (qs[:1], None)):
        want = orc.dequant_swiglu_quant_static(x.numpy(), ws.numpy(), as_.numpy(), scale.numpy(),
                                               None if off is None else off.numpy(), activate_left=left)
        got, sc = torch.ops._C_ascend.npu_dequant_swiglu_quant(
            x.to(DEV), weight_scale=ws.to(DEV), activation_scale=as_.to(DEV).reshape(rows, 1),
            quant_scale=scale.to(DEV), quant_offset=None if off is None else off.to(DEV), activate_left=left,
            quant_mode=0, swiglu_mode=1)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want)
        assert sc.shape == (rows,)


# the general form (groups, biases, swiglu_mode 1, both quant modes) and the row kernel behind swiglu_mode 1 calls
# without groups (the shared expert's call), against the restatement of the reference's grouped kernel class
@pytest.mark.parametrize("rows,n", [(20, 192), (300, 2048), (5, 8448), (64, 4096)])
@pytest.mark.parametrize("left", [True, False])
def test_dequant_swiglu_quant_grouped(K, orc, rows, n, left):
    g = torch.Generator().manual_seed(rows * 7 + n)
    G = 7
    x = torch.randint(-3000, 3000, (rows, n), generator=g, dtype=torch.int32)
    ws = (torch.rand(G, n, generator=g) * 1.8 + 0.2) * 1e-3
    a = torch.rand(rows, generator=g) * 1.5 + 0.5
    bias_i = torch.randint(-50, 50, (G, n), generator=g, dtype=torch.int32)
    bias_f = torch.randn(G, n, generator=g)
    cuts = sorted(torch.randint(0, rows, (G - 1,), generator=g).tolist())
    counts = torch.tensor([b - a_ for a_, b in zip([0] + cuts, cuts + [rows - rows // 5])], dtype=torch.int64).clamp_(min=-1)
    x[1] = 0                                                        # an all-zero row: scale 0, q 0
    dev = lambda t: None if t is None else t.to(DEV)
    npy = lambda t: None if t is None else t.numpy()

    def both(**kw):
        t = {k: dev(v) if torch.is_tensor(v) else v for k, v in kw.items()}
        o = {{"weight_scale": "w_scale", "activation_scale": "a_scale"}.get(k, k): npy(v) if torch.is_tensor(v) else v
             for k, v in kw.items()}
        got = K.dequant_swiglu_quant_grouped(dev(x), activate_left=left, **t)
        torch.cuda.synchronize()
        want = orc.dequant_swiglu_quant_grouped(x.numpy(), activate_left=left, **o)
        assert np.array_equal(got[0].cpu().numpy(), want[0]), kw.keys()
        if kw.get("quant_mode", 1) == 1:
            assert np.array_equal(got[1].cpu().numpy().view(np.uint32), want[1].view(np.uint32)), kw.keys()
        return want

    m1 = dict(swiglu_mode=1, clamp_limit=1.5, glu_alpha=1.702, glu_bias=1.0)
    # one group: the row kernel (what the shared expert runs), plain and with every swiglu_mode 1 parameter
    both(weight_scale=ws[0], activation_scale=a)
    both(weight_scale=ws[0], activation_scale=a, swiglu_mode=1)
    both(weight_scale=ws[0], activation_scale=a, **m1)
    both(weight_scale=ws[0], activation_scale=a, swiglu_mode=1, clamp_limit=0.75)
    both(weight_scale=ws[0], activation_scale=None, **m1)           # no activation scale: the general kernel
    # groups
    w = both(weight_scale=ws, activation_scale=a, group_index=counts)
    total = int(counts.clamp(min=0).sum())
    assert total < rows and not w[0][total:].any() and not w[1][total:].any()
    both(weight_scale=ws, activation_scale=a, group_index=counts, **m1)
    both(weight_scale=ws, activation_scale=a, group_index=counts, bias=bias_i, **m1)
    both(weight_scale=ws, activation_scale=a, group_index=counts, bias=bias_f)
    both(weight_scale=ws, activation_scale=None, group_index=counts, bias=bias_f, **m1)
    # static quantisation: one scale per group, one per group and channel, with and without offsets
    qs_g, qo_g = torch.rand(G, generator=g) * 0.04 + 0.01, torch.randn(G, generator=g)
    qs_c, qo_c = torch.rand(G, n // 2, generator=g) * 0.04 + 0.01, torch.randn(G, n // 2, generator=g)
    both(weight_scale=ws, activation_scale=a, group_index=counts, quant_mode=0, quant_scale=qs_g, quant_offset=qo_g)
    both(weight_scale=ws, activation_scale=a, group_index=counts, quant_mode=0, quant_scale=qs_c, quant_offset=qo_c, **m1)
    both(weight_scale=ws, activation_scale=a, group_index=counts, quant_mode=0, quant_scale=qs_c)


def test_npu_dequant_swiglu_quant_operator_routes_like_the_reference(K, orc):
    """group_index / swiglu_mode 1 -> the grouped kernel class (clamp, alpha, bias, its quantiser); swiglu_mode 0
    without groups -> the older kernels, which ignore clamp_limit (dequant_swiglu_quant_tiling.cpp:555-571)."""
    from vllm_ascend_amd import custom_ops

    custom_ops.enable_custom_op()
    op = torch.ops._C_ascend.npu_dequant_swiglu_quant
    g = torch.Generator().manual_seed(5)
    rows, n, G = 48, 512, 4
    x = torch.randint(-3000, 3000, (rows, n), generator=g, dtype=torch.int32)
    ws = (torch.rand(G, n, generator=g) * 1.8 + 0.2) * 1e-3
    a = torch.rand(rows, 1, generator=g) * 1.5 + 0.5
    counts = torch.tensor([10, 0, 30, 8], dtype=torch.int64)
    y, s = op(x.to(DEV), weight_scale=ws.to(DEV), activation_scale=a.to(DEV), group_index=counts.to(DEV),
              activate_left=True, quant_mode=1)                                   # moe_mlp.py:340-359
    want = orc.dequant_swiglu_quant_grouped(x.numpy(), ws.numpy(), a.numpy(), counts.numpy())
    assert np.array_equal(y.cpu().numpy(), want[0]) and np.array_equal(s.cpu().numpy(), want[1])
    kw = dict(activate_left=True, quant_mode=1, swiglu_mode=1, clamp_limit=2.0, glu_alpha=1.702, glu_bias=1.0)
    y, s = op(x.to(DEV), weight_scale=ws[0].to(DEV), activation_scale=a.to(DEV), **kw)   # shared_experts.py:272-289
    want = orc.dequant_swiglu_quant_grouped(x.numpy(), ws[0].numpy(), a.numpy(), swiglu_mode=1, clamp_limit=2.0,
                                            glu_alpha=1.702, glu_bias=1.0)
    assert np.array_equal(y.cpu().numpy(), want[0]) and np.array_equal(s.cpu().numpy(), want[1])
    y, s = op(x.to(DEV), weight_scale=ws[0].to(DEV), activation_scale=a.to(DEV), activate_left=True, quant_mode=1,
              swiglu_mode=0, clamp_limit=2.0)
    want = orc.dequant_swiglu_quant(x.numpy(), ws[0].numpy(), a.numpy(), True, 0.0)
    assert np.array_equal(y.cpu().numpy(), want[0]) and np.array_equal(s.cpu().numpy(), want[1])
    with pytest.raises(NotImplementedError, match="smooth"):
        op(x.to(DEV), weight_scale=ws[0].to(DEV), activation_scale=a.to(DEV), quant_scale=ws[0, :256].to(DEV), quant_mode=1)
    with pytest.raises(ValueError, match="group_index"):
        op(x.to(DEV), weight_scale=ws.to(DEV), activation_scale=a.to(DEV), quant_mode=1, swiglu_mode=1)


@pytest.mark.parametrize("act", ["gelu", "gelu_tanh", "swiglustep", "swigluoai"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_act_mul_quant(K, orc, act, dtype):
    limit, alpha, beta = (7.0, 1.0, 0.0) if act == "swiglustep" else ((3.0, 1.702, 1.0) if act == "swigluoai" else (0.0, 1.0, 0.0))
    g = torch.Generator().manual_seed(17)
    for rows, n in ((5, 192), (33, 1536), (2, 8320)):
        h = (torch.randn(rows, n, generator=g) * 4).to(dtype)
        h[0, :4] = torch.tensor([0.0, -0.0, 100.0, -100.0]).to(dtype)
        with orc.half_kind("bf16" if dtype == torch.bfloat16 else "f16"):
            q_want, s_want = orc.act_mul_quant(bits(h), act, limit, alpha, beta)
        # rows beyond the group list's total stay untouched
        cnt = torch.tensor([rows - 1, 0], dtype=torch.int64)
        q, s_ = K.act_mul_quant(h.to(DEV), act, limit, alpha, beta)
        torch.cuda.synchronize()
        assert np.array_equal(q.cpu().numpy(), q_want), (act, rows, n)
        assert np.array_equal(s_.cpu().numpy().view(np.uint32), s_want.view(np.uint32))
        for gl, gl_type in ((cnt, 1), (torch.cumsum(cnt, 0), 0)):
            q2, s2 = K.act_mul_quant(h.to(DEV), act, limit, alpha, beta, gl.to(DEV), gl_type)
            torch.cuda.synchronize()
            assert np.array_equal(q2[: rows - 1].cpu().numpy(), q_want[: rows - 1])
            assert np.array_equal(s2[: rows - 1].cpu().numpy().view(np.uint32), s_want[: rows - 1].view(np.uint32))


def test_grouped_matmul_swiglu_quant_v2_against_the_reference_golden(orc):
    """A8W4 operator with per-group scales and an arbitrary assist matrix, against a numpy rendering of
    gmm_swiglu_quant_golden_a8_w4 (tests/e2e/nightly/single_node/ops/singlecard_ops/
    test_grouped_matmul_swiglu_quant.py:58-109) in fp32: out = ((x - 8) . W . scale + bias) * per_token,
    SwiGLU, dynamic int8.  Tolerance of the reference test: int8 +-1, scale rtol 5e-3."""
    from vllm_ascend_amd import npu_ops
    from vllm_ascend_amd.custom_ops import enable_custom_op

    enable_custom_op()
    g = torch.Generator().manual_seed(0)
    E, M, Kd, N, grp = 4, 96, 512, 256, 256
    x = torch.randint(-5, 5, (M, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-5, 5, (E, Kd, N), generator=g, dtype=torch.int8)  # [E, K, N] int4 values
    scale = torch.randn(E, Kd // grp, N, generator=g)
    per_token = torch.randn(M, generator=g)
    bias = torch.rand(E, N, generator=g) * 10 - 5
    cum = torch.tensor([20, 20, 70, 90], dtype=torch.int64)  # rows 90..95 belong to no expert
    pairs = w.reshape(E, Kd, N // 2, 2)
    packed = ((pairs[..., 1] << 4) | (pairs[..., 0] & 0x0F)).to(torch.int8).contiguous().view(torch.int32)
    w_nz = npu_ops.npu_format_cast_int4(packed.to(DEV))
    scale_i64 = torch.from_numpy(scale.numpy().view(np.uint32).astype(np.int64))
    out, out_scale = torch.ops._C_ascend.grouped_matmul_swiglu_quant_v2(
        x=x.to(DEV), weight=[w_nz], weight_scale=[scale_i64.to(DEV)], x_scale=per_token.to(DEV),
        group_list=cum.to(DEV), weight_assist_matrix=[bias.to(DEV)], dequant_mode=0, group_list_type=0)
    # the older entry point of the same kernel takes the assist matrix as `bias`
    out_b, scale_b, _ = torch.ops._C_ascend.grouped_matmul_swiglu_quant(
        x=x.to(DEV), weight=w_nz, bias=bias.to(DEV), group_list=cum.to(DEV), weight_scale=scale_i64.to(DEV),
        x_scale=per_token.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(out_b[:90], out[:90]) and torch.equal(scale_b[:90], out_scale[:90])
    lo = 0
    for e, hi in enumerate(cum.tolist()):
        if hi > lo:
            xe = (x[lo:hi].to(torch.float64) - 8).reshape(hi - lo, Kd // grp, grp)
            we = w[e].to(torch.float64).reshape(Kd // grp, grp, N)
            mm = torch.einsum("mgk,gkn->gmn", xe, we) * scale[e].to(torch.float64)[:, None, :]
            f = (mm.sum(0) + bias[e].to(torch.float64)) * per_token[lo:hi, None].to(torch.float64)
            a, gate = f.chunk(2, dim=-1)
            y = a * torch.sigmoid(a) * gate
            mx = y.abs().max(dim=-1).values
            q_ref = torch.round(y * (127 / mx)[:, None]).to(torch.int8)
            assert (out[lo:hi].cpu().to(torch.int32) - q_ref.to(torch.int32)).abs().max() <= 1
            torch.testing.assert_close(out_scale[lo:hi].cpu().double(), mx / 127, rtol=5e-3, atol=1e-6)
        lo = hi


# ------------------------------------------------------------------ W4A8 grouped GEMMs, chunk boundaries
# rows per expert chosen around the 64-row unit of the int4 kernel (and its 32-row token blocks)
W4_COUNTS = [0, 1, 31, 32, 33, 63, 64, 65, 0, 130, 200, 7]


@pytest.mark.parametrize("Kd,N,group", [(256, 128, 128), (512, 192, 256), (128, 64, 128), (256, 128, 0),
                                        # more than 32 scale groups: the scales no longer fit LDS and are read
                                        # from memory group by group (40 K blocks: whole passes of that
                                        # variant's ring; 36: a remainder)
                                        (2560, 64, 64), (2304, 128, 64)])
@pytest.mark.parametrize("gl_type", [0, 1])
def test_w4_gemms_at_chunk_boundaries(K, orc, Kd, N, group, gl_type):
    print(f"w4 gemms K={Kd} N={N} group={group} gl_type={gl_type}", flush=True)
    g = torch.Generator().manual_seed(Kd + N + group)
    cnt = torch.tensor(W4_COUNTS, dtype=torch.int64)
    E, R = len(W4_COUNTS), int(cnt.sum())
    cum = torch.cumsum(cnt, 0)
    gsz = group if group else Kd
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-8, 8, (E, N, Kd), generator=g, dtype=torch.int8)
    sg = torch.rand(E, Kd // gsz, N, generator=g) * 0.09 + 0.01
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    bias = torch.randn(E, N, generator=g)
    gl = (cum if gl_type == 0 else cnt).to(DEV)
    w4 = K.format_cast_nz_int4(w.to(DEV), 0, N, Kd)
    # down-GEMM form: f = sum_g float(acc_g) * s_g (+ bias), then the token scale, bf16
    f = orc.gmm_w4_grouped(x.numpy(), w.numpy(), sg.numpy(), cum.numpy(), gsz)
    want = orc.w4_rows_to_bf16(f, sx.numpy())
    got = K.gmm2_dequant_w4(x.to(DEV), w4, sg.to(DEV), gsz, sx.to(DEV), gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)
    # gate_up form: token scale, SwiGLU, per-row re-quantisation
    q_want, s_want = orc.swiglu_quant(orc.scale_rows(f, sx.numpy()))
    q, s = K.gmm1_swiglu_quant_w4(x.to(DEV), w4, sg.to(DEV), gsz, sx.to(DEV), gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))
    # the same rows read through a row -> token map from tokens kept in token order
    T = 37
    tq = torch.randint(-128, 128, (T, Kd), generator=g, dtype=torch.int8)
    ts = torch.rand(T, generator=g) * 0.05 + 0.001
    row_token = torch.randint(0, T, (R,), generator=g, dtype=torch.int32)
    idx = row_token.long()
    q_map, s_map = K.gmm1_swiglu_quant_w4_gather(tq.to(DEV), ts.to(DEV), row_token.to(DEV), w4, sg.to(DEV), gsz, gl,
                                                 gl_type, N, Kd)
    q_cpy, s_cpy = K.gmm1_swiglu_quant_w4(tq[idx].contiguous().to(DEV), w4, sg.to(DEV), gsz,
                                          ts[idx].contiguous().to(DEV), gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert torch.equal(q_map, q_cpy) and torch.equal(s_map, s_cpy)
    # with the bias of the offset-corrected A8W4 form (added before the token scale)
    fb = f + np.repeat(bias.numpy(), W4_COUNTS, axis=0)
    got_b = K.gmm2_dequant_w4(x.to(DEV), w4, sg.to(DEV), gsz, sx.to(DEV), gl, gl_type, N, Kd, bias=bias.to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(bits(got_b.cpu()), orc.w4_rows_to_bf16(fb, sx.numpy()))


# rows per expert around the 128-row tile of the LDS-tiled kernel and its 64-row short-tile path, and around the
# 128 / 160 / 256-row shapes of the weight-streaming tiles
TILE_COUNTS = [128, 64, 65, 129, 192, 193, 1, 0, 256, 63, 127, 320, 160, 161, 144, 145]


# K >= 1024 at about 128 rows per expert selects the weight-streaming tiles (tall ones and wide ones of four and of
# five token blocks occur in TILE_COUNTS); the K values leave every remainder of the three-, four- and five-stage
# rings; below K = 1024 the 128-row tiles run, whose closing steps are compiled per remainder of K / 64 by three
# (64 and 128: fewer K blocks than the ring is deep)
@pytest.mark.parametrize("Kd,N", [(64, 128), (128, 256), (256, 256), (192, 128), (320, 128), (384, 192), (512, 320),
                                  (768, 256), (1024, 256), (2112, 128), (4096, 256),
                                  (4160, 320), (4224, 128), (4288, 256), (4352, 192), (4416, 1152)])
def test_tiled_gemms_at_tile_boundaries(K, orc, Kd, N):
    print(f"tiled gemms at tile boundaries K={Kd} N={N}", flush=True)
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(Kd * 3 + N)
    cnt = torch.tensor(TILE_COUNTS, dtype=torch.int64)
    E, R = len(TILE_COUNTS), int(cnt.sum())
    cum = torch.cumsum(cnt, 0)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    acc = K.gmm_i32(x.to(DEV), wnz, cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)
    want = orc.gmm2_dequant(ref, sx.numpy(), sw.numpy(), cum.numpy())
    got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt.to(DEV), 1, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)
    q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw.numpy(), cum.numpy()))
    q, s = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


# Skewed histograms: the host picks a kernel family from the mean rows per expert and, for a large product (a GiB
# of weights) with 12 to 19 rows per expert on average, the device splits the experts between streaming (up to 32
# rows: 31 / 32 / 33 sit on the border) and, above it, the weight-streaming tiles (K from 4096 on) or the 128-row
# tiles.  Small products with the same histogram run on the tiles alone.  The last two cases keep one family (the weight-streaming tiles) over experts far above and below
# its range: 255 / 256 / 257 / 511 / 513 rows.   name -> (rows per expert, K, N)
_HOT = [0, 1, 31, 32, 33, 2, 64, 65, 700, 3, 0, 5, 129, 7, 1, 0]
SKEWED = {
    "stream+wide": (_HOT + [12] * 240, 4096, 1024),
    "stream+wide, nothing above the border": ([16] * 224 + [32] * 32, 4096, 1024),
    "stream+tiled": (_HOT + [12] * 240, 2048, 2048),
    # a decode batch (fewer than 1024 rows, most experts idle) on a product of a GiB: split from one row per expert on
    "stream+wide, decode batch": ([0] * 200 + [1] * 40 + [2] * 8 + [300, 40, 33, 32, 31, 0, 5, 65], 4096, 1024),
    "stream+tiled, decode batch": ([0] * 200 + [1] * 40 + [2] * 8 + [300, 40, 33, 32, 31, 0, 5, 65], 2048, 2048),
    "tiled": (_HOT + [12] * 240, 256, 256),
    "wide": ([255, 256, 257, 511, 513, 1, 0, 33, 128, 160, 161, 192, 193, 40, 90, 100], 1024, 256),
    "wide, K 4096": ([300, 20, 256, 257, 47, 150, 0, 90], 4096, 256),
}


@pytest.mark.parametrize("name", list(SKEWED))
@pytest.mark.parametrize("gl_type", [0, 1])
def test_grouped_gemms_on_skewed_histograms(K, orc, name, gl_type):
    from vllm_ascend_amd._lib import W_ENK, load

    counts, Kd, N = SKEWED[name]
    cnt = torch.tensor(counts, dtype=torch.int64)
    E, R = len(counts), int(cnt.sum())
    print(f"skewed gemm {name}: E={E} R={R} K={Kd} N={N} gl_type={gl_type}", flush=True)
    lib = load()
    for epi in (0, 1, 2):
        kn = lib.moe355_gmm_kernel_name(epi, R, Kd, N, E).decode()
        families = name.split(",")[0].split("+")
        assert families[0] in kn and (" + " in kn) == (len(families) == 2)
        if len(families) == 2:
            assert f"+ gmm_{families[1]}_kernel" in kn
    g = torch.Generator().manual_seed(len(counts) + Kd)
    cum = torch.cumsum(cnt, 0)
    gl = (cum if gl_type == 0 else cnt).to(DEV)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    acc = K.gmm_i32(x.to(DEV), wnz, gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)
    want = orc.gmm2_dequant(ref, sx.numpy(), sw.numpy(), cum.numpy())
    got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)
    q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw.numpy(), cum.numpy()))
    q, s_ = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), gl, gl_type, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s_.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


@pytest.mark.parametrize("Kd,N", [(4096, 1024), (2048, 2048)])
def test_split_grouped_gemms_on_random_histograms(K, orc, Kd, N):
    """The two-launch forms (experts of at most 32 rows streamed, the others on tiles) on random histograms of 12 to
    23 rows per expert: uniform, Zipf-skewed, and with experts set exactly on the borders."""
    from vllm_ascend_amd._lib import W_ENK, load

    E = 256
    lib = load()
    g = torch.Generator().manual_seed(Kd + N)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    w_np, sw_np = w.numpy(), sw.numpy()
    for seed in range(3):
        r = np.random.default_rng(seed)
        avg = int(r.integers(12, 24))
        if seed == 0:
            cnt = r.multinomial(avg * E, np.full(E, 1.0 / E))
        else:
            p = 1.0 / np.arange(1, E + 1) ** r.uniform(0.6, 1.2)
            cnt = r.multinomial(avg * E, r.permutation(p / p.sum()))
        for e, c in zip(r.choice(E, 8, replace=False), (0, 31, 32, 33, 64, 65, 256, 257)):
            cnt[e] = c
        while cnt.sum() // E < 12:
            cnt[int(r.integers(E))] += 40
        while cnt.sum() // E > 23:
            cnt[int(np.argmax(cnt))] //= 2
        cnt = torch.from_numpy(cnt.astype(np.int64))
        R = int(cnt.sum())
        cum = torch.cumsum(cnt, 0)
        print(f"split gemm K={Kd} N={N} seed={seed}: R={R} max={int(cnt.max())} empty={int((cnt == 0).sum())}", flush=True)
        assert " + " in lib.moe355_gmm_kernel_name(1, R, Kd, N, E).decode()
        x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
        sx = torch.rand(R, generator=g) * 0.05 + 0.001
        ref = orc.gmm_i32(x.numpy(), w_np, cum.numpy())
        want = orc.gmm2_dequant(ref, sx.numpy(), sw_np, cum.numpy())
        got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt.to(DEV), 1, N, Kd)
        torch.cuda.synchronize()
        assert np.array_equal(bits(got.cpu()), want)
        q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw_np, cum.numpy()))
        q, s_ = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd)
        torch.cuda.synchronize()
        assert np.array_equal(q.cpu().numpy(), q_want)
        assert np.array_equal(s_.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


def test_w4_scales_of_every_magnitude(K, orc):
    """Subnormal scales, scales near the bottom of the normal range, zero and negative scales next to ordinary
    ones give the checker's bits (a token scale of 2^90 brings the tiny products into bf16 range)."""
    Kd, N, gsz = 256, 128, 128
    g = torch.Generator().manual_seed(11)
    cnt = torch.tensor([40, 70], dtype=torch.int64)
    cum = torch.cumsum(cnt, 0)
    R = int(cnt.sum())
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-8, 8, (2, N, Kd), generator=g, dtype=torch.int8)
    sx = torch.full((R,), 2.0 ** 90)
    w4 = K.format_cast_nz_int4(w.to(DEV), 0, N, Kd)
    base = torch.rand(2, Kd // gsz, N, generator=g) * 0.09 + 0.01
    variants = {"ordinary": base.clone()}
    t = base.clone()
    t[0, :, 5] = 1.0000001e-38                  # subnormal
    t[1, 0, 70] = 1.2345678 * 2.0 ** -124       # normal, a sixteenth of it is not
    t[1, 1, 3] = 0.0
    t[0, 1, 9] = -0.05
    variants["tiny"] = t
    t = base.clone() * 2.0 ** -100              # small everywhere
    t[0, 0, 64] = 2.0 ** -122
    variants["small"] = t
    for name, sg in variants.items():
        f = orc.gmm_w4_grouped(x.numpy(), w.numpy(), sg.numpy(), cum.numpy(), gsz)
        want = orc.w4_rows_to_bf16(f, sx.numpy())
        got = K.gmm2_dequant_w4(x.to(DEV), w4, sg.to(DEV), gsz, sx.to(DEV), cum.to(DEV), 0, N, Kd)
        torch.cuda.synchronize()
        assert np.array_equal(bits(got.cpu()), want), name
        assert np.count_nonzero(want) > want.size // 2, name


def test_w4_group_sum_order_on_the_gpu(K, orc):
    """The order-sensitive case of the CPU suite (terms 2^24, 1, 1 over three scale groups) through the kernel."""
    Kd, g, N = 192, 64, 64
    x = torch.zeros(1, Kd, dtype=torch.int8)
    w = torch.zeros(1, N, Kd, dtype=torch.int8)
    for grp in range(3):
        x[0, 64 * grp] = 1
        w[0, :, 64 * grp] = 1
    w4 = K.format_cast_nz_int4(w.to(DEV), 0, N, Kd)
    one = torch.tensor([1], dtype=torch.int64, device=DEV)
    sx = torch.ones(1, device=DEV)
    for scales, want in (((2.0 ** 24, 1.0, 1.0), 2.0 ** 24), ((1.0, 1.0, 2.0 ** 24), 2.0 ** 24 + 2)):
        sg = torch.tensor(scales, dtype=torch.float32).reshape(1, 3, 1).expand(1, 3, N).contiguous()
        ref = orc.gmm_w4_grouped(x.numpy(), w.numpy(), sg.numpy(), np.array([1], dtype=np.int64), g)
        assert np.all(ref == np.float32(want))
        got = K.gmm2_dequant_w4(x.to(DEV), w4, sg.to(DEV), g, sx, one, 0, N, Kd)
        torch.cuda.synchronize()
        assert np.array_equal(bits(got.cpu()), orc.w4_rows_to_bf16(ref, np.ones(1, dtype=np.float32)))


# streaming / LDS-tiled / 256-row weight-streaming kernel
@pytest.mark.parametrize("R,E,Kd,N", [(24, 8, 256, 128), (sum(TILE_COUNTS), len(TILE_COUNTS), 256, 256),
                                      (sum(TILE_COUNTS), len(TILE_COUNTS), 4096, 128)])
def test_gmm1_swiglu_clamp(K, orc, R, E, Kd, N):
    """swiglu_limit > 0: gate <= L, up in [-L, L] before the activation (the reference's clamp,
    csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:461-485)."""
    print(f"gmm1 clamp R={R} E={E} K={Kd} N={N}", flush=True)
    from vllm_ascend_amd._lib import W_ENK

    g = torch.Generator().manual_seed(R + 5)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    cnt = torch.tensor(TILE_COUNTS, dtype=torch.int64) if R == sum(TILE_COUNTS) else _rand_groups(g, E, R)
    cum = torch.cumsum(cnt, 0)
    f = orc.dequant_acc(orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy()), sx.numpy(), sw.numpy(), cum.numpy())
    limit = float(np.percentile(np.abs(f), 60))  # bites on a large share of the values
    q_want, s_want = orc.swiglu_quant(f, swiglu_limit=limit)
    q_free, _ = orc.swiglu_quant(f)
    assert not np.array_equal(q_want, q_free)
    q, s = K.gmm1_swiglu_quant(x.to(DEV), K.format_cast_nz(w.to(DEV), W_ENK), sw.to(DEV), sx.to(DEV), cum.to(DEV), 0,
                               N, Kd, swiglu_limit=limit)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


def test_w4_gmm1_swiglu_clamp(K, orc):
    Kd, N, gsz = 256, 128, 128
    g = torch.Generator().manual_seed(77)
    cnt = torch.tensor(W4_COUNTS, dtype=torch.int64)
    E, R = len(W4_COUNTS), int(cnt.sum())
    cum = torch.cumsum(cnt, 0)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-8, 8, (E, N, Kd), generator=g, dtype=torch.int8)
    sg = torch.rand(E, Kd // gsz, N, generator=g) * 0.09 + 0.01
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    f = orc.scale_rows(orc.gmm_w4_grouped(x.numpy(), w.numpy(), sg.numpy(), cum.numpy(), gsz), sx.numpy())
    limit = float(np.percentile(np.abs(f), 60))
    q_want, s_want = orc.swiglu_quant(f, swiglu_limit=limit)
    q, s = K.gmm1_swiglu_quant_w4(x.to(DEV), K.format_cast_nz_int4(w.to(DEV), 0, N, Kd), sg.to(DEV), gsz, sx.to(DEV),
                                  cum.to(DEV), 0, N, Kd, swiglu_limit=limit)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


@pytest.mark.parametrize("T,k,E", [(300, 2, 64), (5000, 4, 16), (33, 8, 8)])
def test_init_routing_maximum_skew(K, orc, T, k, E):
    """Every token picks the same k experts (the other experts stay empty): the histogram atomics all collide,
    and the stable order inside an expert is the flat (token, slot) order."""
    print(f"init_routing skew T={T} k={k} E={E}", flush=True)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, 64, generator=g).to(torch.bfloat16)
    hot = torch.randperm(E, generator=g)[:k].to(torch.int32)
    ids = hot.repeat(T, 1).contiguous()
    xs, dst, cnt, sx = K.init_routing(x.to(DEV), ids.to(DEV), E, 1, 1)
    torch.cuda.synchronize()
    xo, do, co, so = orc.init_routing(bits(x), ids.numpy(), E, quant=True)
    assert np.array_equal(dst.cpu().numpy(), do) and np.array_equal(cnt.cpu().numpy(), co)
    assert np.array_equal(bits(xs), xo) and np.array_equal(sx.cpu().numpy().view(np.uint32), so.view(np.uint32))
    assert sorted(co.tolist())[-k:] == [T] * k and int(co.sum()) == T * k


def test_grouped_gemms_with_one_expert_owning_every_row(K, orc):
    """Maximum skew for the GEMMs: one expert in the middle owns all rows, all others are empty
    (both the LDS-tiled and, with few rows, the streaming kernel)."""
    from vllm_ascend_amd._lib import W_ENK

    for R in (20, 900):
        E, Kd, N = 8, 256, 128
        g = torch.Generator().manual_seed(R)
        x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
        w = torch.randint(-127, 128, (E, N, Kd), generator=g, dtype=torch.int8)
        sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
        sx = torch.rand(R, generator=g) * 0.05 + 0.001
        cnt = torch.zeros(E, dtype=torch.int64)
        cnt[5] = R
        cum = torch.cumsum(cnt, 0)
        wnz = K.format_cast_nz(w.to(DEV), W_ENK)
        ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
        assert np.array_equal(K.gmm_i32(x.to(DEV), wnz, cnt.to(DEV), 1, N, Kd).cpu().numpy(), ref)
        got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd)
        assert np.array_equal(bits(got.cpu()), orc.gmm2_dequant(ref, sx.numpy(), sw.numpy(), cum.numpy()))
        q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw.numpy(), cum.numpy()))
        q, s = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt.to(DEV), 1, N, Kd)
        torch.cuda.synchronize()
        assert np.array_equal(q.cpu().numpy(), q_want)
        assert np.array_equal(s.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


# Seeded random problems around the borders of the kernel choice (average rows per expert 47 / 48 / 95 / 96 / 192 /
# 193 / 256 / 257, K 960 / 1024 / 4032 / 4096) with skewed group sizes: all three epilogues of whichever kernel
# the library picks.
def _random_gemm_problem(seed):
    rng = np.random.default_rng(seed)
    E = int(rng.integers(1, 13))
    avg = int(rng.choice([3, 30, 47, 48, 49, 95, 96, 100, 150, 192, 193, 200, 256, 257, 400]))
    Kd = int(rng.choice([64, 192, 512, 960, 1024, 2048, 4032, 4096, 4160]))
    N = int(rng.choice([64, 128, 320, 576]))
    R = max(1, E * avg + int(rng.integers(0, E)))
    w = rng.random(E) ** 3                      # a few experts take most rows
    if E > 2:
        w[rng.permutation(E)[: E // 3]] = 0
    if w.sum() == 0:
        w[0] = 1
    cnt = np.floor(w / w.sum() * R).astype(np.int64)
    cnt[int(np.argmax(w))] += R - cnt.sum()
    return E, R, Kd, N, cnt


@pytest.mark.parametrize("seed", range(24))
def test_grouped_gemms_on_random_problems(K, orc, seed):
    from vllm_ascend_amd._lib import W_ENK

    E, R, Kd, N, cnt = _random_gemm_problem(seed)
    print(f"random gemm seed={seed} E={E} R={R} K={Kd} N={N} counts={cnt.tolist()}", flush=True)
    g = torch.Generator().manual_seed(1000 + seed)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    cnt_t = torch.from_numpy(cnt)
    cum = torch.cumsum(cnt_t, 0)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    acc = K.gmm_i32(x.to(DEV), wnz, cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)
    want = orc.gmm2_dequant(ref, sx.numpy(), sw.numpy(), cum.numpy())
    got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt_t.to(DEV), 1, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)
    limit = 0.0 if seed % 3 else 1.5
    q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw.numpy(), cum.numpy()), swiglu_limit=limit)
    q, s_ = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd, swiglu_limit=limit)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s_.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


# Fewer rows than experts (a decode batch of a few tokens on the sorted path): the grid has a slot per row and a
# workgroup looks up the expert of its slot in the group list.  Random histograms with most experts empty.
@pytest.mark.parametrize("seed", range(10))
def test_grouped_gemms_with_fewer_rows_than_experts(K, orc, seed):
    from vllm_ascend_amd._lib import W_ENK

    rng = np.random.default_rng(500 + seed)
    E = int(rng.integers(2, 320))
    R = int(rng.integers(1, E))
    Kd = int(rng.choice([64, 128, 192, 512, 1024, 2048]))
    N = int(rng.choice([64, 128, 320, 576]))
    cnt = np.zeros(E, dtype=np.int64)
    for _ in range(R):
        cnt[int(rng.integers(E)) if rng.random() < 0.7 else int(rng.integers(min(E, 4)))] += 1
    print(f"few rows seed={seed} E={E} R={R} K={Kd} N={N} experts with rows={int((cnt > 0).sum())}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = torch.randint(-128, 128, (R, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (E, N, Kd), generator=g, dtype=torch.int8)
    sw = torch.rand(E, N, generator=g) * 0.009 + 0.001
    sx = torch.rand(R, generator=g) * 0.05 + 0.001
    cnt_t = torch.from_numpy(cnt)
    cum = torch.cumsum(cnt_t, 0)
    wnz = K.format_cast_nz(w.to(DEV), W_ENK)
    ref = orc.gmm_i32(x.numpy(), w.numpy(), cum.numpy())
    acc = K.gmm_i32(x.to(DEV), wnz, cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)
    want = orc.gmm2_dequant(ref, sx.numpy(), sw.numpy(), cum.numpy())
    got = K.gmm2_dequant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cnt_t.to(DEV), 1, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(got.cpu()), want)
    q_want, s_want = orc.swiglu_quant(orc.dequant_acc(ref, sx.numpy(), sw.numpy(), cum.numpy()))
    q, s_ = K.gmm1_swiglu_quant(x.to(DEV), wnz, sw.to(DEV), sx.to(DEV), cum.to(DEV), 0, N, Kd)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_want)
    assert np.array_equal(s_.cpu().numpy().view(np.uint32), s_want.view(np.uint32))


# The expert MLP of a decode batch in pair order (no sort): every stage against the sorted form of the checker,
# rows moved to pair order through the checker's own expanded_row_idx.
@pytest.mark.parametrize("T,k,E,H,I", [(64, 8, 128, 2048, 768), (8, 8, 128, 2048, 768), (48, 8, 128, 2048, 768),
                                       (40, 8, 256, 1024, 256), (1, 1, 8, 64, 32),
                                       (128, 8, 64, 512, 128), (33, 6, 96, 256, 96), (64, 8, 256, 1024, 256),
                                       (100, 4, 256, 128, 64), (300, 2, 16, 192, 160)])
def test_expert_mlp_in_pair_order(K, orc, T, k, E, H, I):
    from vllm_ascend_amd._lib import W_ENK

    print(f"pair order T={T} k={k} E={E} H={H} I={I}", flush=True)
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if E >= 8:
        ids[:, 0] = ids[0, 0]  # one popular expert: more than 32 rows (several passes) when T allows
    tw = torch.rand(T, k, generator=g).to(torch.bfloat16)
    w13 = torch.randint(-128, 128, (E, 2 * I, H), generator=g, dtype=torch.int8)
    w2 = torch.randint(-128, 128, (E, H, I), generator=g, dtype=torch.int8)
    s13 = torch.rand(E, 2 * I, generator=g) * 0.009 + 0.001
    s2 = torch.rand(E, H, generator=g) * 0.009 + 0.001
    # checker, sorted form
    xs_o, dst_o, cnt_o, sx_o = orc.init_routing(bits(x), ids.numpy(), E, quant=True)
    cum = np.cumsum(cnt_o)
    acc1 = orc.gmm_i32(xs_o, w13.numpy(), cum)
    q1_o, s1_o = orc.swiglu_quant(orc.dequant_acc(acc1, sx_o, s13.numpy(), cum))
    acc2 = orc.gmm_i32(q1_o, w2.numpy(), cum)
    y2_o = orc.gmm2_dequant(acc2, s1_o, s2.numpy(), cum)
    out_o = orc.unpermute(y2_o, dst_o, bits(tw))
    # GPU, pair order
    xq, xsc = K.dynamic_quant(x.to(DEV))
    w13nz, w2nz = K.format_cast_nz(w13.to(DEV), W_ENK), K.format_cast_nz(w2.to(DEV), W_ENK)
    q1, s1 = K.gmm1_swiglu_quant_pairs(xq, xsc, ids.to(DEV), w13nz, s13.to(DEV), 2 * I, H)
    y2 = K.gmm2_dequant_pairs(q1, w2nz, s2.to(DEV), s1, ids.to(DEV), H, I)
    out, cnt = K.token_unpermute_pairs(y2, tw.to(DEV), ids.to(DEV), E)
    torch.cuda.synchronize()
    dst = dst_o.astype(np.int64)
    assert np.array_equal(q1.cpu().numpy(), q1_o[dst])
    assert np.array_equal(s1.cpu().numpy().view(np.uint32), s1_o[dst].view(np.uint32))
    assert np.array_equal(bits(y2.cpu()), y2_o[dst])
    assert np.array_equal(bits(out.cpu()), out_o)
    assert np.array_equal(cnt.cpu().numpy(), cnt_o)
    if K.gmm2_requant_pairs_supported(T, k, H, I, E):
        # the form of four launches: fp32 SwiGLU values out of the first GEMM, re-quantised inside the second
        _, _, y_o = orc.swiglu_quant(orc.dequant_acc(acc1, sx_o, s13.numpy(), cum), want_y=True)
        y = K.gmm1_swiglu_pairs(xq, xsc, ids.to(DEV), w13nz, s13.to(DEV), 2 * I, H)
        y2f = K.gmm2_requant_dequant_pairs(y, w2nz, s2.to(DEV), ids.to(DEV), H, I)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), y_o[dst].view(np.uint32))
        assert np.array_equal(bits(y2f.cpu()), y2_o[dst])
    if T >= 8:
        # dropped pairs (ids outside the range): nobody computes them, the combine and the counts leave them out
        bad = ids.clone()
        bad[1, 0], bad[3, k - 1] = E, -1
        xs_b, dst_b, cnt_b, sx_b = orc.init_routing(bits(x), bad.numpy(), E, quant=True)
        cum_b = np.cumsum(cnt_b)
        q1_b, s1_b = orc.swiglu_quant(orc.dequant_acc(orc.gmm_i32(xs_b, w13.numpy(), cum_b), sx_b, s13.numpy(), cum_b))
        y2_b = orc.gmm2_dequant(orc.gmm_i32(q1_b, w2.numpy(), cum_b), s1_b, s2.numpy(), cum_b)
        out_b = orc.unpermute(y2_b, dst_b, bits(tw))
        q1, s1 = K.gmm1_swiglu_quant_pairs(xq, xsc, bad.to(DEV), w13nz, s13.to(DEV), 2 * I, H)
        y2 = K.gmm2_dequant_pairs(q1, w2nz, s2.to(DEV), s1, bad.to(DEV), H, I)
        out, cnt = K.token_unpermute_pairs(y2, tw.to(DEV), bad.to(DEV), E)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out.cpu()), out_b)
        assert np.array_equal(cnt.cpu().numpy(), cnt_b)
