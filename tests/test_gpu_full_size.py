"""Parity at the full sizes of the benchmark configurations, where the CPU checker cannot redo the whole
layer in test time: properties that do not depend on the size (permutation, sortedness, histogram, quantiser
round trip, linearity of the combine, run-to-run identity) plus bit-exact parity of a SAMPLE of rows — the
rows of this path never interact after the dispatch, so a row's int8 SwiGLU output, its scale and its bf16
expert output can be recomputed by the checker from that row alone."""
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


def _sample_rows(counts: np.ndarray, rng, per_expert=3):
    """Rows at the start, the end and inside of every non-empty expert's range, plus the 128- and 64-row tile
    borders of the first experts."""
    cum = np.cumsum(counts)
    rows = []
    for e, m in enumerate(counts):
        if m == 0:
            continue
        lo = cum[e] - m
        pick = {lo, cum[e] - 1, lo + int(rng.integers(0, m))}
        if e < 8:
            pick |= {lo + b for b in (63, 64, 127, 128) if b < m}
        rows += sorted(pick)[: per_expert + 4]
    return np.array(sorted(set(rows)), dtype=np.int64)


def _run_full(K, orc, cfg, seed=0):
    d = make_layer(cfg, seed=seed)
    from vllm_ascend_amd._lib import W_ENK

    kw = gating_kwargs(cfg)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    y, ids, _ = K.gating_top_k(logits, kw["k"], kw["k_group"], kw["group_count"], 1, kw["renorm"], kw["norm_type"],
                               False, kw["routed_scaling_factor"], kw["eps"],
                               d["bias"].to(DEV) if cfg.bias else None)
    w_bf16 = y.to(torch.bfloat16)
    xs, dst, cnt, sx = K.init_routing(x, ids, cfg.E, 1, 1)
    if cfg.w4_group >= 0:
        g = cfg.w4_group
        w13 = K.format_cast_nz_int4(d["w13"].to(DEV), 0, 2 * cfg.I, cfg.H)
        w2 = K.format_cast_nz_int4(d["w2"].to(DEV), 0, cfg.H, cfg.I)
        sg13 = d["s13"].transpose(1, 2).contiguous().to(DEV)   # [E, N, G] -> [E, G, N]
        sg2 = d["s2"].transpose(1, 2).contiguous().to(DEV)
        q1, s1 = K.gmm1_swiglu_quant_w4(xs, w13, sg13, g, sx, cnt, 1, 2 * cfg.I, cfg.H)
        o = K.gmm2_dequant_w4(q1, w2, sg2, g, s1, cnt, 1, cfg.H, cfg.I)
    else:
        w13 = K.format_cast_nz(d["w13"].to(DEV), W_ENK)
        w2 = K.format_cast_nz(d["w2"].to(DEV), W_ENK)
        s13, s2 = d["s13"].to(DEV), d["s2"].to(DEV)
        q1, s1 = K.gmm1_swiglu_quant(xs, w13, s13, sx, cnt, 1, 2 * cfg.I, cfg.H)
        o = K.gmm2_dequant(q1, w2, s2, s1, cnt, 1, cfg.H, cfg.I)
    out = K.token_unpermute(o, dst, w_bf16)
    torch.cuda.synchronize()
    return d, dict(x=x, ids=ids, w=w_bf16, xs=xs, dst=dst, cnt=cnt, sx=sx, q1=q1, s1=s1, o=o, out=out)


@pytest.mark.parametrize("name", ["c3_qwen3_prefill", "c4_dsv3_reduced", "c5_w4a8_reduced"])
def test_full_size_properties_and_sampled_rows(K, orc, name):
    import dataclasses

    if name == "c4_dsv3_reduced":
        # DeepSeek-V3's real K and N (7168 / 2 x 2048) and its rows per expert (about 128), with 16 of the 256
        # experts so that the weights fit a test (0.7 GB instead of 11 GB)
        cfg = dataclasses.replace(CONFIGS["c4_dsv3_prefill"], name=name, T=256, E=16, n_group=4, topk_group=2,
                                  shared=False)
    elif name == "c5_w4a8_reduced":
        # the W4A8 configuration's real K, N, group size and Zipf skew with 16 of its 256 experts
        cfg = dataclasses.replace(CONFIGS["c5_w4a8_zipf"], name=name, E=16, n_group=4, topk_group=2)
    else:
        cfg = CONFIGS[name]
    print(f"full size {name}: T={cfg.T} E={cfg.E} H={cfg.H} I={cfg.I}", flush=True)
    d, r = _run_full(K, orc, cfg)
    R = cfg.T * cfg.k
    ids = r["ids"].cpu().numpy()
    dst = r["dst"].cpu().numpy().astype(np.int64)
    cnt = r["cnt"].cpu().numpy()

    # ---- dispatch: a permutation, sorted by expert, stable, with the right histogram
    assert np.array_equal(np.sort(dst), np.arange(R))
    flat = ids.reshape(-1).astype(np.int64)
    assert np.array_equal(cnt, np.bincount(flat, minlength=cfg.E))
    expert_of_row = np.empty(R, dtype=np.int64)
    expert_of_row[dst] = flat
    assert np.all(np.diff(expert_of_row) >= 0)                      # rows sorted by expert
    src_of_row = np.empty(R, dtype=np.int64)
    src_of_row[dst] = np.arange(R)
    same = np.diff(expert_of_row) == 0
    assert np.all(np.diff(src_of_row)[same] > 0)                    # stable inside an expert
    assert np.array_equal(dst, np.argsort(np.argsort(flat, kind="stable"), kind="stable"))

    # ---- quantiser round trip on every row: |x - q*s| <= s/2 (+ bf16-exact inputs), scale = absmax / 127
    xs, sx = r["xs"], r["sx"]
    tok_of_row = torch.from_numpy(src_of_row // cfg.k).to(DEV)
    xf = r["x"].float()[tok_of_row]
    amax = xf.abs().amax(dim=1).cpu().numpy()          # exact: a maximum of bf16 values
    assert np.array_equal(sx.cpu().numpy(), amax / np.float32(127.0))   # IEEE fp32 division on the host
    err = (xs.float() * sx[:, None] - xf).abs()
    assert bool((err <= sx[:, None] * 0.50001).all())
    del xf, err

    # ---- sampled rows, bit for bit, through the checker (a miniature grouped problem with the same experts)
    rng = np.random.default_rng(1)
    rows = _sample_rows(cnt, rng)
    e_rows = expert_of_row[rows]
    cum_s = np.cumsum(np.bincount(e_rows, minlength=cfg.E)).astype(np.int64)
    rows_t = torch.from_numpy(rows).to(DEV)
    xs_s = xs[rows_t].cpu().numpy()
    sx_s = sx[rows_t].cpu().numpy()
    if cfg.w4_group >= 0:
        sg13 = np.ascontiguousarray(d["s13"].numpy().transpose(0, 2, 1))
        sg2 = np.ascontiguousarray(d["s2"].numpy().transpose(0, 2, 1))
        f1 = orc.scale_rows(orc.gmm_w4_grouped(xs_s, d["w13"].numpy(), sg13, cum_s, cfg.w4_group), sx_s)
        q_want, s_want = orc.swiglu_quant(f1)
        o_want = orc.w4_rows_to_bf16(orc.gmm_w4_grouped(q_want, d["w2"].numpy(), sg2, cum_s, cfg.w4_group), s_want)
    else:
        acc1 = orc.gmm_i32(xs_s, d["w13"].numpy(), cum_s)
        q_want, s_want = orc.swiglu_quant(orc.dequant_acc(acc1, sx_s, d["s13"].numpy(), cum_s))
        o_want = orc.gmm2_dequant(orc.gmm_i32(q_want, d["w2"].numpy(), cum_s), s_want, d["s2"].numpy(), cum_s)
    assert np.array_equal(r["q1"][rows_t].cpu().numpy(), q_want)
    assert np.array_equal(r["s1"][rows_t].cpu().numpy().view(np.uint32), s_want.view(np.uint32))
    assert np.array_equal(bits(r["o"][rows_t]), o_want)

    # ---- combine: sampled tokens recomputed from their k expert rows; linear in the routing weights
    toks = np.unique(rng.integers(0, cfg.T, size=48))
    o_cpu = {}
    for t in toks:
        rr = dst[t * cfg.k:(t + 1) * cfg.k]
        o_cpu[t] = bits(r["o"][torch.from_numpy(rr).to(DEV)])
    w_bits = bits(r["w"])
    for t in toks:
        want = orc.unpermute(o_cpu[t], np.arange(cfg.k, dtype=np.int32), w_bits[t:t + 1])
        assert np.array_equal(bits(r["out"][int(t):int(t) + 1]), want)
    out2 = K.token_unpermute(r["o"], r["dst"], (r["w"].float() * 2).to(torch.bfloat16))
    assert torch.equal(out2.float(), r["out"].float() * 2)

    # ---- a second run gives the same bits
    _, r2 = _run_full(K, orc, cfg)
    for key in ("dst", "xs", "q1", "s1", "o", "out"):
        assert torch.equal(r[key], r2[key]), key
