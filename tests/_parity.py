"""Parity of one full-size layer pass against the CPU checker, shared by the full-size GPU tests and by the
benchmark's parity block.

The whole batch goes through the checker where that is cheap (routing, permutation, histogram, the first
quantisation: a few hundred MB of byte work).  The grouped GEMMs are checked on a SAMPLE of rows: after the dispatch
the rows of this path never interact, so a row's int32 accumulators, its int8 SwiGLU output, its scale and its
16-bit expert output can be recomputed by the checker from that row alone, and a token's final output from its k
rows.  The sample holds the k rows of a few tokens plus rows at the start, the end and the tile borders of expert
ranges."""
from __future__ import annotations

import numpy as np
import torch

from _inputs import LayerCfg, bits, gating_kwargs


def to_cpu(d: dict) -> dict:
    return {k: v.cpu() for k, v in d.items()}


def staged_run(K, cfg: LayerCfg, dg: dict, want_acc: bool = True) -> dict:
    """The layer stage by stage through the tensor-level launchers (the calls the plugin path makes), keeping every
    intermediate on the GPU.  dg: the layer's tensors on the GPU."""
    from vllm_ascend_amd._lib import W_ENK

    kw = gating_kwargs(cfg)
    x, logits = dg["x"], dg["logits"]
    y, ids, _ = K.gating_top_k(logits, kw["k"], kw["k_group"], kw["group_count"], 1, kw["renorm"], kw["norm_type"],
                               False, kw["routed_scaling_factor"], kw["eps"], dg["bias"] if cfg.bias else None)
    w_half = y.to(x.dtype)
    xs, dst, cnt, sx = K.init_routing(x, ids, cfg.E, 1, 1)
    acc1 = acc2 = None
    if cfg.w4_group >= 0:
        g = cfg.w4_group
        w13 = K.format_cast_nz_int4(dg["w13"], 0, 2 * cfg.I, cfg.H)
        w2 = K.format_cast_nz_int4(dg["w2"], 0, cfg.H, cfg.I)
        sg13 = dg["s13"].transpose(1, 2).contiguous()   # [E, N, G] -> [E, G, N]
        sg2 = dg["s2"].transpose(1, 2).contiguous()
        g13 = g if g else cfg.H
        g2 = g if g else cfg.I
        q1, s1 = K.gmm1_swiglu_quant_w4(xs, w13, sg13, g13, sx, cnt, 1, 2 * cfg.I, cfg.H)
        o = K.gmm2_dequant_w4(q1, w2, sg2, g2, s1, cnt, 1, cfg.H, cfg.I)
    else:
        w13 = K.format_cast_nz(dg["w13"], W_ENK)
        w2 = K.format_cast_nz(dg["w2"], W_ENK)
        q1, s1 = K.gmm1_swiglu_quant(xs, w13, dg["s13"], sx, cnt, 1, 2 * cfg.I, cfg.H)
        o = K.gmm2_dequant(q1, w2, dg["s2"], s1, cnt, 1, cfg.H, cfg.I)
        if want_acc:
            acc1 = K.gmm_i32(xs, w13, cnt, 1, 2 * cfg.I, cfg.H)
            acc2 = K.gmm_i32(q1, w2, cnt, 1, cfg.H, cfg.I)
    del w13, w2
    out = K.token_unpermute(o, dst, w_half)
    torch.cuda.synchronize()
    return dict(x=x, ids=ids, w=w_half, xs=xs, dst=dst, cnt=cnt, sx=sx, acc1=acc1, q1=q1, s1=s1, acc2=acc2, o=o,
                out=out)


def sample_rows(counts: np.ndarray, rng, dst: np.ndarray, tokens: np.ndarray, k: int, border_experts: int = 8):
    """Rows of the sampled tokens, plus the first, the last and one inner row of every non-empty expert and the
    64 / 128 / 160 / 256-row tile borders of the first experts."""
    cum = np.cumsum(counts)
    rows = set()
    for t in tokens:
        rows.update(int(r) for r in dst[t * k:(t + 1) * k])
    for e, m in enumerate(counts):
        if m == 0:
            continue
        lo = int(cum[e] - m)
        rows.update({lo, int(cum[e]) - 1, lo + int(rng.integers(0, m))})
        if e < border_experts:
            rows.update(lo + b for b in (63, 64, 127, 128, 159, 160, 255, 256) if b < m)
    return np.array(sorted(rows), dtype=np.int64)


def dense_reference_tokens(orc, cfg: LayerCfg, dc: dict, x_tok: np.ndarray, w_tok: np.ndarray, ids_tok: np.ndarray):
    """The layer without any activation quantisation for a few tokens: weights dequantised (int x scale), the two
    matrix products in fp32 (products of an int8 weight and a 16-bit activation are exact there), activation,
    routing weights and the sum over experts in float64.  The tolerance reference of the 16-bit output.
    x_tok [n, H] and w_tok [n, k] as fp32 values."""
    n, k = ids_tok.shape
    out = np.zeros((n, cfg.H), dtype=np.float64)
    xf = np.ascontiguousarray(x_tok, dtype=np.float32)
    w13, w2, s13, s2 = dc["w13"].numpy(), dc["w2"].numpy(), dc["s13"].numpy(), dc["s2"].numpy()
    g = cfg.w4_group

    def mlp(x_rows, w_up, s_up, w_down, s_down):
        if g >= 0:  # int4 weights: scales [N, G], one per group of values along K (one group: per channel)
            wu = w_up.astype(np.float32) * np.repeat(s_up, w_up.shape[1] // s_up.shape[1], axis=1)
            wd = w_down.astype(np.float32) * np.repeat(s_down, w_down.shape[1] // s_down.shape[1], axis=1)
            gu = (x_rows @ wu.T).astype(np.float64)
        else:
            gu = (x_rows @ w_up.astype(np.float32).T).astype(np.float64) * s_up.astype(np.float64)[None, :]
        half = gu.shape[1] // 2
        gate, up = gu[:, :half], gu[:, half:]
        act = (gate / (1.0 + np.exp(-gate)) * up).astype(np.float32)
        if g >= 0:
            return (act @ wd.T).astype(np.float64)
        return (act @ w_down.astype(np.float32).T).astype(np.float64) * s_down.astype(np.float64)[None, :]

    for e in np.unique(ids_tok):
        tok, slot = np.nonzero(ids_tok == e)
        o = mlp(xf[tok], w13[e], s13[e], w2[e], s2[e])
        np.add.at(out, tok, o * w_tok[tok, slot].astype(np.float64)[:, None])
    if cfg.shared and "sw13" in dc:
        g = -1  # the shared expert is int8 per channel
        out += mlp(xf, dc["sw13"][0].numpy(), dc["ss13"][0].numpy(), dc["sw2"][0].numpy(), dc["ss2"][0].numpy())
    return out


def layer_parity(orc, cfg: LayerCfg, dc: dict, r: dict, n_tokens: int = 8, seed: int = 1, layer_out=None,
                 shared: bool = False, full_dispatch: bool = True) -> dict:
    """Compare the GPU intermediates `r` (staged_run) with the checker.  dc: the layer's tensors on the CPU.
    layer_out: the final output of the plugin path (layer.forward_impl) for the same batch, when given it is what
    the sampled tokens' outputs are compared with (with the shared expert's output added when `shared`).
    Returns a dict of findings; `failed` lists the gates that did not hold."""
    res: dict = {}
    failed = []

    def gate(name, ok):
        res[name] = bool(ok)
        if not ok:
            failed.append(name)

    T, k, E = cfg.T, cfg.k, cfg.E
    R = T * k
    kw = gating_kwargs(cfg)
    # ---- routing: whole batch
    y, ids_want, _ = orc.gating_top_k(dc["logits"].numpy(), k, bias=dc["bias"].numpy() if cfg.bias else None,
                                      k_group=kw["k_group"], group_count=kw["group_count"], group_select_mode=1,
                                      renorm=kw["renorm"], norm_type=kw["norm_type"],
                                      routed_scaling_factor=kw["routed_scaling_factor"], x_dtype="f32")
    w_want = orc.f32_to_half(y)
    ids = r["ids"].cpu().numpy()
    gate("ids_bit_exact", np.array_equal(ids, ids_want))
    gate("topk_weights_bit_exact", np.array_equal(bits(r["w"]), w_want))
    # ---- dispatch: whole batch
    dst = r["dst"].cpu().numpy()
    cnt = r["cnt"].cpu().numpy()
    x_bits = bits(dc["x"])
    if full_dispatch:
        xs_want, dst_want, cnt_want, sx_want = orc.init_routing(x_bits, ids_want, E, quant=True)
        gate("permutation_bit_exact", np.array_equal(dst, dst_want))
        gate("expert_tokens_bit_exact", np.array_equal(cnt, cnt_want))
        gate("xs_int8_bit_exact", np.array_equal(r["xs"].cpu().numpy(), xs_want))
        gate("xs_scale_bit_exact", np.array_equal(r["sx"].cpu().numpy().view(np.uint32), sx_want.view(np.uint32)))
        del xs_want
    else:
        flat = ids_want.reshape(-1).astype(np.int64)
        gate("permutation_bit_exact", np.array_equal(dst, np.argsort(np.argsort(flat, kind="stable"), kind="stable")))
        gate("expert_tokens_bit_exact", np.array_equal(cnt, np.bincount(flat, minlength=E)))
    # ---- grouped GEMMs: sampled rows
    rng = np.random.default_rng(seed)
    tokens = np.unique(rng.integers(0, T, size=n_tokens))
    rows = sample_rows(cnt, rng, dst.astype(np.int64), tokens, k)
    expert_of_row = np.searchsorted(np.cumsum(cnt), rows, side="right")
    cum_s = np.cumsum(np.bincount(expert_of_row, minlength=E)).astype(np.int64)
    rows_t = torch.from_numpy(rows).to(r["xs"].device)
    xs_s = r["xs"][rows_t].cpu().numpy()
    sx_s = r["sx"][rows_t].cpu().numpy()
    w13, w2 = dc["w13"].numpy(), dc["w2"].numpy()
    acc2_want = None
    if cfg.w4_group >= 0:
        g13 = cfg.w4_group if cfg.w4_group else cfg.H
        g2 = cfg.w4_group if cfg.w4_group else cfg.I
        sg13 = np.ascontiguousarray(dc["s13"].numpy().transpose(0, 2, 1))
        sg2 = np.ascontiguousarray(dc["s2"].numpy().transpose(0, 2, 1))
        f1 = orc.scale_rows(orc.gmm_w4_grouped(xs_s, w13, sg13, cum_s, g13), sx_s)
        q_want, s_want = orc.swiglu_quant(f1)
        f2 = orc.gmm_w4_grouped(q_want, w2, sg2, cum_s, g2)
        o_want = orc.w4_rows_to_bf16(f2, s_want)
        res["acc1_int32_bit_exact"] = res["acc2_int32_bit_exact"] = None  # per-group fp32 partial sums, no int32 tensor
    else:
        acc1_want = orc.gmm_i32(xs_s, w13, cum_s)
        q_want, s_want = orc.swiglu_quant(orc.dequant_acc(acc1_want, sx_s, dc["s13"].numpy(), cum_s))
        acc2_want = orc.gmm_i32(q_want, w2, cum_s)
        o_want = orc.gmm2_dequant(acc2_want, s_want, dc["s2"].numpy(), cum_s)
        if r.get("acc1") is not None:
            gate("acc1_int32_bit_exact", np.array_equal(r["acc1"][rows_t].cpu().numpy(), acc1_want))
            gate("acc2_int32_bit_exact", np.array_equal(r["acc2"][rows_t].cpu().numpy(), acc2_want))
    gate("q1_int8_bit_exact", np.array_equal(r["q1"][rows_t].cpu().numpy(), q_want))
    gate("q1_scale_bit_exact", np.array_equal(r["s1"][rows_t].cpu().numpy().view(np.uint32), s_want.view(np.uint32)))
    gate("expert_out_bit_exact", np.array_equal(bits(r["o"][rows_t]), o_want))
    res["rows_sampled"] = int(rows.size)
    # ---- combine (and the shared expert): sampled tokens, from the checker's own rows
    pos = {int(rw): i for i, rw in enumerate(rows)}
    tok_rows = np.array([[pos[int(dst[t * k + j])] for j in range(k)] for t in tokens])
    x_tok_bits = x_bits[tokens]
    add = None
    if shared and cfg.shared:
        add = orc.shared_expert_forward(x_tok_bits, dc["sw13"][0].numpy(), dc["ss13"][0].numpy(),
                                        dc["sw2"][0].numpy(), dc["ss2"][0].numpy())
    out_want = np.stack([
        orc.unpermute(o_want[tok_rows[i]], np.arange(k, dtype=np.int32), w_want[t:t + 1],
                      add[i:i + 1] if add is not None else None)[0] for i, t in enumerate(tokens)])
    final = layer_out if layer_out is not None else r["out"]
    tok_t = torch.from_numpy(tokens).to(final.device)
    got_bits = bits(final[tok_t])
    gate("output_bit_exact", np.array_equal(got_bits, out_want))
    res["tokens_sampled"] = int(tokens.size)
    # ---- tolerance of the 16-bit output on the sampled tokens
    got = orc.half_to_f32(got_bits).astype(np.float64)
    x_tok = orc.half_to_f32(x_tok_bits)
    w_tok = orc.half_to_f32(w_want[tokens])
    ref = dense_reference_tokens(orc, cfg if shared else _without_shared(cfg), dc, x_tok, w_tok, ids_want[tokens])
    res["rel_err_vs_fp32_dequant_reference"] = float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))
    res["max_abs_err_vs_fp32_dequant_reference"] = float(np.abs(got - ref).max())
    if acc2_want is not None and not (shared and cfg.shared):
        # the same quantised pipeline with the floating-point tail in float64 and no 16-bit rounding
        s2 = dc["s2"].numpy().astype(np.float64)
        o64 = acc2_want.astype(np.float64) * s_want.astype(np.float64)[:, None] * s2[expert_of_row]
        ref_q = (o64[tok_rows] * w_tok.astype(np.float64)[:, :, None]).sum(axis=1)
        res["rel_err_vs_quantized_fp64_reference"] = float(np.linalg.norm(got - ref_q) /
                                                           max(np.linalg.norm(ref_q), 1e-30))
        res["max_abs_err_vs_quantized_fp64_reference"] = float(np.abs(got - ref_q).max())
    if cfg.w4_group < 0:
        # where that error comes from: the reference's golden math in numpy (no checker code) on the same tokens,
        # routed experts only, with the first / the second / both activation quantisers in place
        from _noise import error_split

        sp = error_split(x_tok, w_tok, ids_want[tokens], w13, dc["s13"].numpy(), w2, dc["s2"].numpy())
        res["rel_err_split_routed_experts_golden_math"] = {
            "first_quant_only": sp["first_quant_only"], "second_quant_only": sp["second_quant_only"],
            "both": sp["both"]}
    res["failed"] = failed
    return res


def _without_shared(cfg: LayerCfg) -> LayerCfg:
    import dataclasses

    return dataclasses.replace(cfg, shared=False)
