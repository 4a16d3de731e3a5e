"""Torch-native CPU rendering of the W8A8-dynamic (and W4A8) MoE layer, for the benchmark's CPU baseline.

Test infrastructure, like the rest of this folder: only ``bench.py``'s ``cpu_baseline`` leg and the tests import it;
the product never does.  It restates the reference's semantics with plain torch CPU operators, the way the
reference's own golden functions do:
  routing        softmax / sigmoid, bias for selection only, group score = sum of the top 2, top-k, renorm
                 (tests/e2e/nightly/single_node/ops/singlecard_ops/test_npu_moe_gating_top_k.py:33-112)
  dispatch       stable sort of the flattened expert ids (vllm_ascend/lora/fused_moe.py:190-204)
  quantiser      scale = absmax / 127, q = round(x / scale)   [the rule this build fixes]
  expert MLP     torch.matmul on int32 tensors (exact; torch has no int8 x int8 -> int32 CPU GEMM), fp32 scales,
                 x * sigmoid(x) * up, 127 / max re-quantisation
                 (tests/e2e/nightly/single_node/ops/singlecard_ops/test_gmm_swiglu_quant_weight_nz_tensor_list.py:14-55)
  combine        fp32 index_add of the weighted 16-bit expert rows
                 (tests/e2e/nightly/single_node/ops/singlecard_ops/test_fused_moe.py:85-97)
It is NOT bit-identical to the CPU checker (torch's exp and the golden's 127 / max differ from the fixed
operation sequence in the last place); the benchmark reports how close the two are on the rows it ran.
Weights are converted int8 -> int32 once per expert outside the timed sections, as a serving process would at load.
"""
from __future__ import annotations

import time

import torch


def route(logits, k, scoring="softmax", bias=None, n_group=1, topk_group=1, renorm=1, scale=1.0, eps=1e-20):
    x = logits.float()
    p = torch.softmax(x, dim=-1) if scoring == "softmax" else torch.sigmoid(x)
    sel = p + bias.float() if bias is not None else p
    T, E = sel.shape
    if n_group > 1:
        g = sel.view(T, n_group, E // n_group)
        score = g.topk(2, dim=-1).values.sum(-1)
        keep = score.topk(topk_group, dim=-1).indices
        mask = torch.zeros(T, n_group, dtype=torch.bool).scatter_(1, keep, True)
        sel = sel.masked_fill(~mask[:, :, None].expand_as(g).reshape(T, E), float("-inf"))
    ids = torch.sort(sel, dim=-1, descending=True, stable=True).indices[:, :k]
    w = p.gather(1, ids)
    if scoring == "sigmoid" or renorm:
        w = w / (w.sum(-1, keepdim=True) + eps)
    return (w * scale), ids.to(torch.int32)


def quantise(v):
    a = v.abs().amax(dim=-1)
    s = a / 127.0
    q = torch.round(v / s[:, None]).clamp_(-128, 127)
    q = torch.where(a[:, None] > 0, q, torch.zeros_like(q))
    return q.to(torch.int8), torch.where(a > 0, s, torch.zeros_like(s))


def expert_mlp(xq, sx, w13_i32, s13, w2_i32, s2, group=0, out_dtype=torch.bfloat16):
    """Rows of one expert: xq int8 [m, H], sx [m]; weights int32 [2I, H] / [H, I]; per-channel scales [2I] / [H],
    or per-group scales [2I, G] / [H, G] when group > 0.  Returns the 16-bit expert rows [m, H]."""
    def product(a_i8, w_i32, s):
        a = a_i8.to(torch.int32)
        if group > 0:
            f = torch.zeros(a.shape[0], w_i32.shape[0], dtype=torch.float32)
            for gi in range(w_i32.shape[1] // group):
                sl = slice(gi * group, (gi + 1) * group)
                f += torch.matmul(a[:, sl], w_i32[:, sl].T).float() * s[:, gi][None, :]
            return f
        return torch.matmul(a, w_i32.T).float() * s[None, :]

    c = product(xq, w13_i32, s13) * sx[:, None]
    gate, up = c.chunk(2, dim=-1)
    y = gate * torch.sigmoid(gate) * up
    mx = y.abs().amax(dim=-1)
    qscale = 127.0 / mx
    q1 = torch.round(y * qscale[:, None]).clamp_(-128, 127)
    q1 = torch.where(mx[:, None] > 0, q1, torch.zeros_like(q1)).to(torch.int8)
    s1 = torch.where(mx > 0, 1.0 / qscale, torch.zeros_like(mx))
    return (product(q1, w2_i32, s2) * s1[:, None]).to(out_dtype)


def timed_layer(cfg, d, max_rows=2048, max_experts=8, threads=None):
    """One pass of the layer with the expert MLPs run on a SAMPLE of experts (the rows of the busiest few, so the
    rows-per-expert regime is the workload's own up to the row budget) and extrapolated linearly in rows; routing, quantisation,
    dispatch and combine run on the whole batch.  d: the layer's tensors on the CPU (tests/_inputs.make_layer).
    Returns a dict with tokens/s, the timed seconds by part, the sampled rows and their 16-bit expert outputs."""
    if threads:
        torch.set_num_threads(threads)
    x = d["x"].float()
    T, k = cfg.T, cfg.k
    group = cfg.w4_group if cfg.w4_group > 0 else 0
    t = {}
    t0 = time.perf_counter()
    w, ids = route(d["logits"], k, cfg.scoring, d.get("bias") if cfg.bias else None, cfg.n_group, cfg.topk_group,
                   cfg.renorm, cfg.routed_scaling_factor)
    w = w.to(d["x"].dtype)
    xq, sx = quantise(x)
    flat = ids.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices          # sorted row -> flat pair
    row_token = order // k
    counts = torch.bincount(flat, minlength=cfg.E)
    t["front"] = time.perf_counter() - t0
    # ---- sample: the busiest experts first, until the row budget is spent
    cum = torch.cumsum(counts, 0)
    chosen, rows_sample = [], 0  # (expert, rows taken): a hot expert above the budget gives its first rows only
    for e in torch.argsort(counts, descending=True).tolist():
        m = min(int(counts[e]), max_rows - rows_sample)
        if m <= 0 or len(chosen) >= max_experts:
            break
        chosen.append((e, m))
        rows_sample += m
    R = int(counts.sum())
    o = torch.zeros(R, cfg.H, dtype=d["x"].dtype)
    t["experts_sample"] = 0.0
    rows_done = []
    for e, m in chosen:
        lo = int(cum[e] - counts[e])
        hi = lo + m
        w13_i32, w2_i32 = d["w13"][e].to(torch.int32), d["w2"][e].to(torch.int32)  # load-time work: not timed
        s13, s2 = d["s13"][e], d["s2"][e]
        if cfg.w4_group == 0:  # int4 weights with one scale per channel, held as [N, 1]
            s13, s2 = s13[:, 0], s2[:, 0]
        t0 = time.perf_counter()
        tok = row_token[lo:hi]
        o[lo:hi] = expert_mlp(xq[tok], sx[tok], w13_i32, s13, w2_i32, s2, group, d["x"].dtype)
        t["experts_sample"] += time.perf_counter() - t0
        rows_done.append((lo, hi))
        del w13_i32, w2_i32
    t["experts"] = t["experts_sample"] * (R / max(rows_sample, 1))
    t["shared"] = 0.0
    if cfg.shared:
        n = min(T, 256)
        sw13, sw2 = d["sw13"][0].to(torch.int32), d["sw2"][0].to(torch.int32)
        t0 = time.perf_counter()
        expert_mlp(xq[:n], sx[:n], sw13, d["ss13"][0], sw2, d["ss2"][0], 0, d["x"].dtype)
        t["shared"] = (time.perf_counter() - t0) * (T / n)
    t0 = time.perf_counter()
    out = torch.zeros(T, cfg.H, dtype=torch.float32)
    dst = torch.empty_like(order)
    dst[order] = torch.arange(R)
    out.index_add_(0, row_token, o.float() * w.float().reshape(-1)[order][:, None])
    out = out.to(d["x"].dtype)
    t["combine"] = time.perf_counter() - t0
    total = t["front"] + t["experts"] + t["shared"] + t["combine"]
    return {"tokens_per_s": T / total, "seconds": {k_: round(v, 4) for k_, v in t.items()}, "rows_sampled": rows_sample,
            "experts_sampled": len(chosen), "rows": R, "row_ranges": rows_done, "expert_rows": o,
            "threads": torch.get_num_threads(), "ids": ids, "dst": dst}
