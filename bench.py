#!/usr/bin/env python3
"""Benchmark of the W8A8-dynamic fused-MoE layer on one MI355X.

One step = one pass of the whole routed-experts layer (router logits -> final bf16, shared expert included where
the configuration has one) over one batch of synthetic tokens, through the plugin interface
(router.select_experts -> quant_method.apply).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME[,NAME...]] [--mode graph|eager]

Without --workload every configured workload runs in this one process: the DeepSeek-V3-shaped 4096-token prefill
(the largest single-GPU configuration and the shape the target is stated on: the top-level `value`, `ms_per_step`,
`roofline` and `cpu_baseline` are its figures), the Qwen3-30B-A3B-shaped decode and prefill batches, the W4A8
Zipf-routed batch, the DeepSeek-V3-shaped 64-token decode batch and the same shape with int8 weights under
Zipf(1.1)-skewed routing at 512 and 4096 tokens; `workloads` carries the same figures for each.
Inputs are resident in HBM before the timed region (they are drawn on the GPU by a seeded generator).
Per workload:
  ms_per_step   K timed steps (one HIP-graph replay per step) after W warm-up steps
  roofline      the dominant kernel (the gate_up grouped GEMM), timed with HIP events that bracket exactly that kernel
                in every step of a second, eager pass; its name comes from the library
  parity        the bit-exact gates of the layer against the CPU checker (routing ids and weights, permutation,
                histogram and the first int8 quantisation on the whole batch; both int32 accumulators, the int8 SwiGLU
                output, the expert output and the final output on sampled rows / tokens) and the relative error of
                the 16-bit output against a reference without activation quantisation
  cpu_baseline  a torch-native CPU rendering of the layer (torch.matmul on int32 tensors; oracle/torch_native.py) timed
                on this host on a bounded sample of the same batch, with the C checker (OpenMP) beside it as `c_port`
"""
from __future__ import annotations

import argparse
import ctypes
import dataclasses
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA

HEADLINE = "c4_dsv3_prefill"
WORKLOADS = ["c4_dsv3_prefill", "c2_qwen3_decode", "c3_qwen3_prefill", "c5_w4a8_zipf", "c6_dsv3_decode",
             "c7_w8a8_zipf", "c7_w8a8_zipf_4096"]

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc runs (FETCH_SIZE / WRITE_SIZE scaled by a copy
# kernel of known size), taken from the committed summaries: NOT measured in this run.
TRAFFIC_FROM_PROFILES = {
    "c2_qwen3_decode": (401_500_000, "profiles/moe_layer_qwen3_decode_kernel_trace.md"),
    "c3_qwen3_prefill": (952_400_000, "profiles/moe_layer_qwen3_prefill_kernel_trace.md"),
    "c4_dsv3_prefill": (8_030_700_000, "profiles/moe_layer_dsv3_prefill_kernel_trace.md"),
    "c5_w4a8_zipf": (1_662_500_000, "profiles/moe_layer_w4a8_zipf_kernel_trace.md"),
    "c6_dsv3_decode": (6_600_600_000, "profiles/moe_layer_dsv3_decode_kernel_trace.md"),
    "c7_w8a8_zipf": (2_892_100_000, "profiles/moe_layer_w8a8_zipf_kernel_trace.md"),
    "c7_w8a8_zipf_4096": (8_314_400_000, "profiles/moe_layer_w8a8_zipf_4096_kernel_trace.md"),
}


def weight_bytes(cfg, n, k) -> float:
    """bytes of one expert's [n, k] weight and its scales (int8 per channel, or int4 with group scales)"""
    if cfg.w4_group >= 0:
        groups = k // cfg.w4_group if cfg.w4_group else 1
        return n * k / 2 + groups * n * 4
    return n * k + n * 4


def algorithmic_bytes_gmm1(cfg, counts) -> int:
    """gate_up GEMM: weights and channel scales of every expert that has at least one row, the int8
    activations and their scales in, the int8 SwiGLU output and its scales out."""
    active = int((counts > 0).sum())
    R = int(counts.sum())
    w = int(active * weight_bytes(cfg, 2 * cfg.I, cfg.H))
    # the sorted int8 rows and their scales, as the op is defined (the plain W8A8 path reads fewer bytes than that:
    # it keeps one quantised row per token and a row -> token map)
    act_in = R * cfg.H + R * 4
    act_out = R * cfg.I + R * 4
    return w + act_in + act_out


def algorithmic_ops(cfg, R) -> int:
    ops = 2 * R * cfg.H * 2 * cfg.I + 2 * R * cfg.I * cfg.H
    if cfg.shared:
        ops += 2 * cfg.T * cfg.H * 2 * cfg.I + 2 * cfg.T * cfg.I * cfg.H
    return ops


def layer_bytes(cfg, counts) -> int:
    """Whole-layer algorithmic HBM traffic (weights of touched experts + activations in/out of each stage)."""
    active = int((counts > 0).sum())
    R = int(counts.sum())
    T = cfg.T
    w = int(active * (weight_bytes(cfg, 2 * cfg.I, cfg.H) + weight_bytes(cfg, cfg.H, cfg.I)))
    if cfg.shared:
        w += 2 * cfg.I * cfg.H + cfg.H * cfg.I + (2 * cfg.I + cfg.H) * 4
    # tokens and logits in, sorted int8 rows and scales written and read, int8 SwiGLU rows and scales written and
    # read, expert outputs written and read, result out: the accounting of the operator sequence, whatever part
    # of it a fused path avoids
    act = (T * cfg.H * 2 + T * cfg.E * 4 + 2 * R * cfg.H + 2 * R * 4 + 2 * R * cfg.I + 2 * R * 4
           + 2 * R * cfg.H * 2 + T * cfg.H * 2)
    return w + act


def log(msg: str) -> None:
    print(f"bench.py: {msg}", file=sys.stderr, flush=True)


def capture(step, torch):
    """HIP graph of one step, checked against the eager result; None when capture is not possible."""
    want = step().routed_out
    torch.cuda.synchronize()
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            gres = step()
        # several replays with the program's own work between them, each checked against the eager result
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(gres.routed_out, want):
                raise RuntimeError("graph replay differs from the eager result")
        return graph
    except Exception as exc:  # capture not possible: measure eager and say so
        log(f"HIP graph capture failed ({exc}); timing eager launches")
        return None


def time_steps(run, steps, warmup, torch) -> float:
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def single_steps_us(run, n, torch, before=None):
    """n steps, each between its own pair of events; `before` runs (untimed) in front of every step."""
    pev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for s, e in pev:
        if before is not None:
            before()
        s.record()
        run()
        e.record()
    torch.cuda.synchronize()
    us = sorted(s.elapsed_time(e) * 1e3 for s, e in pev)

    def pct(p):
        return round(us[min(len(us) - 1, int(p * len(us)))], 2)

    return {"p10": pct(0.10), "p50": pct(0.50), "p90": pct(0.90), "n": n}


def run_workload(name, args, lib, torch, np):
    from _inputs import CONFIGS, make_layer
    from _layer_utils import build_layer, oracle_layer
    from _parity import layer_parity, staged_run, to_cpu

    from vllm_ascend_amd import kernels as K

    dev = "cuda:0"
    cfg = CONFIGS[name]
    if args.tokens:
        cfg = dataclasses.replace(cfg, T=args.tokens)  # the same layer on a batch of another size
    if args.zipf is not None:
        cfg = dataclasses.replace(cfg, zipf=args.zipf)  # ... with another skew of the expert popularity
    t_start = time.perf_counter()
    dg = make_layer(cfg, seed=0, gen_device=dev)
    layer = build_layer(cfg, dg, dev, shared=cfg.shared, overlap=False)
    x, logits = dg["x"], dg["logits"]
    torch.cuda.synchronize()
    log(f"{name}: layer built in {time.perf_counter() - t_start:.1f} s")

    gate = None
    if args.with_gate:
        from vllm_ascend_amd.fused_moe.gate_linear import AscendGateLinear

        gate = AscendGateLinear(cfg.H, cfg.E, device=dev)
        gate.weight.data.copy_(torch.randn(cfg.E, cfg.H, generator=torch.Generator().manual_seed(1)) * 0.05)

    def step():
        if gate is not None:
            return layer.forward_impl(x, gate(x)[0])
        return layer.forward_impl(x, logits)

    res = step()
    torch.cuda.synchronize()
    counts = res.expert_tokens.cpu().numpy()
    R = int(counts.sum())

    # ---------------- K steps of the whole layer
    mode = args.mode
    graph = capture(step, torch) if mode == "graph" else None
    if graph is None:
        mode = "eager"
    run = graph.replay if graph is not None else step
    ms_per_step = time_steps(run, args.steps, args.warmup, torch)
    tokens_per_s = cfg.T / (ms_per_step * 1e-3)
    n_pct = min(args.steps, 100)
    spread = single_steps_us(run, n_pct, torch)
    out = {
        "tokens_per_s": round(tokens_per_s, 1),
        "ms_per_step": round(ms_per_step, 5),
        "us_per_layer": round(ms_per_step * 1e3, 2),
        "us_per_layer_single_steps": spread,
        "config": {"workload": cfg.name, "tokens": cfg.T, "hidden": cfg.H, "experts": cfg.E, "top_k": cfg.k,
                   "moe_intermediate": cfg.I, "scoring": cfg.scoring, "shared_expert": bool(cfg.shared),
                   "weights": "int4 group %d" % cfg.w4_group if cfg.w4_group >= 0 else "int8 per channel",
                   "launch": mode, "router_gate": gate is not None, "experts_touched": int((counts > 0).sum()),
                   "rows": R},
    }
    lbytes, lops = layer_bytes(cfg, counts), algorithmic_ops(cfg, R)
    out["layer_frac_of_peak"] = {"hbm": round(lbytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                 "mfma": round(lops / (ms_per_step * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                                 "layer_algorithmic_bytes": lbytes, "layer_algorithmic_ops": lops}
    if cfg.T <= 64:
        # decode: the same steps with the caches emptied in front of each (a 1 GiB fill: four times the 256 MB of
        # the Infinity Cache); only the step itself is between the events
        flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        out["us_per_layer_single_steps_after_cache_flush"] = single_steps_us(run, min(n_pct, 50), torch,
                                                                              before=flush.zero_)
        del flush
    if cfg.shared and not args.no_side_stream:
        # the shared expert on the side stream, next to the routed experts
        layer.shared_experts.multistream_overlap = True
        g2 = capture(step, torch) if mode == "graph" else None
        ms2 = time_steps(g2.replay if g2 is not None else step, args.steps, args.warmup, torch)
        out["shared_expert_on_side_stream"] = {"ms_per_step": round(ms2, 5), "launch": "graph" if g2 else "eager"}
        layer.shared_experts.multistream_overlap = False
        del g2

    # ---------------- eager pass with events around the dominant kernel only
    roofline = None
    if not args.no_roofline:
        n = min(args.steps, 100)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for _ in range(min(args.warmup, 10)):
            step()
        torch.cuda.synchronize()
        hooked = {"i": 0, "fired": 0}
        # the launchers of the routed gate_up GEMM (batches past a decode batch read their rows through a
        # row -> token map, decode batches run in pair order)
        hook_names = (["gmm1_swiglu_quant_w4", "gmm1_swiglu_quant_w4_gather"] if cfg.w4_group >= 0
                      else ["gmm1_swiglu_quant", "gmm1_swiglu_quant_gather", "gmm1_swiglu_quant_pairs", "gmm1_swiglu_pairs"])
        origs = {h: getattr(K, h) for h in hook_names}

        def make_timed(orig, routed):
            def timed_gmm1(x_, *a, **kw):
                if not routed(x_):  # the shared expert's dense GEMMs go through the same launcher
                    return orig(x_, *a, **kw)
                s, e = evs[hooked["i"]]
                hooked["fired"] += 1
                # create the underlying hipEvent handles, then let the library record them around the GEMM kernel
                s.record()
                e.record()
                lib.moe355_profile_next_gemm(ctypes.c_void_p(s.cuda_event), ctypes.c_void_p(e.cuda_event))
                return orig(x_, *a, **kw)
            return timed_gmm1

        for h in hook_names:
            setattr(K, h, make_timed(origs[h], (lambda x_: True) if h.endswith(("gather", "pairs"))
                                     else (lambda x_: x_.shape[0] == R)))
        try:
            torch.cuda.synchronize()
            te0 = time.perf_counter()
            for i in range(n):
                hooked["i"] = i
                step()
            torch.cuda.synchronize()
            out["eager_ms_per_step"] = round((time.perf_counter() - te0) * 1e3 / n, 5)
        finally:
            for h in hook_names:
                setattr(K, h, origs[h])
        if hooked["fired"] == n:
            durs = sorted(s.elapsed_time(e) for s, e in evs)  # ms
            avg_ms = sum(durs) / len(durs)
            abytes = algorithmic_bytes_gmm1(cfg, counts)
            ops1 = 2 * R * cfg.H * 2 * cfg.I
            gbs = abytes / (avg_ms * 1e-3) / 1e9
            tops = ops1 / (avg_ms * 1e-3) / 1e12
            # the binding roofline of this kernel: HBM when the weight stream outweighs the MFMA time
            hbm_bound = abytes / (HBM_PEAK_GBS * 1e9) >= ops1 / (INT8_PEAK_TOPS * 1e12)
            if hbm_bound:
                roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(gbs / HBM_PEAK_GBS, 4)}
            else:
                roofline = {"bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                            "frac": round(tops / INT8_PEAK_TOPS, 4)}
            if cfg.w4_group >= 0:
                kernel = "gmm_w4_stream_kernel"
            else:
                kernel = lib.moe355_gmm_kernel_name(1, R, cfg.H, 2 * cfg.I, cfg.E).decode()
            traffic = None if (args.tokens or args.zipf is not None) else TRAFFIC_FROM_PROFILES.get(name)
            roofline.update({
                "traffic": traffic[0] if traffic else None,
                "traffic_source": (traffic[1] + " (rocprofv3 --pmc of an earlier run of this command, not measured "
                                                "in this run)") if traffic else None,
                "kernel": kernel + "<EPI_SWIGLU> (gate_up grouped GEMM + dequant + SwiGLU)",
                "kernel_avg_us": round(avg_ms * 1e3, 2),
                "kernel_p50_us": round(durs[len(durs) // 2] * 1e3, 2),
                "algorithmic_bytes": abytes,
                "algorithmic_ops": ops1,
                "other_frac": {"hbm": round(gbs / HBM_PEAK_GBS, 4), "mfma": round(tops / INT8_PEAK_TOPS, 4)},
            })
    out["roofline"] = roofline

    # ---------------- parity gates against the CPU checker
    dc = None
    gpu_expert_rows = None
    if not args.no_parity or not args.no_cpu_baseline:
        t0 = time.perf_counter()
        dc = to_cpu(dg)
        log(f"{name}: host copies of the tensors in {time.perf_counter() - t0:.1f} s")
    if not args.no_parity and gate is None:
        from oracle import oracle as orc

        t0 = time.perf_counter()
        r = staged_run(K, cfg, dg)
        big = cfg.H * cfg.I >= 4096 * 2048
        parity = layer_parity(orc, cfg, dc, r, n_tokens=4 if big else 16, layer_out=res.routed_out,
                              shared=cfg.shared)
        parity["seconds"] = round(time.perf_counter() - t0, 1)
        out["parity"] = parity
        gpu_expert_rows = r["o"]  # kept for the torch-native CPU leg below
        del r
        log(f"{name}: parity {'FAILED ' + str(parity['failed']) if parity['failed'] else 'ok'} "
            f"in {parity['seconds']} s")

    # ---------------- CPU baseline: the C checker on this host, a bounded sample of the same batch
    if not args.no_cpu_baseline and gate is None:
        from oracle import oracle as orc

        sample_T = cfg.T
        budget_ops = 1.5e11  # per pass: a few seconds of the C port on 16 cores
        if algorithmic_ops(cfg, cfg.T * cfg.k) > budget_ops:
            sample_T = max(cfg.k, int(cfg.T * budget_ops / algorithmic_ops(cfg, cfg.T * cfg.k)))
        d2 = dict(dc)
        d2["x"] = dc["x"][:sample_T].contiguous()
        d2["logits"] = dc["logits"][:sample_T].contiguous()
        scfg = dataclasses.replace(cfg, T=sample_T)
        passes, elapsed, tr = 0, 0.0, None
        while passes < 1 or (elapsed < args.cpu_seconds and passes < 1000):
            tc0 = time.perf_counter()
            tr = oracle_layer(scfg, d2, keep_acc=False, shared=cfg.shared)
            elapsed += time.perf_counter() - tc0
            passes += 1
        from _inputs import bits

        ok = bool(np.array_equal(bits(res.routed_out[:sample_T]), tr.out))
        c_port = {
            "value": round(sample_T * passes / elapsed, 2), "unit": "tokens/s", "cores": orc.num_threads(),
            "kind": "port", "rendering": "the C checker (oracle/moe_oracle.c) with OpenMP",
            "sample": f"the first {sample_T} of {cfg.T} tokens of the same workload, {passes} pass(es) of the whole "
                      f"layer in {elapsed:.2f} s",
            "gpu_output_bit_exact_vs_cpu_on_sample": ok}
        log(f"{name}: CPU baseline (C port) {c_port['value']} tokens/s ({passes} passes, {elapsed:.1f} s)")
        # the torch-native rendering: plain torch CPU operators, the expert MLPs on all rows of the busiest experts
        # (the workload's own rows-per-expert regime) and extrapolated linearly in rows
        from oracle import torch_native

        per_row = algorithmic_ops(dataclasses.replace(cfg, shared=False), 1)
        tn = torch_native.timed_layer(cfg, dc, max_rows=max(64, int(args.cpu_torch_ops / per_row)), max_experts=16,
                                      threads=orc.num_threads())
        rel = None
        if gpu_expert_rows is not None and tn["row_ranges"]:
            a = torch.cat([tn["expert_rows"][lo:hi] for lo, hi in tn["row_ranges"]]).double()
            b = torch.cat([gpu_expert_rows[lo:hi].cpu() for lo, hi in tn["row_ranges"]]).double()
            rel = float((a - b).norm() / b.norm().clamp_min(1e-30))
        out["cpu_baseline"] = {
            "value": round(tn["tokens_per_s"], 2), "unit": "tokens/s", "cores": tn["threads"],
            "kind": "torch-native", "kind_in_the_terms_of_the_contract": "port",
            "dtype_path": "torch.matmul on int32 CPU tensors (int8 activations and weights widened; the weights once, "
                          "outside the timed region), fp32 scales and SwiGLU, "
                          + ("per-group fp32 accumulation over int4 groups" if cfg.w4_group > 0 else
                             "per-channel scales"),
            "sample": f"routing, quantisation, dispatch and combine on all {cfg.T} tokens; expert MLPs on "
                      f"{tn['rows_sampled']} rows of the {tn['experts_sampled']} busiest experts, scaled to the "
                      f"{tn['rows']} rows of the batch" + (f"; shared expert on {min(cfg.T, 256)} rows, scaled"
                                                          if cfg.shared else ""),
            "seconds_by_part": tn["seconds"],
            "rel_err_of_its_expert_rows_vs_gpu": rel,
            "c_port": c_port}
        log(f"{name}: CPU baseline (torch-native) {out['cpu_baseline']['value']} tokens/s, parts {tn['seconds']}, "
            f"expert rows vs GPU rel {rel}")
        del tn
    else:
        out["cpu_baseline"] = None
    del layer, dg, dc, graph, gpu_expert_rows
    torch.cuda.empty_cache()
    log(f"{name}: {out['us_per_layer']} us per layer, done in {time.perf_counter() - t_start:.1f} s")
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None,
                    help="one workload or a comma-separated list; default: all of " + ", ".join(WORKLOADS))
    ap.add_argument("--tokens", type=int, default=0,
                    help="run the named workload(s) on a batch of this many tokens instead of their own")
    ap.add_argument("--zipf", type=float, default=None,
                    help="expert popularity ~ rank^-S for the named workload(s) instead of their own (0: uniform)")
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph")
    ap.add_argument("--with-gate", action="store_true",
                    help="start the step one operator earlier: the fp32 router gate GEMM (hidden states -> logits, "
                         "random fp32 weight) runs inside every step; the headline metric starts at the logits")
    ap.add_argument("--cpu-seconds", type=float, default=6.0, help="CPU-baseline time per workload")
    ap.add_argument("--cpu-torch-ops", type=float, default=1.2e11,
                    help="integer operations the torch-native CPU leg spends on its sample of expert rows")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--no-side-stream", action="store_true",
                    help="skip the extra timing with the shared expert on its side stream (kernel profiles: keeps "
                         "overlapped launches out of the per-kernel durations)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the whole MoE layer on ONE GPU (no expert parallelism, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from vllm_ascend_amd import _lib

    lib = _lib.load()  # raises if the HIP library is missing: there is no fallback
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    names = args.workload.split(",") if args.workload else list(WORKLOADS)
    head_name = HEADLINE if HEADLINE in names else names[0]
    results = {}
    for name in names:
        results[name] = run_workload(name, args, lib, torch, np)
    head = results[head_name]
    all_ok = all(not w.get("parity", {}).get("failed") for w in results.values())
    out = {
        "metric": "W8A8 MoE-layer tokens/sec at 1 GPU",
        "value": head["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "us_per_layer": head["us_per_layer"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic (seed 0, drawn on the GPU: bf16 N(0,1) activations, N(0,1) router logits, int8 U[-127,127] "
                "weights, fp32 U(0.001,0.01) channel scales; int4 U[-8,7] weights with group-256 scales and "
                "Zipf(1.1) routing for the W4A8 workload)",
        "config": head["config"],
        "layer_frac_of_peak": head["layer_frac_of_peak"],
        "roofline": head["roofline"],
        "cpu_baseline": head["cpu_baseline"],
        "parity": head.get("parity"),
        "parity_gates_hold_on_every_workload": all_ok,
        "workloads": results,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
