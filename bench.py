#!/usr/bin/env python3
"""Benchmark of the W8A8-dynamic fused-MoE layer on one MI355X.

One step = one pass of the whole routed-experts layer (router logits -> final bf16)
over one batch of synthetic tokens, through the plugin interface
(router.select_experts -> quant_method.apply).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--mode graph|eager]

The default workload is the Qwen3-30B-A3B-shaped decode batch (64 tokens), the
configuration the headline metric is quoted on.  Inputs are resident in HBM before the
timed region.  `roofline` describes the dominant kernel (the gate_up grouped GEMM), timed
with HIP events that bracket exactly that kernel in every step of a second, eager pass.
`cpu_baseline` is the CPU checker (a C port, OpenMP) timed on this host on the same batch.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA

# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE,
# scaled by a copy kernel of known size); filled in from the summaries under profiles/.
MEASURED_TRAFFIC_BYTES = {
    # profiles/moe_layer_qwen3_decode_hbm_traffic.md: 194220.8 KiB x 2.00 fetched + 1536.0 KiB x 1.00 written
    "c2_qwen3_decode": 399_300_000,
    # profiles/moe_layer_qwen3_prefill_kernel_trace.md: 384107.5 KiB x 2.00 + 196608.0 KiB
    "c3_qwen3_prefill": 988_000_000,
    # profiles/moe_layer_dsv3_prefill_kernel_trace.md: 3842493.7 KiB x 2.00 + 262144.0 KiB
    "c4_dsv3_prefill": 8_137_900_000,
    # profiles/moe_layer_w4a8_zipf_kernel_trace.md: 900832.3 KiB x 2.00 + 32921.8 KiB
    "c5_w4a8_zipf": 1_878_600_000,
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
    act = (T * cfg.H * 2 + T * cfg.E * 4 + 2 * R * cfg.H + 2 * R * 4 + 2 * R * cfg.I + 2 * R * 4
           + 2 * R * cfg.H * 2 + T * cfg.H * 2)
    return w + act


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2_qwen3_decode")
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph")
    ap.add_argument("--with-gate", action="store_true",
                    help="start the step one operator earlier: the fp32 router gate GEMM (hidden states -> logits, "
                         "random fp32 weight) runs inside every step; the headline metric starts at the logits")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the whole MoE layer on ONE GPU (no expert parallelism, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from _inputs import CONFIGS, bits, make_layer
    from _layer_utils import build_layer, oracle_layer

    from vllm_ascend_amd import _lib

    lib = _lib.load()  # raises if the HIP library is missing: there is no fallback
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = "cuda:0"
    cfg = CONFIGS[args.workload]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, dev, shared=cfg.shared)
    x, logits = d["x"].to(dev), d["logits"].to(dev)
    del d["w13"], d["w2"]  # the host copies are only needed again for the CPU baseline

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

    # ---------------- headline: K steps of the whole layer
    graph = None
    mode = args.mode
    if mode == "graph":
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
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(gres.routed_out, res.routed_out):
                raise RuntimeError("graph replay differs from the eager result")
        except Exception as exc:  # capture not possible: measure eager and say so
            print(f"bench.py: HIP graph capture failed ({exc}); timing eager launches", file=sys.stderr)
            graph = None
            mode = "eager"
    run = graph.replay if graph is not None else step
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    tokens_per_s = cfg.T / (ms_per_step * 1e-3)

    # ---------------- spread of single steps: each of up to 100 steps between its own pair of events
    n_pct = min(args.steps, 100)
    pev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_pct)]
    for s, e in pev:
        s.record()
        run()
        e.record()
    torch.cuda.synchronize()
    step_us = sorted(s.elapsed_time(e) * 1e3 for s, e in pev)

    def pct(p):
        return round(step_us[min(len(step_us) - 1, int(p * len(step_us)))], 2)

    # ---------------- eager pass with events around the dominant kernel only
    roofline = None
    eager_ms = None
    if not args.no_roofline:
        n = min(args.steps, 100)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for _ in range(min(args.warmup, 10)):
            step()
        torch.cuda.synchronize()
        hooked = {"i": 0}
        from vllm_ascend_amd import kernels as K

        hook_name = "gmm1_swiglu_quant_w4" if cfg.w4_group >= 0 else "gmm1_swiglu_quant"
        orig = getattr(K, hook_name)

        def timed_gmm1(*a, **kw):
            s, e = evs[hooked["i"]]
            hooked["fired"] = hooked.get("fired", 0) + 1
            # create the underlying hipEvent handles, then let the library record them around the GEMM kernel
            s.record()
            e.record()
            lib.moe355_profile_next_gemm(ctypes.c_void_p(s.cuda_event), ctypes.c_void_p(e.cuda_event))
            return orig(*a, **kw)

        setattr(K, hook_name, timed_gmm1)
        try:
            torch.cuda.synchronize()
            te0 = time.perf_counter()
            for i in range(n):
                hooked["i"] = i
                step()
            torch.cuda.synchronize()
            te1 = time.perf_counter()
        finally:
            setattr(K, hook_name, orig)
        eager_ms = (te1 - te0) * 1e3 / n
        fired = hooked.get("fired", 0) > 0
        durs = sorted(s.elapsed_time(e) for s, e in evs) if fired else [1.0]  # ms
        avg_ms = sum(durs) / len(durs)
        abytes = algorithmic_bytes_gmm1(cfg, counts)
        ops1 = 2 * R * cfg.H * 2 * cfg.I
        achieved_gbs = abytes / (avg_ms * 1e-3) / 1e9
        achieved_tops = ops1 / (avg_ms * 1e-3) / 1e12
        # the binding roofline of this kernel: HBM when the weight stream outweighs the MFMA time
        hbm_bound = abytes / (HBM_PEAK_GBS * 1e9) >= ops1 / (INT8_PEAK_TOPS * 1e12)
        if not fired:
            roofline = None
        elif hbm_bound:
            roofline = {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(achieved_gbs / HBM_PEAK_GBS, 4)}
        else:
            roofline = {"bound": "mfma", "achieved": round(achieved_tops, 1), "peak": INT8_PEAK_TOPS,
                        "unit": "TOP/s", "frac": round(achieved_tops / INT8_PEAK_TOPS, 4)}
        if roofline is not None:
            roofline.update({
                "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                # the same rule as the library's choice of GEMM kernel (rows per expert and K)
                "kernel": ("gmm_w4_stream_kernel<EPI_SWIGLU>" if cfg.w4_group >= 0 else
                           "gmm_stream_kernel<EPI_SWIGLU>" if (R // cfg.E < 48 or cfg.H % 64 != 0) else
                           "gmm_wide_kernel<EPI_SWIGLU>" if ((R // cfg.E <= 256 and cfg.H >= 4096) or
                                                             (96 <= R // cfg.E <= 192 and cfg.H >= 1024)) else
                           "gmm_tiled_kernel<EPI_SWIGLU>") + " (gate_up grouped GEMM + dequant + SwiGLU)",
                "kernel_avg_us": round(avg_ms * 1e3, 2),
                "kernel_p50_us": round(durs[len(durs) // 2] * 1e3, 2),
                "algorithmic_bytes": abytes,
                "algorithmic_ops": ops1,
                "other_frac": {"hbm": round(achieved_gbs / HBM_PEAK_GBS, 4),
                               "mfma": round(achieved_tops / INT8_PEAK_TOPS, 4)},
            })

    # ---------------- CPU baseline: the C checker on this host, same batch
    cpu = None
    if not args.no_cpu_baseline and gate is None:  # the CPU baseline covers the path from the logits on
        from oracle import oracle as orc

        d2 = make_layer(cfg, seed=0)
        sample_T = cfg.T
        # bound the CPU work to roughly 10-30 s: shrink the batch for the prefill shapes
        budget_ops = 4.0e11
        if algorithmic_ops(cfg, cfg.T * cfg.k) > budget_ops:
            sample_T = max(cfg.k, int(cfg.T * budget_ops / algorithmic_ops(cfg, cfg.T * cfg.k)))
            d2["x"] = d2["x"][:sample_T].contiguous()
            d2["logits"] = d2["logits"][:sample_T].contiguous()
        import dataclasses

        scfg = dataclasses.replace(cfg, T=sample_T)
        passes, elapsed, tr = 0, 0.0, None
        while passes < 3 or (elapsed < 10.0 and passes < 1000):
            tc0 = time.perf_counter()
            tr = oracle_layer(scfg, d2, keep_acc=False, shared=cfg.shared)
            elapsed += time.perf_counter() - tc0
            passes += 1
        if sample_T == cfg.T:
            ok = bool(np.array_equal(bits(res.routed_out), tr.out))
        else:
            ok = None
        cpu = {"value": round(sample_T * passes / elapsed, 2), "unit": "tokens/s", "cores": orc.num_threads(),
               "kind": "port",
               "sample": f"{sample_T} of {cfg.T} tokens of the same workload, {passes} passes of the whole layer "
                         f"in {elapsed:.2f} s",
               "gpu_output_bit_exact_vs_cpu": ok}

    lbytes = layer_bytes(cfg, counts)
    lops = algorithmic_ops(cfg, R)
    out = {
        "metric": "W8A8 MoE-layer tokens/sec at 1 GPU",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "us_per_layer": round(ms_per_step * 1e3, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic (seed 0: bf16 N(0,1) activations, N(0,1) router logits, int8 U[-127,127] weights, "
                "fp32 U(0.001,0.01) channel scales)",
        "config": {"workload": cfg.name, "tokens": cfg.T, "hidden": cfg.H, "experts": cfg.E, "top_k": cfg.k,
                   "moe_intermediate": cfg.I, "scoring": cfg.scoring, "launch": mode, "router_gate": gate is not None,
                   "experts_touched": int((counts > 0).sum()), "rows": R},
        "layer_frac_of_peak": {"hbm": round(lbytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                               "mfma": round(lops / (ms_per_step * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                               "layer_algorithmic_bytes": lbytes, "layer_algorithmic_ops": lops},
        "us_per_layer_single_steps": {"p10": pct(0.10), "p50": pct(0.50), "p90": pct(0.90), "n": n_pct},
        "eager_ms_per_step": None if eager_ms is None else round(eager_ms, 5),
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
