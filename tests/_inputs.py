"""Seeded synthetic inputs for the configured MoE-layer shapes (generated on the CPU so
the CPU checker and the GPU kernels see identical bits)."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class LayerCfg:
    name: str
    T: int
    H: int
    E: int
    k: int
    I: int
    scoring: str = "softmax"  # or "sigmoid"
    n_group: int = 1
    topk_group: int = 1
    renorm: int = 1
    routed_scaling_factor: float = 1.0
    bias: bool = False
    shared: bool = False
    w4_group: int = -1  # >= 0: W4A8 (int4 weights); 0 = per-channel scales, g > 0 = groups of g along K
    zipf: float = 0.0  # > 0: router logits biased so that expert popularity follows Zipf(s)


CONFIGS = {
    # the benchmark configurations (full sizes) and reduced variants for CPU-checkable parity
    "c1_tiny": LayerCfg("c1_tiny", 64, 1024, 8, 2, 1408),
    "c2_qwen3_decode": LayerCfg("c2_qwen3_decode", 64, 2048, 128, 8, 768),
    "c3_qwen3_prefill": LayerCfg("c3_qwen3_prefill", 8192, 2048, 128, 8, 768),
    "c4_dsv3_prefill": LayerCfg("c4_dsv3_prefill", 4096, 7168, 256, 8, 2048, scoring="sigmoid", n_group=8,
                                topk_group=4, routed_scaling_factor=2.5, bias=True, shared=True),
    "c5_w4a8_zipf": LayerCfg("c5_w4a8_zipf", 512, 7168, 256, 8, 2048, scoring="sigmoid", n_group=8, topk_group=4,
                             routed_scaling_factor=2.5, bias=True, w4_group=256, zipf=1.1),
    # the north star's decode target: the DeepSeek-V3 shape with a 64-token batch
    "c6_dsv3_decode": LayerCfg("c6_dsv3_decode", 64, 7168, 256, 8, 2048, scoring="sigmoid", n_group=8, topk_group=4,
                               routed_scaling_factor=2.5, bias=True, shared=True),
    # W8A8 under skewed routing: the DeepSeek-V3 shape with Zipf(1.1) expert popularity, a small and a prefill batch
    "c7_w8a8_zipf": LayerCfg("c7_w8a8_zipf", 512, 7168, 256, 8, 2048, scoring="sigmoid", n_group=8, topk_group=4,
                             routed_scaling_factor=2.5, bias=True, zipf=1.1),
    "c7_w8a8_zipf_4096": LayerCfg("c7_w8a8_zipf_4096", 4096, 7168, 256, 8, 2048, scoring="sigmoid", n_group=8,
                                  topk_group=4, routed_scaling_factor=2.5, bias=True, zipf=1.1),
    "c7_small": LayerCfg("c7_small", 512, 512, 64, 4, 256, scoring="sigmoid", n_group=8, topk_group=4,
                         routed_scaling_factor=2.5, bias=True, zipf=1.1),
    "c5_small": LayerCfg("c5_small", 80, 512, 32, 4, 256, scoring="sigmoid", n_group=4, topk_group=2,
                         routed_scaling_factor=2.5, bias=True, w4_group=128, zipf=1.1),
    "c5_small_perchannel": LayerCfg("c5_small_perchannel", 40, 256, 16, 2, 128, w4_group=0),
    # reduced shapes with the same structure
    "c2_small": LayerCfg("c2_small", 48, 512, 32, 4, 256),
    "c3_small": LayerCfg("c3_small", 640, 512, 16, 4, 256),
    "c4_small": LayerCfg("c4_small", 96, 512, 64, 8, 192, scoring="sigmoid", n_group=8, topk_group=4,
                         routed_scaling_factor=2.5, bias=True, shared=True),
}


def make_layer(cfg: LayerCfg, seed: int = 0, device: str = "cpu", gen_device: str = "cpu"):
    """Returns a dict of torch tensors: x bf16, logits fp32, w13 int8 [E,2I,H], s13 fp32 [E,2I],
    w2 int8 [E,H,I], s2 fp32 [E,H], optional bias fp32 [E] and shared-expert weights.
    gen_device: where the seeded generator runs.  "cpu" (the default; every committed fixture comes from it)
    returns CPU tensors, moved to `device` when that is given.  A GPU generator draws a different, equally
    deterministic stream and returns the tensors where they were drawn (the 11 GB of the DeepSeek-V3-shaped
    configurations take seconds instead of minutes that way; the CPU checker then works on copies)."""
    gd = gen_device
    g = torch.Generator(device=gd).manual_seed(seed)
    d = {}
    d["x"] = torch.randn(cfg.T, cfg.H, generator=g, dtype=torch.float32, device=gd).to(torch.bfloat16)
    d["logits"] = torch.randn(cfg.T, cfg.E, generator=g, dtype=torch.float32, device=gd)
    if cfg.zipf > 0:
        # popularity ~ rank^-s over a fixed random ordering of the experts, added as log-prior to the logits
        order = torch.randperm(cfg.E, generator=g, device=gd)
        pmf = torch.arange(1, cfg.E + 1, dtype=torch.float64, device=gd) ** (-cfg.zipf)
        prior = torch.empty(cfg.E, dtype=torch.float64, device=gd)
        prior[order] = torch.log(pmf / pmf.sum())
        d["logits"] = (d["logits"].double() + prior).float()
    if cfg.w4_group >= 0:
        # int4 values, one per int8 (checkpoint form [E, N, K]); scales [E, N, K/g] (g = K when per channel)
        d["w13"] = torch.randint(-8, 8, (cfg.E, 2 * cfg.I, cfg.H), generator=g, dtype=torch.int8, device=gd)
        d["w2"] = torch.randint(-8, 8, (cfg.E, cfg.H, cfg.I), generator=g, dtype=torch.int8, device=gd)
        g13 = cfg.H // cfg.w4_group if cfg.w4_group else 1
        g2 = cfg.I // cfg.w4_group if cfg.w4_group else 1
        d["s13"] = torch.rand(cfg.E, 2 * cfg.I, g13, generator=g, dtype=torch.float32, device=gd) * 0.09 + 0.01
        d["s2"] = torch.rand(cfg.E, cfg.H, g2, generator=g, dtype=torch.float32, device=gd) * 0.09 + 0.01
    else:
        d["w13"] = torch.randint(-127, 128, (cfg.E, 2 * cfg.I, cfg.H), generator=g, dtype=torch.int8, device=gd)
        d["w2"] = torch.randint(-127, 128, (cfg.E, cfg.H, cfg.I), generator=g, dtype=torch.int8, device=gd)
        d["s13"] = torch.rand(cfg.E, 2 * cfg.I, generator=g, dtype=torch.float32, device=gd) * 0.009 + 0.001
        d["s2"] = torch.rand(cfg.E, cfg.H, generator=g, dtype=torch.float32, device=gd) * 0.009 + 0.001
    if cfg.bias:
        d["bias"] = torch.randn(cfg.E, generator=g, dtype=torch.float32, device=gd) * 0.01
    if cfg.shared:
        d["sw13"] = torch.randint(-127, 128, (1, 2 * cfg.I, cfg.H), generator=g, dtype=torch.int8, device=gd)
        d["sw2"] = torch.randint(-127, 128, (1, cfg.H, cfg.I), generator=g, dtype=torch.int8, device=gd)
        d["ss13"] = torch.rand(1, 2 * cfg.I, generator=g, dtype=torch.float32, device=gd) * 0.009 + 0.001
        d["ss2"] = torch.rand(1, cfg.H, generator=g, dtype=torch.float32, device=gd) * 0.009 + 0.001
    if gd == "cpu" and device != "cpu":
        d = {k: v.to(device) for k, v in d.items()}
    return d


def gating_kwargs(cfg: LayerCfg) -> dict:
    return dict(k=cfg.k, k_group=cfg.topk_group, group_count=cfg.n_group, group_select_mode=1, renorm=cfg.renorm,
                norm_type=0 if cfg.scoring == "softmax" else 1, routed_scaling_factor=cfg.routed_scaling_factor,
                eps=1e-20)


def bits(t: torch.Tensor) -> np.ndarray:
    """torch tensor -> numpy, 16-bit floats as raw uint16."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()
