"""The whole layer against the checker on seeded random configurations: shapes, fan-outs, expert counts, group
structures, scoring functions, biases, scaling factors, skewed routing, shared expert and the W4A8 scheme drawn at
random, so that the borders between the kernel families (pair order / sorted decode batches, streaming / tiled /
split grouped GEMMs, fused / separate re-quantisation) are crossed in combinations nobody wrote down by hand.
Output and per-expert counts bit for bit."""
import numpy as np
import pytest
import torch

from _inputs import LayerCfg, bits, make_layer
from _layer_utils import build_layer, oracle_layer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _draw(seed: int) -> LayerCfg:
    r = np.random.default_rng(1000 + seed)
    w4 = seed % 8 == 7
    H = int(r.choice([256, 512, 768, 1024] if w4 else [128, 192, 256, 320, 512, 1024, 4096]))
    I = int(r.choice([128, 256] if w4 else [64, 128, 192, 256, 384]))
    E = int(r.choice([4, 8, 16, 24, 32, 64, 96, 128]))
    k = int(r.integers(1, min(8, E) + 1))
    n_group = topk_group = 1
    if r.random() < 0.4:
        cands = [g for g in (2, 4, 8) if E % g == 0 and E // g >= 2]
        if cands:
            n_group = int(r.choice(cands))
            topk_group = int(r.integers(1, n_group + 1))
            if k > topk_group * (E // n_group):
                k = topk_group * (E // n_group)
            # the router's guard in front of the fused gating op (it measures the hidden size, as the reference's does)
            if k > H / (n_group * topk_group) or H // n_group <= 2:
                n_group = topk_group = 1
    # mostly decode-sized batches, some with enough rows for the tiled kernels; bounded checker time
    T = int(r.choice([1, 3, 17, 64, 130, 257, 700, 1500, 2600]))
    while T * k * H * I > 1.2e10 and T > 1:
        T //= 2
    scoring = "sigmoid" if r.random() < 0.5 else "softmax"
    cfg = LayerCfg(f"rnd{seed}", T, H, E, k, I, scoring=scoring, n_group=n_group, topk_group=topk_group,
                   renorm=int(r.random() < 0.7), routed_scaling_factor=float(r.choice([1.0, 2.5])),
                   bias=bool(r.random() < 0.5), shared=bool(not w4 and r.random() < 0.3),
                   w4_group=(int(r.choice([0, 128])) if w4 else -1), zipf=float(r.choice([0.0, 0.0, 1.1])))
    return cfg


# front: the layer's own choice (pair order where it applies, else the fused front end), the sorted fused form, and
# the reference's operator sequence one operator at a time
CASES = [(s, "default") for s in range(64)] + [(s, f) for s in range(0, 64, 3) for f in ("sorted", "op-by-op")]


@pytest.mark.parametrize("seed,front", CASES)
def test_random_layer_matches_the_checker(seed, front):
    cfg = _draw(seed)
    print(f"random layer {cfg} front={front}", flush=True)
    d = make_layer(cfg, seed=seed)
    layer = build_layer(cfg, d, DEV, shared=cfg.shared)
    layer.use_fused_small_batch = front != "op-by-op"
    layer.use_pair_order = front == "default"
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d, shared=cfg.shared)
    assert np.array_equal(res.expert_tokens.cpu().numpy(), tr.expert_tokens)
    if cfg.shared:
        assert np.array_equal(bits(res.shared_out), tr.extra["shared_out"])
    assert np.array_equal(bits(res.routed_out), tr.out)
