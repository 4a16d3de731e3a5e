"""The tiny configured layer against the committed fixture tests/golden/c1_tiny_layer.npz:
the CPU checker must reproduce it (no GPU), and so must the HIP path (GPU)."""
import os

import numpy as np
import pytest
import torch

from _inputs import CONFIGS, bits, make_layer
from _layer_utils import build_layer, oracle_layer
from golden.make_golden import BIG, SMALL, digest, sample

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_tiny_layer.npz"))


def check(name, arr):
    arr = np.ascontiguousarray(arr)
    if name in SMALL:
        assert np.array_equal(arr, FIX[name]), name
    else:
        assert tuple(FIX[name + "_shape"]) == arr.shape, name
        assert np.array_equal(sample(arr), FIX[name + "_sample"]), name
        assert digest(arr) == bytes(FIX[name + "_sha256"]).hex(), name


def test_checker_reproduces_the_fixture():
    cfg = CONFIGS["c1_tiny"]
    tr = oracle_layer(cfg, make_layer(cfg, seed=0))
    for name in SMALL + BIG:
        check(name, getattr(tr, name))


@pytest.mark.gpu
def test_hip_path_reproduces_the_fixture():
    from vllm_ascend_amd import kernels as K

    dev = "cuda:0"
    cfg = CONFIGS["c1_tiny"]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, dev)
    x, logits = d["x"].to(dev), d["logits"].to(dev)
    w, ids = layer.router.select_experts(x, logits)
    check("topk_ids", ids.cpu().numpy())
    check("topk_weights", bits(w))
    xs, dst, cnt, sx = K.init_routing(x, ids, cfg.E, 1, 1)
    check("expanded_row_idx", dst.cpu().numpy())
    check("expert_tokens", cnt.cpu().numpy())
    check("xs", xs.cpu().numpy())
    check("sx", sx.cpu().numpy())
    check("acc1", K.gmm_i32(xs, layer.w13_weight.data, cnt, 1, 2 * cfg.I, cfg.H).cpu().numpy())
    q1, s1 = K.gmm1_swiglu_quant(xs, layer.w13_weight.data, layer.w13_weight_scale_fp32, sx, cnt, 1, 2 * cfg.I, cfg.H)
    check("q1", q1.cpu().numpy())
    check("s1", s1.cpu().numpy())
    check("acc2", K.gmm_i32(q1, layer.w2_weight.data, cnt, 1, cfg.H, cfg.I).cpu().numpy())
    check("o", bits(K.gmm2_dequant(q1, layer.w2_weight.data, layer.w2_weight_scale_fp32, s1, cnt, 1, cfg.H, cfg.I)))
    check("out", bits(layer.forward_impl(x, logits).routed_out))
