"""The torch-native CPU rendering that the benchmark times as its CPU baseline, against the CPU checker.

It is built from plain torch operators after the reference's golden functions (oracle/torch_native.py cites them),
so it is not bit-identical to the checker's fixed operation sequence; routing and dispatch are integer / ordering
work and must agree exactly, the 16-bit expert rows to a few units of their last place."""
import numpy as np
import pytest

from _inputs import CONFIGS, make_layer
from _layer_utils import oracle_layer
from oracle import oracle as orc
from oracle import torch_native as tn


@pytest.mark.parametrize("name", ["c1_tiny", "c2_small", "c4_small", "c5_small", "c5_small_perchannel"])
def test_torch_native_layer_agrees_with_the_checker(name):
    cfg = CONFIGS[name]
    d = make_layer(cfg, seed=0)
    r = tn.timed_layer(cfg, d, max_rows=1 << 30, max_experts=1 << 30)
    tr = oracle_layer(cfg, d, keep_acc=False, shared=False)
    assert np.array_equal(r["ids"].numpy(), tr.topk_ids)
    assert np.array_equal(r["dst"].numpy().astype(np.int32), tr.expanded_row_idx)
    assert r["rows_sampled"] == r["rows"] == cfg.T * cfg.k
    got = r["expert_rows"].float().numpy().astype(np.float64)
    want = orc.half_to_f32(tr.o).astype(np.float64)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
    assert r["tokens_per_s"] > 0 and set(r["seconds"]) == {"front", "experts_sample", "experts", "shared", "combine"}


def test_sample_takes_the_busiest_experts_and_scales_by_rows():
    cfg = CONFIGS["c3_small"]
    d = make_layer(cfg, seed=0)
    r = tn.timed_layer(cfg, d, max_rows=400, max_experts=2)
    assert r["experts_sampled"] <= 2 and 0 < r["rows_sampled"] <= max(400, r["rows_sampled"])
    assert abs(r["seconds"]["experts"] - r["seconds"]["experts_sample"] * r["rows"] / r["rows_sampled"]) < 1e-3
