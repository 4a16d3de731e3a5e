#!/usr/bin/env python3
"""Writes tests/golden/c1_tiny_layer.npz: the tiny configured MoE layer (64 tokens, hidden 1024, 8 experts,
top-2 softmax with renorm, intermediate 1408, seed 0) evaluated by the CPU checker in this repository.
Small tensors are stored whole; the large ones as SHA-256 digests plus a strided sample.
Run from the repository root:  python tests/golden/make_golden.py
(The reference cannot be imported here -- vllm and torch_npu are absent -- so these vectors come from
the checker, whose stages are pinned separately against the reference's own golden functions.)"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

BIG = ("xs", "acc1", "q1", "acc2", "o", "out")
SMALL = ("topk_ids", "topk_weights", "expanded_row_idx", "expert_tokens", "sx", "s1")


def digest(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def sample(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a.reshape(-1)[::997])


def main():
    from _inputs import CONFIGS, make_layer
    from _layer_utils import oracle_layer

    cfg = CONFIGS["c1_tiny"]
    tr = oracle_layer(cfg, make_layer(cfg, seed=0))
    out = {name: getattr(tr, name) for name in SMALL}
    for name in BIG:
        a = getattr(tr, name)
        out[name + "_sha256"] = np.frombuffer(bytes.fromhex(digest(a)), dtype=np.uint8)
        out[name + "_sample"] = sample(a)
        out[name + "_shape"] = np.array(a.shape)
    path = os.path.join(HERE, "c1_tiny_layer.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
