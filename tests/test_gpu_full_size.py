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


def _make(cfg, seed=0):
    """The configuration's tensors, drawn on the GPU (seconds for the 11 GB of the DeepSeek-V3 shapes), and CPU
    copies of them for the checker."""
    from _parity import to_cpu

    dg = make_layer(cfg, seed=seed, gen_device=DEV)
    torch.cuda.synchronize()
    return dg, to_cpu(dg)


@pytest.mark.parametrize("name", ["c3_qwen3_prefill", "c4_dsv3_prefill", "c5_w4a8_zipf", "c6_dsv3_decode",
                                  "c3_qwen3_prefill@32768", "c7_w8a8_zipf", "c7_w8a8_zipf_4096"])
def test_full_size_properties_and_sampled_rows(K, orc, name):
    """The benchmark configurations at their full sizes (all 256 experts of the DeepSeek-V3 shapes, 4096 / 512 / 64
    tokens), stage by stage; "name@T": the same shape on a batch of T tokens (four times the benchmark's prefill
    batch: 262,144 sorted rows)."""
    import dataclasses

    from _parity import layer_parity, staged_run

    base, _, tokens = name.partition("@")
    cfg = CONFIGS[base] if not tokens else dataclasses.replace(CONFIGS[base], T=int(tokens))
    print(f"full size {name}: T={cfg.T} E={cfg.E} H={cfg.H} I={cfg.I}", flush=True)
    dg, dc = _make(cfg)
    print("  tensors ready", flush=True)
    r = staged_run(K, cfg, dg)
    print("  GPU pass done", flush=True)
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

    # ---- every gate of the layer against the checker: routing, permutation and the first quantisation on the
    # whole batch; int32 accumulators, int8 SwiGLU output, expert output and the combine on sampled rows / tokens
    p = layer_parity(orc, cfg, dc, r, n_tokens=12)
    print(f"  parity {p}", flush=True)
    assert not p["failed"], p
    assert p["rel_err_vs_fp32_dequant_reference"] <= 5e-2
    if "rel_err_vs_quantized_fp64_reference" in p:
        assert p["rel_err_vs_quantized_fp64_reference"] <= 1e-2

    # ---- the combine is linear in the routing weights
    out2 = K.token_unpermute(r["o"], r["dst"], (r["w"].float() * 2).to(torch.bfloat16))
    assert torch.equal(out2.float(), r["out"].float() * 2)

    # ---- a second run gives the same bits
    r2 = staged_run(K, cfg, dg, want_acc=False)
    for key in ("dst", "xs", "q1", "s1", "o", "out"):
        assert torch.equal(r[key], r2[key]), key


@pytest.mark.parametrize("name", ["c4_dsv3_prefill", "c6_dsv3_decode"])
def test_full_size_layer_with_shared_expert(K, orc, name):
    """The DeepSeek-V3-shaped layer at full size through the plugin interface, with its shared expert on the main
    stream and on the side stream: histogram on the whole batch, final output of sampled tokens recomputed by the
    checker (routed rows, shared expert and the fused add)."""
    from _layer_utils import build_layer
    from _parity import layer_parity, staged_run

    cfg = CONFIGS[name]
    print(f"full size layer {name} with shared expert", flush=True)
    dg, dc = _make(cfg)
    r = staged_run(K, cfg, dg, want_acc=False)
    layer = build_layer(cfg, dg, DEV, shared=True, overlap=False)
    print("  layer built", flush=True)
    outs = {}
    for overlap in (False, True):
        layer.shared_experts.multistream_overlap = overlap
        for _ in range(2):
            res = layer.forward_impl(dg["x"], dg["logits"])
        torch.cuda.synchronize()
        outs[overlap] = res.routed_out
        assert torch.equal(res.expert_tokens, r["cnt"])
        p = layer_parity(orc, cfg, dc, r, n_tokens=6, layer_out=res.routed_out, shared=True, full_dispatch=False)
        print(f"  overlap={overlap} parity {p}", flush=True)
        assert not p["failed"], p
        assert p["rel_err_vs_fp32_dequant_reference"] <= 5e-2
    assert torch.equal(outs[False], outs[True])
