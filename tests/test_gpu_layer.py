"""GPU parity of the whole routed-experts layer through the plugin interface
(router -> quant_method.apply -> FusedExpertsResult) against the CPU checker."""
import numpy as np
import pytest
import torch

from _inputs import CONFIGS, bits, make_layer
from _layer_utils import build_layer, oracle_layer, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# fused: batches of at most 1024 pairs run in pair order (nothing sorted: gating + quantisation, the GEMMs collect
# their pairs themselves); "sorted": the form before it, gating + dispatch in one kernel and GEMMs on the sorted
# order; False: op by op.  c3_small (2560 pairs) is beyond the first two either way
@pytest.mark.parametrize("fused", [True, "sorted", False])
@pytest.mark.parametrize("name", ["c1_tiny", "c2_small", "c3_small", "c4_small", "c7_small", "c2_qwen3_decode"])
def test_layer_bit_exact(name, fused):
    from oracle import oracle as orc

    cfg = CONFIGS[name]
    print(f"layer {name} fused={fused}", flush=True)
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV)
    layer.use_fused_small_batch = bool(fused)
    layer.use_pair_order = fused is True
    takes_fused = layer.quant_method.supports_small_batch(layer, d["x"].to(DEV), d["logits"].to(DEV), layer.router)
    assert takes_fused  # every plain W8A8 call has a router-fused form (one launch up to 1024 pairs)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d)
    # routing
    w, ids = layer.router.select_experts(x, logits)
    assert np.array_equal(ids.cpu().numpy(), tr.topk_ids)
    assert np.array_equal(bits(w), tr.topk_weights)
    # histogram
    assert res.group_list_type == 1
    assert np.array_equal(res.expert_tokens.cpu().numpy(), tr.expert_tokens)
    # final output, bit for bit
    assert np.array_equal(bits(res.routed_out), tr.out)
    got = orc.bf16_to_f32(bits(res.routed_out))
    # tolerance gate 1 (rel <= 1e-2): the same quantised pipeline with the floating-point tail in float64
    ref_q = orc.quantized_fp64_reference(tr, d["s2"].numpy())
    err_q = rel_err(got, ref_q)
    # tolerance gate 2: dense fp32/fp64 layer with dequantised weights and NO activation quantisation.
    # 8-bit dynamic activation quantisation alone puts about 2.5 % of noise on this synthetic data
    # (Gaussian activations, heavy-tailed SwiGLU output), so the bound here is 5e-2; the value is reported.
    ref = orc.fp32_dequant_reference(bits(d["x"]), tr.topk_weights, tr.topk_ids, d["w13"].numpy(), d["s13"].numpy(),
                                     d["w2"].numpy(), d["s2"].numpy())
    err = rel_err(got, ref)
    print(f"  rel err vs quantised fp64 reference {err_q:.3e} (max abs {np.abs(got - ref_q).max():.3e}); "
          f"vs unquantised-activation reference {err:.3e} (max abs {np.abs(got - ref).max():.3e})", flush=True)
    assert err_q <= 1e-2
    assert err <= 5e-2


@pytest.mark.parametrize("name", ["c1_tiny", "c4_small"])
def test_layer_intermediates_bit_exact(name):
    """Every bit-exact gate of the layer: permutation, int8 activations at both quantisation
    points, int32 accumulators of both GEMMs."""
    from vllm_ascend_amd import kernels as K

    cfg = CONFIGS[name]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    tr = oracle_layer(cfg, d)
    _, ids = layer.router.select_experts(x, logits)
    xs, dst, cnt, sx = K.init_routing(x, ids, cfg.E, 1, 1)
    assert np.array_equal(dst.cpu().numpy(), tr.expanded_row_idx)
    assert np.array_equal(xs.cpu().numpy(), tr.xs)
    assert np.array_equal(sx.cpu().numpy().view(np.uint32), tr.sx.view(np.uint32))
    acc1 = K.gmm_i32(xs, layer.w13_weight.data, cnt, 1, 2 * cfg.I, cfg.H)
    assert np.array_equal(acc1.cpu().numpy(), tr.acc1)
    q1, s1 = K.gmm1_swiglu_quant(xs, layer.w13_weight.data, layer.w13_weight_scale_fp32, sx, cnt, 1, 2 * cfg.I, cfg.H)
    assert np.array_equal(q1.cpu().numpy(), tr.q1)
    assert np.array_equal(s1.cpu().numpy().view(np.uint32), tr.s1.view(np.uint32))
    acc2 = K.gmm_i32(q1, layer.w2_weight.data, cnt, 1, cfg.H, cfg.I)
    assert np.array_equal(acc2.cpu().numpy(), tr.acc2)
    o = K.gmm2_dequant(q1, layer.w2_weight.data, layer.w2_weight_scale_fp32, s1, cnt, 1, cfg.H, cfg.I)
    assert np.array_equal(bits(o), tr.o)


def test_cpu_tensors_are_refused():
    from vllm_ascend_amd import kernels as K

    with pytest.raises(RuntimeError, match="no CPU implementation"):
        K.dynamic_quant(torch.zeros(2, 8, dtype=torch.bfloat16))


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("name", ["c5_small", "c5_small_perchannel"])
def test_w4a8_layer_bit_exact(name, fused):
    """W4A8 variant (int4 weights, per-group or per-channel scales, Zipf-skewed routing); fused: token rows
    quantised once and read through the row -> token map, or the op-by-op path with its permuted copy."""
    cfg = CONFIGS[name]
    print(f"w4a8 layer {name} fused={fused}", flush=True)
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV)
    layer.use_fused_small_batch = fused
    res = layer.forward_impl(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d)
    assert np.array_equal(res.expert_tokens.cpu().numpy(), tr.expert_tokens)
    assert np.array_equal(bits(res.routed_out), tr.out)


def test_w4a8_packed_source_gives_the_same_tiles():
    """The reference's packing (two int4 per byte along N, low nibble = even channel;
    vllm_ascend/quantization/methods/w4a8.py:327-336) and the one-value-per-int8 checkpoint form
    must cast to identical tiled storage."""
    from vllm_ascend_amd import kernels as K

    g = torch.Generator().manual_seed(1)
    E, N, Kd = 3, 64, 128
    w = torch.randint(-8, 8, (E, N, Kd), generator=g, dtype=torch.int8)
    wkn = w.transpose(1, 2).contiguous()  # [E, K, N]
    pairs = wkn.reshape(E, Kd, N // 2, 2)
    packed = ((pairs[..., 1] << 4) | (pairs[..., 0] & 0x0F)).to(torch.int8).contiguous()  # [E, K, N/2]
    a = K.format_cast_nz_int4(w.to(DEV), 0, N, Kd)
    b = K.format_cast_nz_int4(packed.to(DEV), 1, N, Kd)
    assert torch.equal(a, b)


@pytest.mark.parametrize("overlap", [False, True])
def test_layer_with_shared_expert(overlap):
    """DeepSeek-V3-shaped structure (sigmoid, groups, bias, scaling factor) plus the shared expert, whose
    output is added inside the combine; with and without the second stream."""
    cfg = CONFIGS["c4_small"]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV, shared=True, overlap=overlap)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    for _ in range(3):  # repeated calls: the side-stream fences must hold every time
        res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d, shared=True)
    assert np.array_equal(bits(res.shared_out), tr.extra["shared_out"])
    assert np.array_equal(bits(res.routed_out), tr.out)


def test_layer_with_prequantised_hidden_states():
    """ascend_pertoken_scale + int8 hidden states (vllm_ascend/ops/fused_moe/moe_mlp.py:226-242,
    token_dispatcher.py:399-435): the dispatcher moves rows and scales, the MLP does not quantise again.  Handing
    the layer the quantiser's own output must give the bits of the ordinary path."""
    from vllm_ascend_amd import kernels as K

    for name in ("c2_small", "c4_small"):
        cfg = CONFIGS[name]
        d = make_layer(cfg, seed=0)
        layer = build_layer(cfg, d, DEV)
        x, logits = d["x"].to(DEV), d["logits"].to(DEV)
        xq, s = K.dynamic_quant(x)
        layer.ascend_pertoken_scale = s
        res = layer.forward_impl(xq, logits)
        torch.cuda.synchronize()
        layer.ascend_pertoken_scale = None
        tr = oracle_layer(cfg, d, keep_acc=False)
        assert res.routed_out.dtype == torch.bfloat16
        assert np.array_equal(bits(res.routed_out), tr.out), name
        with pytest.raises(ValueError, match="int8 hidden states"):
            layer.ascend_pertoken_scale = s
            try:
                layer.forward_impl(x, logits)
            finally:
                layer.ascend_pertoken_scale = None


def test_apply_router_weight_on_input():
    """top-1 routing with the weight applied to the expert's INPUT (token_dispatcher.py:409-413):
    x' = x * w in the model dtype before the dispatch; the combine still multiplies by w, as the reference's
    does (the metadata keeps topk_weights).  Checked against the checker fed with x'."""
    import dataclasses

    from oracle import oracle as orc

    cfg = dataclasses.replace(CONFIGS["c2_small"], name="top1", k=1, renorm=0)
    d = make_layer(cfg, seed=3)
    layer = build_layer(cfg, d, DEV)
    layer.apply_router_weight_on_input = True
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    kw = dict(k_group=1, group_count=1, group_select_mode=1, renorm=0, norm_type=0, routed_scaling_factor=1.0)
    y, ids, _ = orc.gating_top_k(d["logits"].numpy(), 1, x_dtype="f32", **kw)
    w_bf16 = orc.f32_to_bf16(y)
    # bf16 * bf16 -> bf16 on the GPU (torch): one fp32 product, one rounding
    x_scaled = orc.f32_to_bf16(orc.bf16_to_f32(bits(d["x"])) * orc.bf16_to_f32(w_bf16))
    tr = orc.experts_forward(x_scaled, w_bf16, ids, d["w13"].numpy(), d["s13"].numpy(), d["w2"].numpy(),
                             d["s2"].numpy(), keep_acc=False)
    assert np.array_equal(bits(res.routed_out), tr.out)
    layer.apply_router_weight_on_input = False
    res_plain = layer.forward_impl(x, logits)
    assert not torch.equal(res_plain.routed_out, res.routed_out)
    # top-k > 1 is refused, as in the reference
    cfg2 = CONFIGS["c2_small"]
    d2 = make_layer(cfg2, seed=0)
    layer2 = build_layer(cfg2, d2, DEV)
    layer2.apply_router_weight_on_input = True
    with pytest.raises(AssertionError, match="topk=1"):
        layer2.forward_impl(d2["x"].to(DEV), d2["logits"].to(DEV))


def test_force_load_balance_routes_every_token_to_k_distinct_experts():
    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV)
    layer.enable_force_load_balance = True
    res = layer.forward_impl(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    assert int(res.expert_tokens.sum()) == cfg.T * cfg.k
    assert torch.isfinite(res.routed_out.float()).all()
    w, ids = layer.router.select_experts(d["x"].to(DEV), d["logits"].to(DEV), enable_force_load_balance=True)
    assert all(len(set(r)) == cfg.k for r in ids.cpu().tolist())


def test_force_load_balance_with_log2phy_keeps_the_random_ids_unmapped():
    """Both profile-run flags at once: the reference maps through log2phy and then overwrites the ids with random
    logical ids that are not mapped again (routed_experts.py:452-492), so no token may land on a redundant copy."""
    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV, redundant=(3, 1))
    log2phy = torch.arange(cfg.E, dtype=torch.int32, device=DEV)
    log2phy[3] = cfg.E
    log2phy[1] = cfg.E + 1
    layer.log2phy = log2phy
    layer.enable_force_load_balance = True
    res = layer.forward_impl(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    counts = res.expert_tokens.cpu()
    assert int(counts.sum()) == cfg.T * cfg.k
    assert int(counts[cfg.E:].sum()) == 0          # the copies stay idle: ids were not mapped
    assert int(counts[3]) + int(counts[1]) > 0     # ... and the logical experts 1 and 3 are used as they are
    assert torch.isfinite(res.routed_out.float()).all()


@pytest.mark.parametrize("act", ["gelu", "gelu_tanh", "swiglustep", "swigluoai_uninterleave"])
@pytest.mark.parametrize("name", ["c2_small", "c3_small"])
def test_layer_with_other_activations(name, act):
    """Activations without a fused op take the unfused branch (vllm_ascend/ops/fused_moe/moe_mlp.py:484-569):
    gate_up product to 16 bits, activation * up + dynamic quantisation, down product; bit for bit the checker's."""
    import dataclasses

    from oracle import oracle as orc

    cfg = CONFIGS[name]
    print(f"layer {name} activation={act}", flush=True)
    d = make_layer(cfg, seed=2)
    layer = build_layer(cfg, d, DEV)
    limit, alpha, beta = (0.0, 1.0, 0.0) if act != "swigluoai_uninterleave" else (7.0, 1.702, 1.0)
    layer.activation = act
    layer.moe_config = dataclasses.replace(layer.moe_config, activation=act, swiglu_limit=limit, swiglu_alpha=alpha,
                                           swiglu_beta=beta)
    layer.moe_comm_method.moe_config = layer.moe_config
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    kw = dict(k_group=1, group_count=1, group_select_mode=1, renorm=1, norm_type=0, x_dtype="f32")
    y, ids, _ = orc.gating_top_k(d["logits"].numpy(), cfg.k, **kw)
    tr = orc.experts_forward(bits(d["x"]), orc.f32_to_half(y), ids, d["w13"].numpy(), d["s13"].numpy(),
                             d["w2"].numpy(), d["s2"].numpy(), activation=act.replace("_uninterleave", ""),
                             swiglu_limit=limit, swiglu_alpha=alpha, swiglu_beta=beta)
    assert np.array_equal(res.expert_tokens.cpu().numpy(), tr.expert_tokens)
    assert np.array_equal(bits(res.routed_out), tr.out)
    silu = oracle_layer(cfg, d)
    assert not np.array_equal(tr.out, silu.out)  # the activation is really a different one
    if act == "swigluoai_uninterleave":
        # the interleaved name is not known to the reference's quantised MLP (moe_mlp.py:213): it takes the default
        # branch there, the fused SwiGLU with the limit, and so it does here
        layer.activation = "swigluoai"
        layer.moe_config = dataclasses.replace(layer.moe_config, activation="swigluoai")
        layer.moe_comm_method.moe_config = layer.moe_config
        res = layer.forward_impl(x, logits)
        torch.cuda.synchronize()
        tr = orc.experts_forward(bits(d["x"]), orc.f32_to_half(y), ids, d["w13"].numpy(), d["s13"].numpy(),
                                 d["w2"].numpy(), d["s2"].numpy(), swiglu_limit=limit)
        assert np.array_equal(bits(res.routed_out), tr.out)


def test_layer_with_per_expert_weight_lists():
    """dynamic-EPLB form: every expert's weights and scales are separate tensors; swapping two experts'
    tensors in place must swap what they compute."""
    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV, dynamic_eplb=True)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    res = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d)
    assert np.array_equal(bits(res.routed_out), tr.out)
    # swap experts 0 and 1 in the lists AND in the checker's inputs
    views = layer.quant_method.get_eplb_weight_views(layer)
    for lst in views:
        lst[0], lst[1] = lst[1], lst[0]
    for name in ("w13", "w2", "s13", "s2"):
        t = d[name].clone()
        t[0], t[1] = d[name][1], d[name][0]
        d[name] = t
    res2 = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    assert np.array_equal(bits(res2.routed_out), oracle_layer(cfg, d).out)
    assert not torch.equal(res.routed_out, res2.routed_out)


@pytest.mark.parametrize("fused", [True, False])
def test_expert_load_collection(fused):
    """The layer sums the tokens every expert received over its forward passes (what the load balancer
    reads): one row, or one row per pass of a collection interval; collection can be paused and cleared."""
    print(f"expert load collection fused={fused}", flush=True)
    cfg = CONFIGS["c2_small"]
    d = make_layer(cfg, seed=2)
    plain = build_layer(cfg, d, DEV)
    want = np.bincount(oracle_layer(cfg, d).topk_ids.reshape(-1), minlength=cfg.E)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    for interval in (None, 2):
        # with the interval: also the per-expert weight lists that dynamic load balancing swaps in place
        layer = build_layer(cfg, d, DEV, dynamic_eplb=interval is not None, collect_expert_load=True,
                            heat_interval=interval)
        layer.use_fused_small_batch = fused
        for _ in range(3):
            out = layer.forward_impl(x, logits).routed_out
        layer.eplb_heat_collection_status = False
        layer.forward_impl(x, logits)
        torch.cuda.synchronize()
        assert torch.equal(out, plain.forward_impl(x, logits).routed_out)
        got = layer.moe_load.cpu().numpy()
        if interval is None:
            assert got.dtype == np.int64 and np.array_equal(got, 3 * want)
        else:
            assert got.dtype == np.int32 and np.array_equal(got, np.stack([2 * want, want]))
            assert int(layer.load_counter) == 3
        layer.clear_moe_load()
        assert int(layer.moe_load.abs().sum()) == 0


@pytest.mark.parametrize("name", ["c2_small", "c5_small"])
@pytest.mark.parametrize("fused", [True, "sorted", False])
def test_redundant_experts_through_log2phy(name, fused):
    """Two physical copies of logical experts behind the logical -> physical map: the router scores the logical
    experts, the dispatch runs over the physical ones, the output is the one of the layer without copies, and
    the tokens of a remapped expert are counted on its copy."""
    print(f"log2phy {name} fused={fused}", flush=True)
    cfg = CONFIGS[name]
    d = make_layer(cfg, seed=4)
    x, logits = d["x"].to(DEV), d["logits"].to(DEV)
    plain = build_layer(cfg, d, DEV)
    want = plain.forward_impl(x, logits)
    layer = build_layer(cfg, d, DEV, redundant=(3, 1))
    layer.use_fused_small_batch = bool(fused)
    layer.use_pair_order = fused is True
    log2phy = torch.arange(cfg.E, dtype=torch.int32, device=DEV)
    log2phy[3] = cfg.E  # every token of logical expert 3 goes to its copy; the copy of expert 1 stays idle
    layer.log2phy = log2phy
    got = layer.forward_impl(x, logits)
    torch.cuda.synchronize()
    assert torch.equal(got.routed_out, want.routed_out)
    assert np.array_equal(bits(got.routed_out), oracle_layer(cfg, d).out)
    counts, base = got.expert_tokens.cpu(), want.expert_tokens.cpu()
    assert counts.shape[0] == cfg.E + 2 and int(counts[3]) == 0 and int(counts[cfg.E + 1]) == 0
    assert int(counts[cfg.E]) == int(base[3])
    keep = [e for e in range(cfg.E) if e != 3]
    assert torch.equal(counts[keep], base[keep])
    assert layer.get_log2phy_map() is log2phy


@pytest.mark.parametrize("name", ["c2_small", "c4_small", "c5_small"])
def test_empty_and_single_token_batches(name):
    """T = 0 (a rank with nothing to do in a padded step) returns an empty result without launching anything
    that faults; T = 1 is bit-exact like any other batch."""
    print(f"empty / single-token batch {name}", flush=True)
    import dataclasses

    cfg = CONFIGS[name]
    d = make_layer(cfg, seed=0)
    layer = build_layer(cfg, d, DEV, shared=cfg.shared)
    res = layer.forward_impl(d["x"][:0].to(DEV), d["logits"][:0].to(DEV))
    torch.cuda.synchronize()
    assert tuple(res.routed_out.shape) == (0, cfg.H)
    assert int(res.expert_tokens.sum()) == 0
    d1 = dict(d)
    d1["x"], d1["logits"] = d["x"][:1].contiguous(), d["logits"][:1].contiguous()
    res = layer.forward_impl(d1["x"].to(DEV), d1["logits"].to(DEV))
    torch.cuda.synchronize()
    tr = oracle_layer(dataclasses.replace(cfg, T=1), d1, shared=cfg.shared)
    assert np.array_equal(bits(res.routed_out), tr.out)


def _random_layer_cfg(seed):
    """A random but valid layer: softmax or sigmoid, with or without expert groups / bias / shared expert /
    Zipf-skewed routing / int4 weights, sizes small enough for the CPU checker."""
    from _inputs import LayerCfg

    rng = np.random.default_rng(seed)
    n_group = int(rng.choice([1, 1, 2, 4]))
    per_group = int(rng.choice([2, 4, 8]))
    E = n_group * per_group
    topk_group = int(rng.integers(1, n_group + 1))
    k = int(rng.integers(1, min(8, topk_group * per_group) + 1))
    w4 = seed % 4 == 3
    H = int(rng.choice([256, 512])) if w4 else int(rng.choice([128, 192, 320, 512]))
    I = int(rng.choice([128, 256])) if w4 else int(rng.choice([32, 96, 160, 256]))
    return LayerCfg(
        f"random_{seed}", T=int(rng.choice([1, 7, 33, 130, 600])), H=H, E=E, k=k, I=I,
        scoring=str(rng.choice(["softmax", "sigmoid"])), n_group=n_group, topk_group=topk_group,
        renorm=int(rng.integers(0, 2)), routed_scaling_factor=float(rng.choice([1.0, 2.5])),
        bias=bool(rng.integers(0, 2)), shared=bool(rng.integers(0, 2)) and not w4,
        w4_group=int(rng.choice([0, 128])) if w4 else -1, zipf=float(rng.choice([0.0, 1.1])))


@pytest.mark.parametrize("seed", range(12))
def test_layer_on_random_configurations(seed):
    cfg = _random_layer_cfg(seed)
    print(f"random layer {cfg}", flush=True)
    d = make_layer(cfg, seed=100 + seed)
    layer = build_layer(cfg, d, DEV, shared=cfg.shared)
    res = layer.forward_impl(d["x"].to(DEV), d["logits"].to(DEV))
    torch.cuda.synchronize()
    tr = oracle_layer(cfg, d, shared=cfg.shared)
    if cfg.shared:
        assert np.array_equal(bits(res.shared_out), tr.extra["shared_out"])
    assert np.array_equal(bits(res.routed_out), tr.out)
    assert np.array_equal(res.expert_tokens.cpu().numpy() if res.expert_tokens is not None else tr.expert_tokens,
                          tr.expert_tokens)
