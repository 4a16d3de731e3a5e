"""ModelSlim description file and per-expert checkpoint tensors -> one fused-MoE layer.  The cases of the
configuration part follow the reference's own unit tests (tests/ut/quantization/test_modelslim_config.py); the
loader is checked against the stacked tensors it has to produce, and on the GPU against a layer that was handed
the stacked tensors directly."""
import json
import os
from unittest.mock import MagicMock

import numpy as np
import pytest
import torch

from _inputs import CONFIGS, make_layer
from vllm_ascend_amd.quantization import get_scheme_class
from vllm_ascend_amd.quantization.checkpoint import (SAFETENSORS_INDEX, SafetensorsDirectory, load_routed_experts,
                                                     moe_weight_loader, routed_experts_from_checkpoint)
from vllm_ascend_amd.quantization.modelslim_config import (MODELSLIM_CONFIG_FILENAME, AscendModelSlimConfig,
                                                           _make_modelslim_moe_weight_loader, create_scheme_for_layer,
                                                           get_linear_quant_type, packed_modules_model_mapping)

PREFIX = "model.layers.3.mlp.experts"


def write_checkpoint(path, d, quant_type, n_shards=2, with_index=True, w4=False):
    """Per-expert gate/up/down tensors of the synthetic layer `d` in ModelSlim naming, over `n_shards` files."""
    from safetensors.torch import save_file

    E, two_i, _ = d["w13"].shape
    I = two_i // 2
    tensors = {}
    for e in range(E):
        for module, w, s in (("gate_proj", d["w13"][e, :I], d["s13"][e, :I]), ("up_proj", d["w13"][e, I:], d["s13"][e, I:]),
                             ("down_proj", d["w2"][e], d["s2"][e])):
            tensors[f"{PREFIX}.{e}.{module}.weight"] = w.contiguous()
            tensors[f"{PREFIX}.{e}.{module}.weight_scale"] = (s if w4 else s.reshape(-1, 1)).contiguous()
            if not w4:
                tensors[f"{PREFIX}.{e}.{module}.weight_offset"] = torch.zeros(s.numel(), 1)
    tensors["model.layers.3.mlp.gate.weight"] = torch.zeros(E, d["w13"].shape[2])
    names = sorted(tensors)
    weight_map = {}
    for i in range(n_shards):
        fn = f"model-{i + 1:05d}-of-{n_shards:05d}.safetensors"
        part = {n: tensors[n] for n in names[i::n_shards]}
        save_file(part, os.path.join(path, fn))
        weight_map.update({n: fn for n in part})
    if with_index:
        with open(os.path.join(path, SAFETENSORS_INDEX), "w") as f:
            json.dump({"metadata": {}, "weight_map": weight_map}, f)
    desc = {n: ("FLOAT" if n.endswith("gate.weight") else quant_type) for n in names}
    with open(os.path.join(path, MODELSLIM_CONFIG_FILENAME), "w") as f:
        json.dump(desc, f)
    return desc


# ------------------------------------------------------------------ description file
def test_config_basics():
    sample = {"layer1.weight": "INT8", "layer2.weight": "FLOAT", "fused_layer.weight": "FLOAT",
              "fused_layer.shard1.weight": "FLOAT", "fused_layer.shard2.weight": "FLOAT",
              "shard1.weight": "FLOAT", "shard2.weight": "FLOAT"}
    cfg = AscendModelSlimConfig(sample)
    assert cfg.quant_description == sample
    assert repr(cfg).startswith("AscendModelSlimConfig:\n")
    assert AscendModelSlimConfig.get_name() == "ascend"
    assert AscendModelSlimConfig.get_config_filenames() == []
    assert AscendModelSlimConfig.from_config(sample).quant_description == sample
    assert AscendModelSlimConfig().quant_description == {}
    # FLOAT means "skip quantisation"
    assert not cfg.is_layer_skipped_ascend("layer1")
    assert cfg.is_layer_skipped_ascend("layer2")
    fused = {"fused_layer": ["shard1", "shard2"]}
    assert cfg.is_layer_skipped_ascend("fused_layer", fused)
    with pytest.raises(ValueError):
        AscendModelSlimConfig({"shard1.weight": "FLOAT", "shard2.weight": "INT8"}).is_layer_skipped_ascend(
            "fused_layer", fused)


def test_quant_type_over_packed_shards():
    fused = {"qkv_proj": ["q_proj", "k_proj", "v_proj"]}
    prefix = "model.layers.5.self_attn.qkv_proj"
    desc = {f"model.layers.5.self_attn.{p}.weight": "W8A8_DYNAMIC" for p in ("q_proj", "k_proj", "v_proj")}
    assert get_linear_quant_type(desc, prefix, fused) == "W8A8_DYNAMIC"
    assert get_linear_quant_type({"a.b.weight": "W4A8_DYNAMIC"}, "a.b", {}) == "W4A8_DYNAMIC"
    mixed = dict(desc)
    mixed["model.layers.5.self_attn.v_proj.weight"] = "W8A8"
    with pytest.raises(ValueError, match="Not all shards"):
        get_linear_quant_type(mixed, prefix, fused)
    del desc["model.layers.5.self_attn.q_proj.weight"]
    with pytest.raises(KeyError):
        get_linear_quant_type(desc, prefix, fused)
    with pytest.raises(KeyError):
        AscendModelSlimConfig(desc).is_layer_skipped_ascend(prefix, fused)


def test_scheme_creation_from_the_description():
    experts = packed_modules_model_mapping["qwen3_moe"]
    desc = {f"{PREFIX}.0.{m}.weight": "W8A8_DYNAMIC" for m in ("gate_proj", "up_proj", "down_proj")}
    scheme = create_scheme_for_layer(desc, PREFIX, "moe", experts)
    assert type(scheme) is get_scheme_class("W8A8_DYNAMIC", "moe")
    desc4 = {k: "W4A8_DYNAMIC" for k in desc}
    scheme = AscendModelSlimConfig(desc4).get_moe_scheme(PREFIX, "qwen3_moe", group_size=256)
    assert type(scheme) is get_scheme_class("W4A8_DYNAMIC", "moe") and scheme.group_size == 256
    with pytest.raises(NotImplementedError):
        create_scheme_for_layer({k: "W2A2" for k in desc}, PREFIX, "moe", experts)
    with pytest.raises(NotImplementedError, match="FLOAT"):
        AscendModelSlimConfig({k: "FLOAT" for k in desc}).get_moe_scheme(PREFIX, "qwen3_moe")
    with pytest.raises(NotImplementedError):
        create_scheme_for_layer(desc, PREFIX, "attention", experts)


def test_config_file_lookup(tmp_path):
    cfg = AscendModelSlimConfig({"x.weight": "INT8"})
    cfg.maybe_update_config(str(tmp_path / "nowhere"))     # already populated: nothing is read
    assert cfg.quant_description == {"x.weight": "INT8"}
    data = {"layer.weight": "INT8"}
    (tmp_path / MODELSLIM_CONFIG_FILENAME).write_text(json.dumps(data))
    cfg = AscendModelSlimConfig()
    cfg.maybe_update_config(str(tmp_path))
    assert cfg.quant_description == data
    empty = tmp_path / "float_model"
    empty.mkdir()
    (empty / "config.json").write_text("{}")
    with pytest.raises(ValueError) as exc:
        AscendModelSlimConfig().maybe_update_config(str(empty))
    assert "ModelSlim Quantization Config Not Found" in str(exc.value)
    assert MODELSLIM_CONFIG_FILENAME in str(exc.value) and "config.json" in str(exc.value)
    with pytest.raises(ValueError, match="ModelSlim Quantization Config Not Found"):
        AscendModelSlimConfig().maybe_update_config(str(tmp_path / "not_a_directory"))


def test_modelslim_moe_weight_loader_maps_scale_bias_to_scale_path():
    upstream = MagicMock(return_value=True)
    loader = _make_modelslim_moe_weight_loader(upstream)
    param, loaded = torch.nn.Parameter(torch.empty(1)), torch.empty(1)
    assert loader(param=param, loaded_weight=loaded, weight_name="model.layers.0.mlp.experts.w2_scale_bias",
                  shard_id="w2", expert_id=0, return_success=True)
    upstream.assert_called_once_with(param=param, loaded_weight=loaded,
                                     weight_name="model.layers.0.mlp.experts.w2_scale", shard_id="w2", expert_id=0,
                                     return_success=True)
    upstream.reset_mock()
    loader(param=param, loaded_weight=loaded, weight_name="a.w13_weight", shard_id="w1", expert_id=2)
    assert upstream.call_args.kwargs["weight_name"] == "a.w13_weight"


# ------------------------------------------------------------------ stacking
def test_moe_weight_loader_slices():
    p = torch.nn.Parameter(torch.zeros(3, 8, 5), requires_grad=False)
    g, u = torch.full((4, 5), 1.0), torch.full((4, 5), 2.0)
    assert moe_weight_loader(p, g, "w13_weight", "w1", 1, return_success=True) is True
    assert moe_weight_loader(p, u, "w13_weight", "w3", 1) is None
    assert torch.equal(p.data[1, :4], g) and torch.equal(p.data[1, 4:], u) and p.data[0].abs().sum() == 0
    s = torch.nn.Parameter(torch.zeros(3, 8, 1), requires_grad=False)
    moe_weight_loader(s, torch.arange(4.0), "w13_weight_scale", "w3", 2)          # [N] into [N, 1]
    assert torch.equal(s.data[2, 4:, 0], torch.arange(4.0))
    w2 = torch.nn.Parameter(torch.zeros(3, 5, 4), requires_grad=False)
    moe_weight_loader(w2, torch.ones(5, 4), "w2_weight", "w2", 0)
    assert w2.data[0].sum() == 20
    with pytest.raises(ValueError, match="does not fit"):
        moe_weight_loader(p, torch.zeros(8, 5), "w13_weight", "w1", 0)
    with pytest.raises(IndexError):
        moe_weight_loader(p, g, "w13_weight", "w1", 3)
    with pytest.raises(ValueError, match="shard_id"):
        moe_weight_loader(p, g, "w13_weight", "w4", 0)


class _CpuLayer(torch.nn.Module):
    """The registered parameters of a routed-experts layer without the device side."""

    def __init__(self, scheme, E, I, H):
        super().__init__()
        self.quant_method = scheme
        specs = dict(scheme.get_weight(E, I, H, torch.float32))
        specs.update(scheme.get_dynamic_quant_param(E, I, H, torch.float32))
        for name, t in specs.items():
            self.register_parameter(name, torch.nn.Parameter(torch.zeros_like(t), requires_grad=False))
        self.weight_loader = moe_weight_loader


@pytest.mark.parametrize("with_index", [True, False])
def test_stacking_from_a_sharded_checkpoint(tmp_path, with_index):
    cfg = CONFIGS["c1_tiny"]
    d = make_layer(cfg, seed=3)
    write_checkpoint(str(tmp_path), d, "W8A8_DYNAMIC", n_shards=3, with_index=with_index)
    ckpt = SafetensorsDirectory(str(tmp_path))
    assert len(list(ckpt.names())) == cfg.E * 9 + 1
    conf = AscendModelSlimConfig()
    conf.maybe_update_config(str(tmp_path))
    layer = _CpuLayer(conf.get_moe_scheme(PREFIX, "qwen3_moe"), cfg.E, cfg.I, cfg.H)
    loaded = load_routed_experts(layer, str(tmp_path), PREFIX, post_process=False)
    assert len(loaded) == cfg.E * 9
    assert torch.equal(layer.w13_weight.data, d["w13"]) and torch.equal(layer.w2_weight.data, d["w2"])
    assert torch.equal(layer.w13_weight_scale.data[..., 0], d["s13"])
    assert torch.equal(layer.w2_weight_scale.data[..., 0], d["s2"])
    assert layer.w13_weight_offset.data.abs().sum() == 0


def test_loader_refuses_incomplete_or_foreign_checkpoints(tmp_path):
    from safetensors.torch import save_file

    cfg = CONFIGS["c1_tiny"]
    d = make_layer(cfg, seed=4)
    scheme = get_scheme_class("W8A8_DYNAMIC", "moe")()
    # a tensor the scheme has no parameter for
    a = tmp_path / "a"
    a.mkdir()
    write_checkpoint(str(a), d, "W8A8_DYNAMIC", n_shards=1, with_index=False)
    save_file({f"{PREFIX}.0.gate_proj.deq_scale": torch.zeros(4)}, str(a / "extra.safetensors"))
    with pytest.raises(KeyError, match="w13_deq_scale"):
        load_routed_experts(_CpuLayer(scheme, cfg.E, cfg.I, cfg.H), str(a), PREFIX, post_process=False)
    load_routed_experts(_CpuLayer(scheme, cfg.E, cfg.I, cfg.H), str(a), PREFIX, ignore_suffixes=("deq_scale",),
                        post_process=False)
    # one expert too few in the checkpoint
    with pytest.raises(KeyError, match="not in the checkpoint"):
        load_routed_experts(_CpuLayer(scheme, cfg.E + 1, cfg.I, cfg.H), str(a), PREFIX, ignore_suffixes=("deq_scale",),
                            post_process=False)
    # wrong intermediate size
    with pytest.raises(ValueError, match="does not fit"):
        load_routed_experts(_CpuLayer(scheme, cfg.E, cfg.I * 2, cfg.H), str(a), PREFIX,
                            ignore_suffixes=("deq_scale",), post_process=False)
    with pytest.raises(FileNotFoundError):
        SafetensorsDirectory(str(tmp_path / "missing"))
    b = tmp_path / "b"
    b.mkdir()
    with pytest.raises(FileNotFoundError, match="no safetensors"):
        SafetensorsDirectory(str(b))


# ------------------------------------------------------------------ on the GPU: the loaded layer computes what the
# directly built layer computes, and what the CPU checker computes
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c1_tiny", "w4a8_small"])
def test_layer_from_checkpoint_matches_layer_from_tensors(tmp_path, name):
    import dataclasses

    from _layer_utils import build_layer
    from vllm_ascend_amd.fused_moe.contracts import FusedMoEConfig
    from vllm_ascend_amd.fused_moe.router import AscendFusedTopKRouter

    if name == "w4a8_small":
        cfg = dataclasses.replace(CONFIGS["c5_w4a8_zipf"], name=name, T=48, E=8, H=512, I=256, n_group=1, topk_group=1)
    else:
        cfg = CONFIGS[name]
    w4 = cfg.w4_group >= 0
    print(f"layer from checkpoint {name} w4={w4}", flush=True)
    d = make_layer(cfg, seed=5)
    write_checkpoint(str(tmp_path), d, "W4A8_DYNAMIC" if w4 else "W8A8_DYNAMIC", w4=w4)
    ref_layer = build_layer(cfg, d)
    moe_config = FusedMoEConfig(num_experts=cfg.E, experts_per_token=cfg.k, hidden_dim=cfg.H,
                                intermediate_size_per_partition=cfg.I)
    router = AscendFusedTopKRouter(cfg.k, cfg.E, renormalize=bool(cfg.renorm), use_grouped_topk=cfg.n_group > 1,
                                   num_expert_group=cfg.n_group if cfg.n_group > 1 else None,
                                   topk_group=cfg.topk_group if cfg.n_group > 1 else None, scoring_func=cfg.scoring,
                                   routed_scaling_factor=cfg.routed_scaling_factor,
                                   e_score_correction_bias=d["bias"].to("cuda:0") if cfg.bias else None)
    kwargs = {"group_size": cfg.w4_group} if w4 else {}
    layer = routed_experts_from_checkpoint(str(tmp_path), PREFIX, moe_config, router, "qwen3_moe", device="cuda:0",
                                           **kwargs)
    x, logits = d["x"].to("cuda:0"), d["logits"].to("cuda:0")
    got = layer(x, logits)
    want = ref_layer(x, logits)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert np.isfinite(got.float().cpu().numpy()).all()
    # ... and both compute what the CPU checker computes from the tensors that were written to disk
    from _inputs import bits
    from _layer_utils import oracle_layer

    assert np.array_equal(bits(got), oracle_layer(cfg, d, keep_acc=False).out)
