"""Build the plugin-side layer object from synthetic tensors, and run the CPU checker on the same inputs."""
from __future__ import annotations

import numpy as np
import torch

from _inputs import LayerCfg, bits, gating_kwargs


def build_layer(cfg: LayerCfg, d: dict, device="cuda:0", shared=False, overlap=False, dynamic_eplb=False,
                collect_expert_load=False, heat_interval=None, redundant=()):
    """redundant: logical expert ids whose weights are appended as extra physical experts (the router still
    scores cfg.E logical experts)."""
    from vllm_ascend_amd.fused_moe.contracts import FusedMoEConfig
    from vllm_ascend_amd.fused_moe.layer import AscendRoutedExperts
    from vllm_ascend_amd.fused_moe.router import AscendFusedTopKRouter
    from vllm_ascend_amd.quantization import get_scheme_class

    if redundant:
        d = dict(d)
        idx = torch.tensor(list(range(cfg.E)) + list(redundant))
        for name in ("w13", "w2", "s13", "s2"):
            d[name] = d[name][idx].contiguous()
    moe_config = FusedMoEConfig(num_experts=cfg.E + len(redundant), experts_per_token=cfg.k, hidden_dim=cfg.H,
                                intermediate_size_per_partition=cfg.I)
    router = AscendFusedTopKRouter(
        cfg.k, cfg.E, renormalize=bool(cfg.renorm), use_grouped_topk=cfg.n_group > 1,
        num_expert_group=cfg.n_group if cfg.n_group > 1 else None,
        topk_group=cfg.topk_group if cfg.n_group > 1 else None, scoring_func=cfg.scoring,
        routed_scaling_factor=cfg.routed_scaling_factor,
        e_score_correction_bias=d["bias"].to(device) if cfg.bias else None)
    shared_experts = None
    if shared and cfg.shared:
        from vllm_ascend_amd.fused_moe.shared_experts import AscendSharedExperts

        shared_experts = AscendSharedExperts(d["sw13"][0].to(device), d["ss13"][0].to(device), d["sw2"][0].to(device),
                                             d["ss2"][0].to(device), multistream_overlap=overlap)
    if cfg.w4_group >= 0:
        scheme = get_scheme_class("W4A8_DYNAMIC", "moe")(group_size=cfg.w4_group)
        layer = AscendRoutedExperts(moe_config, scheme, router, params_dtype=torch.float32, device=device)
        layer.load_weights({"w13_weight": d["w13"].to(device), "w2_weight": d["w2"].to(device),
                            "w13_weight_scale": d["s13"].to(device), "w2_weight_scale": d["s2"].to(device)})
        return layer
    scheme = get_scheme_class("W8A8_DYNAMIC", "moe")(dynamic_eplb=dynamic_eplb)
    layer = AscendRoutedExperts(moe_config, scheme, router, params_dtype=torch.float32, device=device,
                                shared_experts=shared_experts, dynamic_eplb=collect_expert_load,
                                expert_heat_collection_interval=heat_interval)
    layer.load_weights({
        "w13_weight": d["w13"].to(device), "w2_weight": d["w2"].to(device),
        "w13_weight_scale": d["s13"].to(device), "w2_weight_scale": d["s2"].to(device),
        "w13_weight_offset": torch.zeros_like(d["s13"]).to(device),
        "w2_weight_offset": torch.zeros_like(d["s2"]).to(device),
    })
    return layer


def oracle_layer(cfg: LayerCfg, d: dict, keep_acc=True, shared=False):
    from oracle import oracle as orc

    kw = gating_kwargs(cfg)
    if cfg.w4_group >= 0:
        y, ids, _ = orc.gating_top_k(d["logits"].numpy(), cfg.k, bias=d["bias"].numpy() if cfg.bias else None,
                                     k_group=kw["k_group"], group_count=kw["group_count"], group_select_mode=1,
                                     renorm=kw["renorm"], norm_type=kw["norm_type"],
                                     routed_scaling_factor=kw["routed_scaling_factor"], x_dtype="f32")
        # scales travel as [E, N, G] in the checkpoint; the checker takes [E, G, N]
        sg13 = np.ascontiguousarray(d["s13"].numpy().transpose(0, 2, 1))
        sg2 = np.ascontiguousarray(d["s2"].numpy().transpose(0, 2, 1))
        return orc.w4a8_experts_forward(bits(d["x"]), orc.f32_to_half(y), ids, d["w13"].numpy(), sg13,
                                        d["w2"].numpy(), sg2, cfg.w4_group)
    sh = None
    if shared and cfg.shared:
        sh = (d["sw13"].numpy(), d["ss13"].numpy(), d["sw2"].numpy(), d["ss2"].numpy())
    return orc.moe_layer(bits(d["x"]), d["logits"].numpy(), d["w13"].numpy(), d["s13"].numpy(), d["w2"].numpy(),
                         d["s2"].numpy(), top_k=cfg.k, bias=d["bias"].numpy() if cfg.bias else None,
                         k_group=kw["k_group"], group_count=kw["group_count"], renorm=kw["renorm"],
                         norm_type=kw["norm_type"], routed_scaling_factor=kw["routed_scaling_factor"],
                         keep_acc=keep_acc, shared=sh)


def rel_err(a: np.ndarray, b: np.ndarray) -> float:
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
