"""From a ModelSlim checkpoint directory to the stacked parameters of one fused-MoE layer.

On disk (``docs/source/developer_guide/Design_Documents/quantization.md:29-47``) every expert is three linear
layers, ``<prefix>.<e>.{gate_proj,up_proj,down_proj}.{weight,weight_scale,weight_offset,...}``, in safetensors
shards listed by ``model.safetensors.index.json``; ``quant_model_description.json`` names their quant type.  In
the reference the stacking is done by vLLM's fused-MoE ``weight_loader`` (shard ``w1`` = gate rows ``[0, I)`` of
``w13``, ``w3`` = up rows ``[I, 2I)``, ``w2`` = the down projection), reached through the ModelSlim wrapper
(``vllm_ascend/quantization/modelslim_config.py:65-91, 759-765``); the scheme's
``process_weights_after_loading`` then casts to the device layout.  This module is that loader for one device
holding every expert.  Tensors are read one at a time through ``safetensors.safe_open`` (nothing is unpickled
and no shard is loaded whole)."""
from __future__ import annotations

import json
import os
import re
from typing import Iterator

import torch

from .modelslim_config import AscendModelSlimConfig, _make_modelslim_moe_weight_loader

SAFETENSORS_INDEX = "model.safetensors.index.json"
# checkpoint module -> (stacked parameter prefix, shard id of the fused-MoE loader)
_EXPERT_MODULES = {"gate_proj": ("w13", "w1"), "up_proj": ("w13", "w3"), "down_proj": ("w2", "w2")}


def moe_weight_loader(param: torch.nn.Parameter, loaded_weight: torch.Tensor, weight_name: str, shard_id: str,
                      expert_id: int, return_success: bool = False) -> bool | None:
    """Copy one expert's tensor into its slice of a stacked parameter ``[E, rows, ...]``.  ``w1`` / ``w3`` fill
    the first / second half of the rows of a ``w13`` parameter, ``w2`` the whole expert slice.  A tensor whose
    shape does not match its slice is an error, not a silent reshape."""
    if shard_id not in ("w1", "w2", "w3"):
        raise ValueError(f"shard_id must be w1, w2 or w3, got {shard_id!r}")
    if not 0 <= expert_id < param.data.shape[0]:
        raise IndexError(f"{weight_name}: expert {expert_id} outside [0, {param.data.shape[0]})")
    dst = param.data[expert_id]
    if shard_id != "w2":
        half = dst.shape[0] // 2
        dst = dst[:half] if shard_id == "w1" else dst[half:]
    src = loaded_weight
    if src.dim() == dst.dim() - 1:  # per-channel vectors are stored [N], the parameters are [N, 1]
        src = src.unsqueeze(-1)
    if tuple(src.shape) != tuple(dst.shape):
        raise ValueError(f"{weight_name} (expert {expert_id}, {shard_id}): checkpoint shape {tuple(src.shape)} "
                         f"does not fit the parameter slice {tuple(dst.shape)}")
    dst.copy_(src.to(dst.dtype))
    return True if return_success else None


class SafetensorsDirectory:
    """Tensor names of a checkpoint directory and lazy access to single tensors."""

    def __init__(self, model_dir: str):
        if not os.path.isdir(model_dir):
            raise FileNotFoundError(f"checkpoint directory {model_dir!r} does not exist")
        self.model_dir = model_dir
        index_path = os.path.join(model_dir, SAFETENSORS_INDEX)
        self.weight_map: dict[str, str] = {}
        if os.path.exists(index_path):
            with open(index_path) as f:
                self.weight_map = dict(json.load(f)["weight_map"])
        else:
            from safetensors import safe_open

            for fn in sorted(os.listdir(model_dir)):
                if fn.endswith(".safetensors"):
                    with safe_open(os.path.join(model_dir, fn), framework="pt") as f:
                        for key in f.keys():
                            self.weight_map[key] = fn
        if not self.weight_map:
            raise FileNotFoundError(f"no safetensors tensors found in {model_dir!r}")
        self._open: dict[str, object] = {}

    def names(self) -> Iterator[str]:
        return iter(self.weight_map)

    def get(self, name: str) -> torch.Tensor:
        from safetensors import safe_open

        fn = self.weight_map[name]
        if fn not in self._open:
            self._open[fn] = safe_open(os.path.join(self.model_dir, fn), framework="pt")
        return self._open[fn].get_tensor(name)

    def close(self) -> None:
        self._open.clear()


def load_routed_experts(layer, model_dir: str, prefix: str, ignore_suffixes: tuple[str, ...] = (),
                        post_process: bool = True) -> list[str]:
    """Fill the stacked parameters of ``layer`` (an ``AscendRoutedExperts``) from the per-expert tensors under
    ``prefix`` (``model.layers.N.mlp.experts``) and run the scheme's post-load processing.  Every registered
    parameter slice must be written exactly once and every checkpoint tensor under the prefix must have a
    parameter (except ``ignore_suffixes``); returns the names loaded.  ``post_process=False`` leaves the
    parameters in checkpoint layout (the cast to the device layout needs the GPU)."""
    ckpt = SafetensorsDirectory(model_dir)
    loader = _make_modelslim_moe_weight_loader(getattr(layer, "weight_loader", moe_weight_loader))
    pat = re.compile(re.escape(prefix) + r"\.(\d+)\.(gate_proj|up_proj|down_proj)\.(.+)$")
    params = dict(layer.named_parameters(recurse=False))
    written: set[tuple[str, int, str]] = set()
    loaded: list[str] = []
    for name in sorted(ckpt.names()):
        m = pat.match(name)
        if m is None:
            continue
        expert_id, module, suffix = int(m.group(1)), m.group(2), m.group(3)
        if suffix in ignore_suffixes:
            continue
        stacked, shard_id = _EXPERT_MODULES[module]
        param_name = target = f"{stacked}_{suffix}"
        if target not in params:
            raise KeyError(f"{name}: the {type(layer.quant_method).__name__} layer has no parameter {target!r} "
                           f"(parameters: {sorted(params)})")
        key = (target, expert_id, shard_id)
        if key in written:
            raise ValueError(f"{name}: slice {key} is written twice")
        loader(param=params[target], loaded_weight=ckpt.get(name), weight_name=f"{prefix}.{param_name}",
               shard_id=shard_id, expert_id=expert_id, return_success=True)
        written.add(key)
        loaded.append(name)
    ckpt.close()
    missing = [(p, e, s) for p, t in params.items() for e in range(t.shape[0])
               for s in (("w1", "w3") if p.startswith("w13") else ("w2",)) if (p, e, s) not in written]
    if missing:
        raise KeyError(f"{len(missing)} parameter slices of {prefix} are not in the checkpoint, first: {missing[:4]}")
    if post_process:
        layer.quant_method.process_weights_after_loading(layer)
    return loaded


def routed_experts_from_checkpoint(model_dir: str, prefix: str, moe_config, router, model_type: str = "qwen3_moe",
                                   params_dtype: torch.dtype = torch.float32, device="cuda", shared_experts=None,
                                   ignore_suffixes: tuple[str, ...] = (), **scheme_kwargs):
    """Description file -> scheme -> layer -> loaded weights, in the order the reference's model loader goes
    through (``get_quant_method`` before ``create_weights``, the weight loop, then
    ``process_weights_after_loading``)."""
    from ..fused_moe.layer import AscendRoutedExperts

    config = AscendModelSlimConfig()
    config.maybe_update_config(model_dir)
    scheme = config.get_moe_scheme(prefix, model_type, **scheme_kwargs)
    layer = AscendRoutedExperts(moe_config, scheme, router, params_dtype=params_dtype, device=device,
                                shared_experts=shared_experts)
    load_routed_experts(layer, model_dir, prefix, ignore_suffixes)
    return layer
