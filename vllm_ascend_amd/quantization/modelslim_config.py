"""ModelSlim checkpoint description for the MoE path: which scheme a layer gets and how its per-expert
tensors are named.

Counterpart of the parts of ``vllm_ascend/quantization/modelslim_config.py`` that the fused-MoE path touches:
``quant_model_description.json`` (one ``"<tensor name>": "<quant type>"`` entry per checkpoint tensor,
``docs/source/developer_guide/Design_Documents/quantization.md:29-47``), the lookup of a layer's quant type
over its packed shards (``modelslim_config.py:431-470``), scheme creation from the registry (``:505-541``), the
FLOAT-skip rule (``:776-808``), the config-file lookup with its error text (``:860-930``) and the name map that
sends ModelSlim's MoE scale-bias tensors down the scale path (``:55-91``).  Attention / KV-cache / linear layers
are outside this path and not handled here."""
from __future__ import annotations

import glob
import json
import os
from functools import wraps
from types import MappingProxyType
from typing import Any, Callable, Mapping

from .base import get_scheme_class

ASCEND_QUANTIZATION_METHOD = "ascend"
# The config filename that ModelSlim generates after quantizing a model.
MODELSLIM_CONFIG_FILENAME = "quant_model_description.json"

# fused module name -> checkpoint module names, per model type (modelslim_config.py:105-330; the MoE entries)
_GATE_UP_EXPERTS = {
    "gate_up_proj": ["gate_proj", "up_proj"],
    "experts": ["experts.0.gate_proj", "experts.0.up_proj", "experts.0.down_proj"],
}
packed_modules_model_mapping: dict[str, dict[str, list[str]]] = {
    "qwen3_moe": {"qkv_proj": ["q_proj", "k_proj", "v_proj"], **_GATE_UP_EXPERTS},
    "deepseek_v2": dict(_GATE_UP_EXPERTS),
    "deepseek_v3": dict(_GATE_UP_EXPERTS),
    "deepseek_v32": dict(_GATE_UP_EXPERTS),
    "kimi_k2": dict(_GATE_UP_EXPERTS),
    "glm4_moe": {"qkv_proj": ["q_proj", "k_proj", "v_proj"], **_GATE_UP_EXPERTS},
}

# ModelSlim stores the MoE scale-bias tensors under their own names; the stacked layer keeps them with the scales
_SCALE_BIAS_SUFFIX = "_scale_bias"


def _make_modelslim_moe_weight_loader(weight_loader: Callable[..., bool | None]) -> Callable[..., bool | None]:
    """Wrap a fused-MoE ``weight_loader`` so that a tensor named ``<...>.w13_scale_bias`` / ``<...>.w2_scale_bias``
    is loaded as ``<...>.w13_scale`` / ``<...>.w2_scale``; every other name passes through unchanged
    (behaviour of ``vllm_ascend/quantization/modelslim_config.py:55-91``)."""

    @wraps(weight_loader)
    def load(param, loaded_weight, weight_name: str, shard_id: str, expert_id: int, return_success: bool = False):
        leaf = weight_name.rsplit(".", 1)[-1]
        if leaf in ("w13" + _SCALE_BIAS_SUFFIX, "w2" + _SCALE_BIAS_SUFFIX):
            weight_name = weight_name[: -len("_bias")]
        return weight_loader(param=param, loaded_weight=loaded_weight, weight_name=weight_name, shard_id=shard_id,
                             expert_id=expert_id, return_success=return_success)

    return load


def _shard_keys(prefix: str, packed_modules_mapping: Mapping[str, list[str]]) -> list[str]:
    """Description keys (``<module>.weight``) that make up the layer at ``prefix``: one per checkpoint module when
    the layer's last name component is a fused module, the layer's own key otherwise."""
    fused_name = prefix.rsplit(".", 1)[-1]
    parts = packed_modules_mapping.get(fused_name)
    if parts is None:
        return [prefix + ".weight"]
    return [prefix.replace(fused_name, part) + ".weight" for part in parts]


def get_linear_quant_type(quant_description: dict[str, Any], prefix: str,
                          packed_modules_mapping: Mapping[str, list[str]]) -> str | None:
    """Quant type of a (possibly packed) layer; every shard of a packed layer must agree.  A shard that the
    description does not list raises ``KeyError``, as the reference does
    (``vllm_ascend/quantization/modelslim_config.py:431-470``)."""
    keys = _shard_keys(prefix, packed_modules_mapping)
    kinds = [quant_description[key] for key in keys]
    for key, kind in zip(keys, kinds):
        if kind != kinds[0]:
            raise ValueError(f"Not all shards of {prefix} are quantized with same quant type: {keys[0]} is "
                             f"{kinds[0]} but {key} is {kind}. Please check quantization config.")
    return kinds[0] if kinds else None


def get_quant_type_for_layer(quant_description: dict[str, Any], prefix: str, layer_type: str,
                             packed_modules_mapping: Mapping[str, list[str]] | None = None) -> str | None:
    if layer_type == "attention":
        raise NotImplementedError("attention / KV-cache quantisation is outside the fused-MoE path")
    return get_linear_quant_type(quant_description, prefix, packed_modules_mapping or {})


def create_scheme_for_layer(quant_description: dict[str, Any], prefix: str, layer_type: str,
                            packed_modules_mapping: Mapping[str, list[str]] | None = None, **scheme_kwargs):
    """Instance of the registered scheme for the layer's quant type.  ``scheme_kwargs`` stand in for what the
    reference's schemes read from the vLLM config in their constructors (dtype, EPLB, group size)."""
    quant_type = get_quant_type_for_layer(quant_description, prefix, layer_type, packed_modules_mapping)
    if quant_type is None:
        raise ValueError(f"Could not determine quantization type for layer {prefix} (layer_type={layer_type}).")
    return get_scheme_class(quant_type, layer_type)(**scheme_kwargs)


class AscendModelSlimConfig:
    """Parsed ``quant_model_description.json``."""

    def __init__(self, quant_config: dict[str, Any] | None = None):
        self.quant_description = quant_config if quant_config is not None else {}
        self.packed_modules_mapping: dict[str, list[str]] = {}

    def __repr__(self) -> str:
        return "AscendModelSlimConfig:\n" + super().__repr__()

    @classmethod
    def get_name(cls) -> str:
        return ASCEND_QUANTIZATION_METHOD

    @classmethod
    def get_config_filenames(cls) -> list[str]:
        # the file is looked up by maybe_update_config, which can say what is wrong when it is missing
        return []

    @classmethod
    def from_config(cls, config: dict[str, Any]) -> "AscendModelSlimConfig":
        return cls(config)

    def maybe_update_config(self, model_name: str) -> None:
        """Load ``quant_model_description.json`` from a local model directory unless a description is already
        present.  (The reference can also fetch it from a hub; there is no network here.)"""
        if self.quant_description:
            return
        config_path = os.path.join(model_name, MODELSLIM_CONFIG_FILENAME)
        if os.path.isdir(model_name) and os.path.exists(config_path):
            with open(config_path) as f:
                self.quant_description = json.load(f)
            return
        json_names = ([os.path.basename(f) for f in glob.glob(os.path.join(model_name, "*.json"))]
                      if os.path.isdir(model_name) else [])
        raise ValueError(
            f"ModelSlim Quantization Config Not Found: '{MODELSLIM_CONFIG_FILENAME}' is missing for model "
            f"'{model_name}'. JSON files found there: {json_names}. The checkpoint must be one that ModelSlim "
            "wrote; a float checkpoint has to be loaded without the ascend quantization method.")

    def is_layer_skipped_ascend(self, prefix: str,
                                fused_mapping: Mapping[str, list[str]] = MappingProxyType({})) -> bool:
        """True when the layer's weights are stored as FLOAT (not quantised).  A fused layer must be FLOAT in all
        of its shards or in none (``vllm_ascend/quantization/modelslim_config.py:776-808``); a plain prefix counts
        as skipped when any ``.weight`` entry below it is FLOAT."""
        if prefix.rsplit(".", 1)[-1] in fused_mapping:
            floats = [self.quant_description[key] == "FLOAT" for key in _shard_keys(prefix, fused_mapping)]
            if any(floats) != all(floats):
                raise ValueError(f"Detected some but not all shards of {prefix} are quantized. All shards of fused "
                                 "layers to have the same precision.")
            return all(floats)
        return any(kind == "FLOAT" for key, kind in self.quant_description.items()
                   if key.startswith(prefix) and key.endswith(".weight"))

    def get_moe_scheme(self, prefix: str, model_type: str = "qwen3_moe", **scheme_kwargs):
        """Scheme for the fused-MoE layer at ``prefix`` (e.g. ``model.layers.3.mlp.experts``): the MoE branch of
        ``get_quant_method`` (modelslim_config.py:752-765).  A FLOAT layer has no quantised scheme here."""
        if model_type in packed_modules_model_mapping:
            self.packed_modules_mapping = packed_modules_model_mapping[model_type]
        if self.is_layer_skipped_ascend(prefix, self.packed_modules_mapping):
            raise NotImplementedError(
                f"{prefix} is stored as FLOAT: the unquantised fused-MoE method is outside this path")
        return create_scheme_for_layer(self.quant_description, prefix, "moe", self.packed_modules_mapping,
                                       **scheme_kwargs)
