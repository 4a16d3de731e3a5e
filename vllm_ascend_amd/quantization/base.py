"""Scheme base class and registry (``vllm_ascend/quantization/methods/base.py:206-287``,
``methods/registry.py:24-62``)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any

import torch

from ..quant_type import QuantType

_SCHEMES: dict[tuple[str, str], type] = {}


def register_scheme(quant_name: str, layer_kind: str):
    def deco(cls):
        _SCHEMES[(quant_name, layer_kind)] = cls
        return cls

    return deco


def get_scheme_class(quant_name: str, layer_kind: str) -> type:
    try:
        return _SCHEMES[(quant_name, layer_kind)]
    except KeyError:
        raise NotImplementedError(f"no MI355X scheme registered for ({quant_name!r}, {layer_kind!r})") from None


class AscendMoEScheme(ABC):
    """A MoE quantisation scheme: weight specs, post-load layout and ``apply``."""

    quant_type: QuantType = QuantType.NONE

    @abstractmethod
    def get_weight(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                   params_dtype: torch.dtype) -> dict[str, Any]: ...

    @abstractmethod
    def get_dynamic_quant_param(self, num_experts: int, intermediate_size_per_partition: int, hidden_sizes: int,
                                params_dtype: torch.dtype) -> dict[str, Any]: ...

    @abstractmethod
    def apply(self, layer: torch.nn.Module, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              shared_experts: Any | None, shared_experts_input: torch.Tensor | None): ...

    def get_eplb_weight_views(self, layer: torch.nn.Module) -> list:
        return []

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        return
