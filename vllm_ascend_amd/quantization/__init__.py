"""Quantisation schemes of the MoE layer (plugin-facing ``apply()`` contract)."""
from .base import AscendMoEScheme, get_scheme_class, register_scheme  # noqa: F401
from .w8a8_dynamic import AscendW8A8DynamicFusedMoEMethod  # noqa: F401
from .w4a8 import AscendW4A8DynamicFusedMoEMethod  # noqa: F401
