"""MI355X-native W8A8-dynamic fused-MoE layer behind vllm-ascend's plugin interface.

Only the routed-experts hot path is here: gating top-k, token dispatch with
fused per-token int8 quantisation, the two int8 grouped GEMMs with their fused
epilogues, and the weighted combine -- hand-written HIP kernels for gfx950
reached through the C ABI of ``libmoe355.so``.
"""

__version__ = "0.1.0"
