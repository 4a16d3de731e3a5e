"""ctypes binding of ``libmoe355.so`` (the C ABI declared in ``include/moe355.h``).

There is no fallback: if the library is missing, or an entry point rejects its
arguments, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libmoe355.so")

DT_F32, DT_BF16, DT_F16 = 0, 1, 2
W_ENK, W_EKN = 0, 1
GL_CUMSUM, GL_COUNT = 0, 1

ABI_VERSION = 1

# name -> (restype, argtypes); mirrors include/moe355.h one to one
PROTOTYPES = {
    "moe355_abi_version": (c_int, []),
    "moe355_strerror": (c_char_p, [c_int]),
    "moe355_dynamic_quant": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "moe355_dynamic_quant_form": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p]),
    "moe355_router_gate_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "moe355_router_gate": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p,
                                   c_size_t, c_void_p]),
    "moe355_gating_top_k": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                    c_void_p]),
    "moe355_init_routing_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "moe355_init_routing": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe355_init_routing_prequant": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int, c_int, c_int,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe355_route_map": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_size_t, c_void_p]),
    "moe355_init_routing_static": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int, c_int, c_int,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe355_route_quant_small_supported": (c_int, [c_int64, c_int, c_int]),
    "moe355_gate_quant_supported": (c_int, [c_int64, c_int, c_int]),
    "moe355_gate_quant": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int, c_int, c_int,
                                  c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p]),
    "moe355_route_quant_small": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int, c_int,
                                         c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p]),
    "moe355_gmm1_swiglu_quant_gather": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                c_int64, c_int64, c_int64, c_int, c_float, c_void_p, c_void_p,
                                                c_void_p, c_size_t, c_void_p]),
    "moe355_format_cast_nz": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "moe355_format_cast_nz_int4": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "moe355_w4_offset_correction": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "moe355_gmm1_swiglu_quant_w4": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                            c_int64, c_int64, c_int64, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                            c_size_t, c_void_p]),
    "moe355_gmm1_swiglu_quant_w4_gather": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                                   c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_float,
                                                   c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe355_gmm2_dequant_w4": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                       c_int64, c_int64, c_int64, c_int, c_void_p, c_int, c_void_p]),
    "moe355_gmm1_swiglu_quant_workspace": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "moe355_gmm1_swiglu_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                         c_int64, c_int, c_float, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe355_gmm1_swiglu_quant_list": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                              c_int64, c_int, c_float, c_void_p, c_void_p, c_void_p, c_size_t,
                                              c_void_p]),
    "moe355_gmm2_dequant_list": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                         c_int64, c_int, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "moe355_gmm2_dequant_workspace": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "moe355_gmm2_dequant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64,
                                    c_int, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "moe355_gmm_i32_workspace": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "moe355_gmm_i32": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p,
                               c_void_p, c_size_t, c_void_p]),
    "moe355_dequant_swiglu_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_float, c_void_p,
                                            c_void_p, c_void_p]),
    "moe355_dequant_swiglu_quant_grouped": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                                     c_int64, c_int64, c_int, c_int, c_float, c_float, c_float, c_int,
                                                     c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe355_dequant_swiglu_quant_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
                                                   c_int64, c_int, c_float, c_void_p, c_void_p]),
    "moe355_act_mul_quant": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int64, c_int64, c_int, c_float,
                                     c_float, c_float, c_void_p, c_void_p, c_void_p]),
    "moe355_silu_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "moe355_gmm_pairs_supported": (c_int, [c_int64, c_int, c_int64, c_int64]),
    "moe355_gmm1_swiglu_quant_pairs_workspace": (c_size_t, [c_int64, c_int, c_int64]),
    "moe355_gmm1_swiglu_quant_pairs": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int64,
                                               c_int64, c_int, c_float, c_void_p, c_void_p, c_void_p, c_size_t,
                                               c_void_p]),
    "moe355_gmm2_dequant_pairs": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                                          c_int64, c_int, c_void_p, c_int, c_void_p]),
    "moe355_gmm1_swiglu_pairs": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int64, c_int64,
                                         c_int, c_float, c_void_p, c_void_p]),
    "moe355_gmm2_requant_pairs_supported": (c_int, [c_int64, c_int, c_int64, c_int64, c_int]),
    "moe355_gmm2_requant_dequant_pairs": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                                                  c_int64, c_int, c_void_p, c_int, c_void_p]),
    "moe355_token_unpermute_pairs": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int,
                                             c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe355_profile_next_gemm": (c_int, [c_void_p, c_void_p]),
    "moe355_gmm_kernel_name": (c_char_p, [c_int, c_int64, c_int64, c_int64, c_int]),
    "moe355_token_unpermute": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_void_p,
                                       c_void_p, c_void_p]),
}

_lib = None


class Moe355Error(RuntimeError):
    """An entry point of libmoe355.so refused its arguments or the launch failed."""


def load() -> ctypes.CDLL:
    """Load the library once.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'` or `python -m vllm_ascend_amd._build`). "
            "There is no CPU or PyTorch fallback for this path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.moe355_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"libmoe355.so has ABI version {got}, this package expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().moe355_strerror(rc).decode()
        raise Moe355Error(f"{what}: {msg} (code {rc})")
