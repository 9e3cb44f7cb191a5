"""ctypes binding of libvig_gla.so (the C ABI declared in include/vig_gla.h).

The library is the product: if it has not been built, loading raises -- there is
no Python or CPU fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libvig_gla.so")

VIG_F32, VIG_BF16 = 0, 1
VIG_OK, VIG_EINVAL, VIG_ENOTSUP, VIG_ENOSPC, VIG_ELAUNCH = 0, -22, -95, -28, -5  # status codes of the C ABI

_c_void_p = ctypes.c_void_p
_c_int = ctypes.c_int
_c_float = ctypes.c_float
_c_size_t = ctypes.c_size_t
_c_longlong = ctypes.c_longlong

# name -> (restype, argtypes); mirrors include/vig_gla.h one to one.
_GLA_SIG = [_c_void_p] * 6 + [_c_void_p, _c_size_t] + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]
SIGNATURES = {
    "vig_gla_version": (ctypes.c_char_p, []),
    "vig_gla_strerror": (ctypes.c_char_p, [_c_int]),
    "vig_gla_bidir_fwd": (_c_int, _GLA_SIG),
    "vig_gla_bidir_fwd_exact": (_c_int, _GLA_SIG),
    "vig_gla_bidir_fwd_wide": (_c_int, _GLA_SIG),
    "vig_gla_bidir_fwd_strided": (_c_int, [_c_void_p] * 6 + [_c_int] * 5 + [_c_void_p] * 3 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_bidir_fwd_workspace": (_c_size_t, [_c_int] * 6),
    "vig_gla_bidir_fwd_noalloc": (_c_int, [_c_void_p] * 6 + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_bidir_fwd_noalloc_max_workspace": (_c_size_t, []),
    "vig_gla_causal_state_fwd": (_c_int, [_c_void_p] * 7 + [_c_void_p, _c_size_t] + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_causal_state_fwd_exact": (_c_int, [_c_void_p] * 7 + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_causal_state_fwd_workspace": (_c_size_t, [_c_int] * 7),
    "vig_gla_bidir_fwd_workspace_for": (_c_size_t, [_c_int] * 8),
    "vig_gla_bidir_bwd": (_c_int, [_c_void_p] * 11 + [_c_void_p, _c_size_t] + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_bidir_bwd_exact": (_c_int, [_c_void_p] * 11 + [_c_void_p, _c_size_t] + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_gla_bidir_bwd_workspace": (_c_size_t, [_c_int] * 6),
    "vig_gla_bidir_bwd_workspace_for": (_c_size_t, [_c_int] * 8),
    "vig_dirgate_fwd": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_dwconv3x3_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p]),
    "vig_gla_bidir_locgate_fwd": (_c_int, [_c_void_p] * 7 + [_c_int] * 7 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_locality_gate_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p]),
    "vig_dirgate_lowrank_fwd": (_c_int, [_c_void_p, _c_longlong, _c_void_p, _c_void_p, _c_void_p] + [_c_int] * 5 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_locality_blend_fwd": (_c_int, [_c_void_p] * 6 + [_c_int, _c_int, _c_int, _c_int, _c_longlong, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_layernorm_fwd": (_c_int, [_c_void_p] * 4 + [_c_longlong, _c_int, _c_float, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p]),
    "vig_rmsnorm_fwd": (_c_int, [_c_void_p] * 5 + [ctypes.c_longlong, _c_int, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_split_heads_fwd": (_c_int, [_c_void_p] * 4 + [_c_int] * 5 + [_c_longlong, _c_int, _c_void_p]),
    "vig_locality_blend_linear_fwd": (_c_int, [_c_void_p] * 7 + [_c_int] * 5 + [_c_longlong, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_linear_swiglu_fwd": (_c_int, [_c_void_p] * 3 + [_c_longlong, _c_int, _c_int, _c_int, _c_void_p]),
    "vig_patch_conv_fwd": (_c_int, [_c_void_p] * 3 + [_c_int] * 10 + [_c_void_p]),
    "vig_locality_blend_bwd_workspace": (_c_size_t, [_c_int] * 3),
    "vig_locality_blend_bwd": (_c_int, [_c_void_p] * 11 + [_c_size_t] + [_c_int] * 4 + [_c_longlong, _c_float, _c_int,
                                                                                        _c_int, _c_void_p]),
    "vig_dwconv3x3_bwd_weight_workspace": (_c_size_t, [_c_int, _c_int]),
    "vig_dwconv3x3_bwd_weight": (_c_int, [_c_void_p] * 4 + [_c_size_t] + [_c_int] * 5 + [_c_void_p]),
    "vig_dirgate_bwd": (_c_int, [_c_void_p] * 3 + [_c_int] * 4 + [_c_float, _c_float, _c_int, _c_int, _c_void_p]),
    "vig_split_heads_bwd": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p]),
    "vig_swiglu_bwd": (_c_int, [_c_void_p] * 3 + [_c_longlong, _c_int, _c_int, _c_void_p]),
    "vig_rmsnorm_bwd_workspace": (_c_size_t, [_c_longlong, _c_int]),
    "vig_rmsnorm_bwd": (_c_int, [_c_void_p] * 7 + [_c_size_t, _c_longlong, _c_int, _c_float, _c_int, _c_void_p]),
    "vig_swiglu_fwd": (_c_int, [_c_void_p, _c_void_p, ctypes.c_longlong, _c_int, _c_int, _c_void_p]),
}

_lib = None


class VigGlaError(RuntimeError):
    pass


def load():
    """Loads the shared library once and types every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise VigGlaError(
            f"{LIB_PATH} is missing: build it with `python -m vig_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().vig_gla_strerror(rc).decode()
        raise VigGlaError(f"{what} failed: {msg} (code {rc})")
