"""Loader of the PyTorch-ROCm operator library (vig_amd/lib/libvig_torch_ext.so, built from csrc/torch_ext.cpp).

The operators (torch.ops.vig_amd.*) are the same C-ABI entry points as the ctypes binding reaches, with the argument
checks, output allocation and stream lookup done in C++: one dispatcher call instead of a few dozen Python
statements per kernel.  The ctypes binding stays the torch-free way in; VIG_AMD_NO_EXT=1 keeps this package on it.
"""
from __future__ import annotations

import os

_HERE = os.path.dirname(os.path.abspath(__file__))
EXT_PATH = os.path.join(_HERE, "lib", "libvig_torch_ext.so")

_ops = None
_tried = False
_error = None


def load():
    """torch.ops.vig_amd, or None when the operator library is not built, fails to load or is switched off."""
    global _ops, _tried, _error
    if _tried:
        return _ops
    _tried = True
    if os.environ.get("VIG_AMD_NO_EXT") == "1":
        _error = "switched off by VIG_AMD_NO_EXT=1"
        return None
    if not os.path.exists(EXT_PATH):
        _error = f"{EXT_PATH} is not built (python -m vig_amd.build)"
        return None
    try:
        import torch

        torch.ops.load_library(EXT_PATH)
        _ops = torch.ops.vig_amd
    except Exception as e:  # an operator library built against another torch: the ctypes binding still works
        _error = f"{type(e).__name__}: {e}"
        _ops = None
        import warnings

        warnings.warn(f"vig_amd: {EXT_PATH} exists but did not load ({_error}); falling back to the ctypes binding, "
                      "which costs about twice the host time per call. Rebuild it with `python -m vig_amd.build`.",
                      RuntimeWarning, stacklevel=2)
    return _ops


def why_not() -> str | None:
    """Why load() returned None (for diagnostics), or None if it did not."""
    load()
    return _error
