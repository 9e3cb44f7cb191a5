"""Builds vig_amd/lib/libvig_gla.so (the C-ABI HIP library) for gfx950 with hipcc.

Usage: python -m vig_amd.build   (cross-compiles without a GPU; a few seconds per file)
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libvig_gla.so")

SOURCES = ["api.hip", "gla_recurrent.hip", "gla_mfma.hip", "gla_tiles.hip", "gates.hip", "block.hip", "gla_backward.hip", "gla_backward_mfma.hip", "patch_conv.hip", "linear.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off: the compiler must not form packed fp32 VALU ops.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-option-ignored",
]


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    return obj


def build_library(extra_flags: list[str] | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    extra = list(extra_flags or [])
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


EXT = os.path.join(LIBDIR, "libvig_torch_ext.so")


def build_torch_extension(verbose: bool = True) -> str:
    """Builds vig_amd/lib/libvig_torch_ext.so: the PyTorch-ROCm operator library over the C ABI (csrc/torch_ext.cpp).
    Host code only, compiled with the host compiler against torch's headers and linked to libvig_gla.so next to it."""
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(LIBDIR, exist_ok=True)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = [f"-I{p}" for p in ce.include_paths()] + ["-I/opt/rocm/include"]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}", "-Wno-deprecated-declarations", *inc,
           os.path.join(CSRC, "torch_ext.cpp"), "-o", EXT, f"-L{LIBDIR}", "-lvig_gla", f"-L{tlib}", "-lc10", "-lc10_hip",
           "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"torch extension build failed:\n{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {EXT}")
    return EXT


if __name__ == "__main__":
    build_library(sys.argv[1:])
    build_torch_extension()
