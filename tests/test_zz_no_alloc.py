"""vig_gla_bidir_fwd_noalloc (the entry point that allocates nothing: its workspace is a device array of the
library) against vig_gla_bidir_fwd with a caller workspace, through the C ABI, bit for bit: two calls in a row, the
second with a smaller input, on the paths that use a workspace (segment states of long sequences, the zero-padded
HierViG head shape, the token-recurrent kernel's parked sums) and on one that uses none."""
import ctypes

import numpy as np
import pytest
import torch

from tests.util import announce, oracle_bidir, max_abs
from vig_amd import _lib
from vig_amd.synthetic import make_gla_inputs

pytestmark = pytest.mark.gpu


def _call(lib, name, t, o, dims, ws=None):
    q, k, v, gf, gb = t
    B, H, L, Dk, Dv = dims
    io = _lib.VIG_BF16 if q.dtype == torch.bfloat16 else _lib.VIG_F32
    gd = _lib.VIG_BF16 if gf.dtype == torch.bfloat16 else _lib.VIG_F32
    st = torch.cuda.current_stream().cuda_stream
    ptrs = [x.data_ptr() for x in (q, k, v, gf)] + [gb.data_ptr() if gb is not None else None, o.data_ptr()]
    tail = [B, H, L, Dk, Dv, Dk ** -0.5, 1.0, io, gd, st]
    if name == "vig_gla_bidir_fwd":
        nbytes = ws.numel() if ws is not None else 0
        return lib.vig_gla_bidir_fwd(*ptrs, ws.data_ptr() if ws is not None else None, nbytes, *tail)
    return lib.vig_gla_bidir_fwd_noalloc(*ptrs, *tail)


def _pair(lib, B, H, L, Dk, Dv, dtype, seed, bidir=True):
    dev = torch.device("cuda:0")
    t = [x.to(dev) for x in make_gla_inputs(B, H, L, Dk, Dv, seed=seed, dtype=dtype)]
    if not bidir:
        t[4] = None
    dims = (B, H, L, Dk, Dv)
    io = _lib.VIG_BF16 if dtype == torch.bfloat16 else _lib.VIG_F32
    need = lib.vig_gla_bidir_fwd_workspace_for(B, H, L, Dk, Dv, io, io, int(bidir))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev) if need else None
    want = torch.full((B, H, L, Dv), float("nan"), dtype=dtype, device=dev)
    got = torch.full((B, H, L, Dv), float("nan"), dtype=dtype, device=dev)
    announce(f"noalloc pair B{B} H{H} L{L} Dk{Dk} Dv{Dv} {dtype} bidir={bidir} need={need}")
    rc = _call(lib, "vig_gla_bidir_fwd", t, want, dims, ws)
    assert rc == 0, rc
    rc = _call(lib, "vig_gla_bidir_fwd_noalloc", t, got, dims)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    return t, got, need


def test_noalloc_matches_workspace_entry_point_two_calls_in_a_row():
    lib = _lib.load()
    assert lib.vig_gla_bidir_fwd_noalloc_max_workspace() == 16 << 20
    # long sequences (segment states in the scratch array), the second call smaller than the first
    t, got, need = _pair(lib, 2, 3, 1000, 64, 64, torch.bfloat16, seed=11)
    assert need > 0
    err = max_abs(got.double().cpu().numpy(), oracle_bidir(*t))
    assert err <= 2e-2, err
    t, got, need2 = _pair(lib, 1, 2, 300, 64, 64, torch.bfloat16, seed=12)
    assert 0 < need2 < need
    err = max_abs(got.double().cpu().numpy(), oracle_bidir(*t))
    assert err <= 2e-2, err
    # Dk = 32, one direction only, then back to a larger one
    _pair(lib, 1, 2, 700, 32, 64, torch.bfloat16, seed=13, bidir=False)
    _pair(lib, 3, 2, 1500, 32, 64, torch.bfloat16, seed=14)
    # the zero-padded head shape and the token-recurrent kernel use the array too
    _pair(lib, 2, 3, 196, 16, 32, torch.bfloat16, seed=15)
    _pair(lib, 1, 2, 130, 16, 32, torch.bfloat16, seed=16)
    _pair(lib, 2, 2, 197, 64, 128, torch.bfloat16, seed=17)
    _pair(lib, 1, 1, 50, 64, 128, torch.bfloat16, seed=18)
    # no workspace at all: whole-sequence slabs, fp32 tensors
    t, got, need = _pair(lib, 4, 6, 196, 64, 64, torch.bfloat16, seed=19)
    assert need == 0
    _pair(lib, 2, 3, 197, 64, 64, torch.float32, seed=20)


def test_noalloc_refuses_shapes_beyond_its_array():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    x = torch.zeros(16, dtype=torch.bfloat16, device=dev)  # never read: the call must fail before any launch
    p = x.data_ptr()
    B, H, L = 64, 8, 4096  # 8192 segments x 2 directions x 16.25 KiB of states
    assert lib.vig_gla_bidir_fwd_workspace_for(B, H, L, 64, 64, 1, 1, 1) > 16 << 20
    rc = lib.vig_gla_bidir_fwd_noalloc(p, p, p, p, p, p, B, H, L, 64, 64, 0.125, 1.0, 1, 1, None)
    assert rc == _lib.VIG_ENOSPC
    assert lib.vig_gla_bidir_fwd_noalloc(p, p, p, p, p, p, 0, 1, 1, 64, 64, 0.125, 1.0, 1, 1, None) == _lib.VIG_EINVAL
    torch.cuda.synchronize()


def test_noalloc_allocates_nothing_and_replays_from_a_graph():
    """After one warm-up call per device (kernel attributes, the array's address) the entry point neither allocates
    device memory (free memory as the driver reports it stays put over repeated calls) nor does anything a HIP graph
    capture refuses: a captured call on a long sequence, replayed with eager calls in between, reproduces the eager
    output bit for bit."""
    lib = _lib.load()
    dev = torch.device("cuda:0")
    B, H, L, Dk, Dv = 2, 3, 1000, 64, 64
    announce("noalloc: no device allocation, graph capture and replays")
    t = [x.to(dev) for x in make_gla_inputs(B, H, L, Dk, Dv, seed=31, dtype=torch.bfloat16)]
    dims = (B, H, L, Dk, Dv)
    eager = torch.empty(B, H, L, Dv, dtype=torch.bfloat16, device=dev)
    got = torch.full_like(eager, float("nan"))
    assert _call(lib, "vig_gla_bidir_fwd_noalloc", t, eager, dims) == 0  # warm-up, outside any capture
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info(dev)[0]
    for _ in range(3):
        assert _call(lib, "vig_gla_bidir_fwd_noalloc", t, eager, dims) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = _call(lib, "vig_gla_bidir_fwd_noalloc", t, got, dims)
    assert rc == 0
    other = [x.to(dev) for x in make_gla_inputs(1, 2, 300, Dk, Dv, seed=32, dtype=torch.bfloat16)]
    scratch_out = torch.empty(1, 2, 300, Dv, dtype=torch.bfloat16, device=dev)
    for i in range(3):
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16)), f"replay {i}"
        # eager work on the same array between the replays
        assert _call(lib, "vig_gla_bidir_fwd_noalloc", other, scratch_out, (1, 2, 300, Dk, Dv)) == 0
        torch.cuda.synchronize()
