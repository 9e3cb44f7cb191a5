"""The C-ABI library loads and exports every symbol include/vig_gla.h declares (no GPU)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "vig_gla.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vig_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    syms = _declared_symbols()
    for s in ("vig_gla_bidir_fwd", "vig_gla_bidir_fwd_workspace", "vig_dirgate_fwd", "vig_locality_gate_fwd"):
        assert s in syms


def test_library_exports_every_declared_symbol():
    from vig_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here (python -m vig_amd.build)")
    lib = _lib.load()
    for s in _declared_symbols():
        assert hasattr(lib, s), f"{s} declared in vig_gla.h but not exported"
        assert s in _lib.SIGNATURES, f"{s} has no ctypes signature"
    assert b"gfx950" in lib.vig_gla_version()


def test_argument_validation_without_gpu():
    """Bad arguments are rejected before anything touches a device."""
    from vig_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here")
    lib = _lib.load()
    rc = lib.vig_gla_bidir_fwd(None, None, None, None, None, None, None, 0, 1, 1, 1, 64, 64, 1.0, 1.0, 0, 0, None)
    assert rc == -22
    one = 1 << 20  # non-null dummy addresses; the call must fail on shape before any launch
    rc = lib.vig_gla_bidir_fwd(one, one, one, one, one, one, None, 0, 1, 1, 8, 48, 64, 1.0, 1.0, 0, 0, None)
    assert rc == -95
    rc = lib.vig_gla_bidir_fwd(one, one, one, one, one, one, None, 0, 0, 1, 8, 64, 64, 1.0, 1.0, 0, 0, None)
    assert rc == -22
    rc = lib.vig_gla_bidir_fwd_exact(one, one, one, one, one, one, None, 0, 1, 1, 8, 64, 64, 1.0, 1.0, 1, 1, None)
    assert rc == -28  # bf16 bidirectional exact path needs workspace
    assert lib.vig_gla_strerror(-28) == b"workspace too small"
    assert lib.vig_dirgate_fwd(one, one, 1, 1, 1, 12, 1.0, 0.0, 0, 0, None) == -95
    # launch geometry is checked before anything is enqueued: B*H beyond int range, row counts beyond int range, and
    # more (sequence, direction) pairs than the long-sequence scan's grid takes
    assert lib.vig_gla_bidir_fwd(one, one, one, one, one, one, one, 1 << 40, 40000, 2, 300, 64, 64, 1.0, 1.0, 1, 1,
                                 None) == -95
    # one direction: 40000 pairs fit the grid, so the call gets as far as the workspace check, which refuses it (no
    # workspace is offered: a call on dummy addresses must never reach a launch)
    assert lib.vig_gla_bidir_fwd(one, one, one, one, None, one, None, 0, 40000, 1, 300, 64, 64, 1.0, 1.0, 1, 1,
                                 None) == -28
    big = 1 << 40
    assert lib.vig_gla_bidir_bwd(one, one, one, one, one, one, one, one, one, one, one, one, big, 70000, 70000, 8, 64,
                                 64, 1.0, 1.0, 1, 1, None) == -22
    assert lib.vig_rmsnorm_bwd(one, one, one, None, one, None, None, 0, 1 << 31, 384, 1e-6, 1, None) == -22
    assert lib.vig_gla_bidir_fwd_workspace_for(128, 6, 196, 64, 64, 1, 1, 1) == 0
    assert lib.vig_gla_bidir_fwd_workspace_for(128, 6, 196, 64, 64, 1, 0, 1) == 128 * 6 * 196 * 64 * 4
    assert lib.vig_gla_bidir_fwd_workspace_for(2, 3, 197, 64, 64, 1, 0, 0) == 0


def test_ops_refuse_cpu_tensors():
    import torch

    import vig_amd
    from vig_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here")
    q = torch.zeros(1, 1, 4, 64)
    with pytest.raises(_lib.VigGlaError):
        vig_amd.gla_bidir_forward(q, q, q, q, q)


def test_reference_signatures():
    """Positional order and defaults of the mirrored ops (chunk_fuse.py:554-596, recurrent_fuse.py:659-669)."""
    import inspect

    import vig_amd

    p = list(inspect.signature(vig_amd.fused_chunk_gla).parameters)
    assert p == ["q", "k", "v", "g", "scale", "initial_state", "output_final_state"]
    p = list(inspect.signature(vig_amd.batch_bid_fused_chunk_gla).parameters)
    assert p == ["q", "k", "v", "g", "scale", "initial_state", "output_final_state"]
    sig = inspect.signature(vig_amd.bid_fused_recurrent_gla)
    assert list(sig.parameters) == ["q", "k", "v", "gk", "gv", "scale", "initial_state", "output_final_state", "causal"]
    assert sig.parameters["scale"].default == -1 and sig.parameters["causal"].default is True
