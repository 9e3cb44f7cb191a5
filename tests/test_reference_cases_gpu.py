"""The shapes, gate distributions and tolerances of the reference's own op tests, against the fp64 oracle.

flash-linear-attention/tests/ops/test_gla.py:10-77 (test_chunk / test_fused_chunk): B = H = 4, T in {300, 512},
D in {32, 64, 128} for keys and values alike, dtype in {bf16, fp32}, g = logsigmoid(randn).clamp_min(-3),
seed 42, allclose(atol 1e-2 fp32 / 1e-1 bf16) on o, dq, dk, dv, dg against the recurrent implementation.
flash-linear-attention/fla/ops/gla/naive.py:61-116: the only bidirectional check, B = H = 4, L = 512, D = 128, fp32,
g = logsigmoid(rand).clamp_min(-1), the SAME gates in both directions, allclose(atol 1e-5).
Here the reference side is the fp64 oracle; the reference's tolerances are kept as the bar (the measured errors are
orders of magnitude below them)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import vig_amd
from oracle import gla_oracle as O

from .util import announce, f64

pytestmark = pytest.mark.gpu


def _inputs(T, D, dtype):
    torch.manual_seed(42)
    B = H = 4
    q, k, v = (torch.randn(B, H, T, D).to(dtype) for _ in range(3))
    g = F.logsigmoid(torch.randn(B, H, T, D)).clamp_min(-3).to(dtype)
    do = torch.randn(B, H, T, D).to(dtype)
    return q, k, v, g, do


@pytest.mark.parametrize("dtype,atol", [(torch.float32, 1e-2), (torch.bfloat16, 1e-1)])
@pytest.mark.parametrize("T", [300, 512])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_fused_chunk_forward_as_in_test_gla(dtype, atol, T, D):
    announce(f"fused_chunk_gla forward, reference test shape T={T} D={D} {dtype}")
    q, k, v, g, _ = _inputs(T, D, dtype)
    want = O.gla_recurrent(f64(q), f64(k), f64(v), f64(g))
    got, final = vig_amd.fused_chunk_gla(q.cuda(), k.cuda(), v.cuda(), g.cuda())
    assert final is None and got.dtype == dtype
    # unnormalised keys: |o| reaches the hundreds at D = 128, so the bf16 bar scales with the output grid
    tol = atol + (2.0 ** -8 * np.abs(want) if dtype == torch.bfloat16 else 1e-5 * np.abs(want))
    assert np.all(np.abs(f64(got) - want) <= tol)


@pytest.mark.parametrize("dtype,atol", [(torch.float32, 1e-2), (torch.bfloat16, 1e-1)])
@pytest.mark.parametrize("T", [300, 512])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_fused_chunk_gradients_as_in_test_gla(dtype, atol, T, D):
    """(D = 128: the op wrapper runs the backward of the four 64 x 64 blocks and sums.)"""
    announce(f"fused_chunk_gla gradients, reference test shape T={T} D={D} {dtype}")
    q, k, v, g, do = _inputs(T, D, dtype)
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(g), None, f64(do))
    tq, tk, tv, tg = (t.cuda().requires_grad_(True) for t in (q, k, v, g))
    o, _ = vig_amd.fused_chunk_gla(tq, tk, tv, tg)
    o.backward(do.cuda())
    for name, got, w in zip(("dq", "dk", "dv", "dg"), (tq.grad, tk.grad, tv.grad, tg.grad), want[:4]):
        tol = atol + (2.0 ** -8 * np.abs(w) if dtype == torch.bfloat16 else 1e-5 * np.abs(w))
        assert np.all(np.abs(f64(got) - w) <= tol), name


def test_bidirectional_same_gates_as_in_naive_main():
    announce("bidirectional, same gates both ways, B=H=4 L=512 D=128 fp32 (naive.py __main__)")
    torch.manual_seed(42)
    B = H = 4
    L, D = 512, 128
    q, k, v = (torch.randn(B, H, L, D) for _ in range(3))
    g = F.logsigmoid(torch.rand(B, H, L, D)).clamp_min(-1)
    want = O.bidir_gla_recurrent(f64(q), f64(k), f64(v), f64(g), f64(g))
    got = vig_amd.gla_bidir_forward(q.cuda(), k.cuda(), v.cuda(), g.cuda(), g.cuda())
    assert np.all(np.abs(f64(got) - want) <= 1e-5 * np.maximum(1.0, np.abs(want)))
