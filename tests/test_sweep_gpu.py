"""Seeded random sweep over shapes, directions and gate strengths: the forward against the fp64 oracle, the strided
entry point against the contiguous one (bit for bit), the matrix-core backward against the fp32-arithmetic backward.
Shapes straddle the kernels' tile (32), chunk (64) and slab (256) boundaries."""
import random

import numpy as np
import pytest
import torch

import vig_amd
from vig_amd import ops
from vig_amd.synthetic import make_gla_inputs

from .util import announce, f64, oracle_bidir

pytestmark = pytest.mark.gpu

_LENGTHS = [1, 7, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 196, 255, 256, 257, 300, 513]


def _cases(seed, n):
    rng = random.Random(seed)
    return [(rng.choice([32, 64]), rng.choice([1, 2, 3, 6]), rng.choice([1, 2, 3, 5]), rng.choice(_LENGTHS),
             rng.random() < 0.8, rng.choice([1.0 / 16, 1.0 / 16, 0.25, 1.0]), 8 * rng.randint(0, 4)) for _ in range(n)]


@pytest.mark.parametrize("i,case", list(enumerate(_cases(7, 24))))
def test_random_shapes(i, case):
    Dk, H, B, L, both, gate_scale, extra = case
    announce(f"sweep {i}: B={B} H={H} L={L} Dk={Dk} both={both} gates x{gate_scale * 16:g}")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, Dk, 64, seed=2000 + i)
    q, k, v, gf, gb = (t.bfloat16().cuda() for t in (q, k, v, gf * (gate_scale * 16), gb * (gate_scale * 16)))
    if not both:
        gb = None
    want = oracle_bidir(q, k, v, gf, gb)
    o = vig_amd.gla_bidir_forward(q, k, v, gf, gb)
    # (half an output ulp on top of the absolute tolerance: |o| grows with the sequence length)
    assert np.all(np.abs(f64(o) - want) <= 2e-2 + 2.0 ** -8 * np.abs(want))
    if L <= 256:  # q, k, v as column blocks of one wider matrix, read in place
        row = H * (2 * Dk + 64) + extra
        z = torch.randn(B, L, row, device="cuda").bfloat16()
        z[..., :H * Dk] = q.transpose(1, 2).reshape(B, L, H * Dk)
        z[..., H * Dk:2 * H * Dk] = k.transpose(1, 2).reshape(B, L, H * Dk)
        z[..., 2 * H * Dk:2 * H * Dk + H * 64] = v.transpose(1, 2).reshape(B, L, H * 64)
        qs, ks, vs = (t.unflatten(-1, (H, d)).transpose(1, 2)
                      for t, d in zip(z[..., :H * (2 * Dk + 64)].split((H * Dk, H * Dk, H * 64), -1), (Dk, Dk, 64)))
        assert torch.equal(vig_amd.gla_bidir_forward(qs, ks, vs, gf, gb), o)
    d_o = torch.randn_like(v)
    fast = ops.gla_bidir_backward(q, k, v, gf, gb, d_o)
    exact = ops.gla_bidir_backward(q, k, v, gf, gb, d_o, exact=True)
    for name, a, b in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), fast, exact):
        if a is None:
            continue
        scale = float(b.float().abs().max()) + 1e-6
        if name.startswith("dg"):
            # q dq - k dk is a difference of products (exactly zero for a single token): its error scales with the
            # products, not with their difference
            scale = max(scale, float((q.float() * exact[0].float()).abs().max()),
                        float((k.float() * exact[1].float()).abs().max()))
        err = float((a.float() - b.float()).abs().max()) / scale
        assert err <= 2e-2, (name, err)
