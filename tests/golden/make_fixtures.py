"""Writes the small input/output vectors under tests/golden/ from the fp64 oracle.

The reference holds no golden vectors for this path and cannot be imported here, so these
fixtures freeze the oracle's own answers (the oracle itself is pinned by closed forms in
tests/test_oracle.py): a later change of the oracle, of the synthetic input generator or of a
kernel shows up against data that does not move.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import gla_oracle as O  # noqa: E402
from vig_amd.synthetic import make_gla_inputs, make_locality_weight  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def _randn(shape, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).double().numpy()


def main():
    # bidirectional GLA, fp32 inputs, ragged length, two head sizes
    for name, (B, H, L, Dk, Dv, seed) in {"gla_f32_L37_D16_32": (1, 2, 37, 16, 32, 11),
                                          "gla_f32_L70_D64_64": (1, 1, 70, 64, 64, 12)}.items():
        q, k, v, gf, gb = (t.double().numpy() for t in make_gla_inputs(B, H, L, Dk, Dv, seed))
        o = O.bidir_gla_recurrent(q, k, v, gf, gb, out_scale=0.5)
        o_causal = O.gla_recurrent(q, k, v, gf)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q.astype(np.float32), k=k.astype(np.float32),
                            v=v.astype(np.float32), gf=gf.astype(np.float32), gb=gb.astype(np.float32),
                            o_bidir_half=o, o_causal=o_causal)
    # bf16-representable inputs at the ViG-S head shape (Dk 32, Dv 64), one slab of 14x14 tokens
    q, k, v, gf, gb = (t.double().numpy() for t in make_gla_inputs(1, 2, 196, 32, 64, 13, torch.bfloat16))
    np.savez_compressed(os.path.join(HERE, "gla_bf16_L196_D32_64.npz"), q=q.astype(np.float32), k=k.astype(np.float32),
                        v=v.astype(np.float32), gf=gf.astype(np.float32), gb=gb.astype(np.float32),
                        o_bidir_quarter=O.bidir_gla_recurrent(q, k, v, gf, gb, out_scale=0.25))
    # neighbours of the op on a 5x4 token grid
    B, hw, H, Dk, Dv = 2, (5, 4), 2, 16, 32
    L, C = hw[0] * hw[1], H * Dv
    gk_lin = _randn((B, L, 2 * H * Dk), 21, 3.0)
    x = _randn((B, L, C), 22)
    w = make_locality_weight(C, 23).double().numpy()
    bias = _randn((C,), 24, 0.1)
    o = _randn((B, H, L, Dv), 25)
    glin = _randn((B, L, C), 26)
    wg, wl = 1.0 + _randn((Dv,), 27, 0.1), 1.0 + _randn((Dv,), 28, 0.1)
    res = _randn((B, L, C), 29, 2.0)
    wn = 1.0 + _randn((C,), 30, 0.1)
    gu = _randn((B, L, 2 * 24), 31, 2.0)
    np.savez_compressed(
        os.path.join(HERE, "neighbours_grid5x4.npz"),
        gk_lin=gk_lin, dirgate=O.dirgate_reference(gk_lin, H, 16.0), dirgate_clamped=O.dirgate_reference(gk_lin, H, 16.0, clamp_min=-0.03),
        x=x, conv_w=w, conv_b=bias, dwconv_silu=O.dwconv3x3_reference(x, w, hw, bias=bias, silu=True),
        o=o, locality_gate=O.locality_sigmoid_gate_reference(o, w, hw),
        glin=glin, w_g=wg, w_l=wl, blend=O.locality_blend_reference(o, x, glin, wg, wl, eps=1e-6, silu_out=False),
        residual=res, w_norm=wn, rmsnorm_y=O.rmsnorm_residual_reference(x, wn, 1e-6, residual=res)[0],
        gate_up=gu, swiglu=O.swiglu_reference(gu))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
