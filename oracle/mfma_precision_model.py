"""CPU emulation of the bf16 MFMA kernel's arithmetic (which operands are rounded where).

TEST INFRASTRUCTURE ONLY.  It rebuilds the end-anchored chunk algebra of vig_amd/csrc/gla_mfma.hip in numpy with
explicit bf16 roundings, so the precision design (which operands carry a bf16 hi + lo pair) can be checked on the
CPU against the fp64 oracle.  Chunk algebra as in flash-linear-attention/fla/ops/gla/chunk_util.py:9-78 and
chunk_fuse.py:76-97 with the anchor moved to the chunk end.

splits:  qk = number of score terms (1: hi*hi, 3: + lo*hi + hi*lo),  p = P terms in P V (1 or 2),
         iq = q~ terms in the inter-chunk product, st = state terms, u = k~ terms in the state update.
The shipped kernel is qk=3, p=2, iq=1, st=1, u=1.
"""
from __future__ import annotations

import numpy as np


def bf16_round(x):
    """fp32 array rounded to bf16 (round to nearest even), returned as fp32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) & 0xFFFF0000).astype(np.uint32).view(np.float32)


def _split(x):
    hi = bf16_round(x)
    return hi, bf16_round(x - hi)


def _mm(a, b):
    return np.matmul(a.astype(np.float32), b.astype(np.float32))


SHIPPED = dict(qk=3, p=2, iq=1, st=1, u=1)
PLAIN = dict(qk=1, p=1, iq=1, st=1, u=1)


def emulate(q, k, v, gf, gb, chunk, splits=SHIPPED):
    """q, k, gf, gb [N, L, Dk], v [N, L, Dv] (bf16-representable fp32).  Returns fp32 o [N, L, Dv] before the
    final bf16 store, scale Dk^-0.5, directions summed."""
    N, L, Dk = q.shape
    Dv = v.shape[-1]
    s = np.float32(Dk ** -0.5)
    nchunk = -(-L // chunk)
    o = np.zeros((N, L, Dv), np.float32)
    T = lambda x: x.transpose(0, 2, 1)
    for direction in (0, 1):
        g = gf if direction == 0 else gb
        S = np.zeros((N, Dk, Dv), np.float32)
        order = range(nchunk) if direction == 0 else range(nchunk - 1, -1, -1)
        for c in order:
            sl = slice(c * chunk, min(L, (c + 1) * chunk))
            gc = g[:, sl].astype(np.float32)
            if direction == 0:
                G = np.cumsum(gc, axis=1, dtype=np.float32)
                Gend = G[:, -1:, :]
            else:
                G = np.flip(np.cumsum(np.flip(gc, 1), axis=1, dtype=np.float32), 1)
                Gend = G[:, :1, :]
            qt = q[:, sl] * np.exp(G - Gend).astype(np.float32)
            kt = k[:, sl] * np.exp(Gend - G).astype(np.float32)
            vc = v[:, sl]
            n = qt.shape[1]
            tri = np.tril(np.ones((n, n), np.float32)) if direction == 0 else np.triu(np.ones((n, n), np.float32))
            qh, ql = _split(qt)
            kh, kl = _split(kt)
            P = _mm(qh, T(kh))
            if splits["qk"] >= 3:
                P += _mm(ql, T(kh)) + _mm(qh, T(kl))
            P *= tri
            Ph, Pl = _split(P)
            oc = _mm(Ph, vc)
            if splits["p"] >= 2:
                oc += _mm(Pl, vc)
            Sd = S * T(np.exp(Gend).astype(np.float32))
            Sh, Sl = _split(Sd)
            oc += _mm(qh, Sh)
            if splits["iq"] >= 2:
                oc += _mm(ql, Sh)
            if splits["st"] >= 2:
                oc += _mm(qh, Sl)
            o[:, sl] += s * oc
            S = Sd + _mm(T(kh), vc)
            if splits["u"] >= 2:
                S += _mm(T(kl), vc)
    return o
