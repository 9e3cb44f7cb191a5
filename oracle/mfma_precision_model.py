"""CPU emulation of the MFMA kernels' arithmetic (which operands are rounded where).

TEST INFRASTRUCTURE ONLY.  `emulate_tiles` rebuilds the tile-pair algebra of vig_amd/csrc/gla_tiles.hip (the forward
that ships: 32-token tiles, q^ = q exp(G), k^ = k exp(T - G), k' = k exp(-G), D = exp(T), everything the matrix cores
see rounded to fp16), `emulate` the chunk algebra of vig_amd/csrc/gla_mfma.hip, in numpy with explicit
roundings, so the precision design (which operands are fp16, which carry a bf16 hi + lo pair) can be checked on the
CPU against the fp64 oracle.  Chunk algebra as in flash-linear-attention/fla/ops/gla/chunk_util.py:9-78 and
chunk_fuse.py:76-97, here with the anchor at half the chunk total: q~ = q*exp(G - G_end/2), k~ = k*exp(G_end/2 - G),
so state update and inter-chunk product carry exp(G_end/2) each.

splits:  qk = score operands: "f16" (one fp16 rounding each), 1 (bf16 hi*hi) or 3 (+ lo*hi + hi*lo),
         p = P terms in P V: "f16" (P rounded once to fp16; V is exact in fp16), 1 or 2 (bf16 hi, hi + lo),
         iq = q~ terms in the inter-chunk product, st = state terms, or st = "direct": no chained state, every earlier
         chunk j of the direction adds f16(q~) @ f16(E * f16(U_j)) with U_j = k~^T V of that chunk and the per-channel
         factor E = h_c h_j prod(h_i^2, i between), h = exp(G_end/2) in fp16, every product rounded to fp16,
         u = k~ in the state update: "f16" (the score operand again), 1 or 2 bf16 terms.
The shipped kernel is qk="f16", p="f16", st="direct", u="f16" for whole slabs (SHIPPED) and qk="f16", p="f16", iq=1,
st=1, u="f16" for the chained segments of long sequences (SHIPPED_SEGMENTS); for chunks whose gate total or operand
magnitudes leave the fp16 range it falls back to qk=3, p=2, iq=1, st=1, u=1 (FALLBACK).
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


def f16_round(x):
    """fp32 array rounded to fp16 (round to nearest even), returned as fp32."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


SHIPPED = dict(qk="f16", p="f16", iq=1, st="direct", u="f16")
SHIPPED_SEGMENTS = dict(qk="f16", p="f16", iq=1, st=1, u="f16")
FALLBACK = dict(qk=3, p=2, iq=1, st=1, u=1)
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
        earlier = []  # (st == "direct") fp16 contribution and fp16 half decay of every chunk walked so far, nearest first
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
            half = np.float32(0.5) * Gend
            qt = q[:, sl] * np.exp(G - half).astype(np.float32)
            kt = k[:, sl] * np.exp(half - G).astype(np.float32)
            vc = v[:, sl]
            n = qt.shape[1]
            tri = np.tril(np.ones((n, n), np.float32)) if direction == 0 else np.triu(np.ones((n, n), np.float32))
            qh, ql = _split(qt)
            kh, kl = _split(kt)
            if splits["qk"] == "f16":
                P = _mm(f16_round(qt), T(f16_round(kt)))
            else:
                P = _mm(qh, T(kh))
                if splits["qk"] >= 3:
                    P += _mm(ql, T(kh)) + _mm(qh, T(kl))
            P *= tri
            if splits["p"] == "f16":
                oc = _mm(f16_round(P), vc)
            else:
                Ph, Pl = _split(P)
                oc = _mm(Ph, vc)
                if splits["p"] >= 2:
                    oc += _mm(Pl, vc)
            sd = T(np.exp(half).astype(np.float32))  # half decay per key channel
            Sd = S * sd
            if splits["st"] == "direct":
                h16 = f16_round(np.exp(half).astype(np.float32))  # [N, 1, Dk]
                base = h16
                for Uj16, hj16 in earlier:
                    e = f16_round(base * hj16)
                    oc += _mm(f16_round(qt), f16_round(Uj16 * T(e)))
                    base = f16_round(e * hj16)
            else:
                Sh, Sl = _split(Sd)
                oc += _mm(qh, Sh)
                if splits["iq"] >= 2:
                    oc += _mm(ql, Sh)
                if splits["st"] >= 2:
                    oc += _mm(qh, Sl)
            o[:, sl] += s * oc
            if splits["u"] == "f16":
                U = _mm(T(f16_round(kt)), vc)
            else:
                U = _mm(T(kh), vc)
                if splits["u"] >= 2:
                    U += _mm(T(kl), vc)
            if splits["st"] == "direct":
                earlier.insert(0, (f16_round(U), f16_round(np.exp(half).astype(np.float32))))
            S = (Sd + U) * sd
    return o


def emulate_tiles(q, k, v, gf, gb, tile=32):
    """The tile-pair kernel's fp16 form.  Same arguments and result as `emulate`.  Per direction and 32-token tile:
    tile-local cumulative gates G (fp32), total T; a = f16(exp(G)), b = f16(exp(-G)), d = f16(exp(T));
    q^ = f16(q a), k' = f16(k b), k^ = f16(k' d); own tile: P = mask(k' q^T), rounded to fp16 per direction and the two
    directions added in fp16; another tile j walked outwards: q^ <- f16(q^ d_m) for every tile m passed, P = k^_j q^T
    rounded once to fp16; O += P V with fp32 accumulation (chunk_util.py:37-78 with the anchors per tile)."""
    N, L, Dk = q.shape
    Dv = v.shape[-1]
    s = np.float32(Dk ** -0.5)
    nt = -(-L // tile)
    T_ = lambda x: x.transpose(0, 2, 1)
    sl = [slice(i * tile, min(L, (i + 1) * tile)) for i in range(nt)]
    acc = np.zeros((N, L, Dv), np.float32)
    diag = [np.zeros((N, sl[i].stop - sl[i].start, sl[i].stop - sl[i].start), np.float32) for i in range(nt)]
    for direction in (0, 1):
        g = gf if direction == 0 else gb
        qh, kc, kh, d = [], [], [], []
        for i in range(nt):
            gc = g[:, sl[i]].astype(np.float32)
            if direction == 0:
                G = np.cumsum(gc, axis=1, dtype=np.float32)
                Tt = G[:, -1:, :]
            else:
                G = np.flip(np.cumsum(np.flip(gc, 1), axis=1, dtype=np.float32), 1)
                Tt = G[:, :1, :]
            a16, b16 = f16_round(np.exp(G)), f16_round(np.exp(-G))
            d16 = f16_round(np.exp(Tt))
            qh.append(f16_round(q[:, sl[i]] * a16))
            kci = f16_round(k[:, sl[i]] * b16)
            kc.append(kci)
            kh.append(f16_round(kci * d16))
            d.append(d16)
        for i in range(nt):
            n = qh[i].shape[1]
            tri = np.tril(np.ones((n, n), np.float32)) if direction == 0 else np.triu(np.ones((n, n), np.float32))
            # own tile: P[i, j] over the pairs the direction keeps; the two directions meet in fp16
            diag[i] = f16_round(diag[i] + f16_round(_mm(qh[i], T_(kc[i])) * tri))
            qw = qh[i]
            others = range(i - 1, -1, -1) if direction == 0 else range(i + 1, nt)
            for step, j in enumerate(others):
                if step > 0:
                    qw = f16_round(qw * d[j + 1 if direction == 0 else j - 1])
                acc[:, sl[i]] += _mm(f16_round(_mm(qw, T_(kh[j]))), v[:, sl[j]])
    for i in range(nt):
        acc[:, sl[i]] += _mm(diag[i], v[:, sl[i]])
    return s * acc
