"""CPU oracle for ViG's bidirectional gated-linear-attention (GLA) forward path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; it
is the checker used by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py.  The product path is the HIP library and fails loudly without it.

Every function restates, in float64 numpy (or float32 torch for the timed CPU
baseline), the arithmetic of one reference routine; the reference file:line it
follows is cited in each docstring (paths relative to the reference checkout).

Pinning status (what fixes each function besides its own formula):
  * gla_recurrent / bidir_gla_recurrent  -- pinned by tests/test_oracle.py:
        L=1 closed form, g=0 (plain tril/triu matmul), g=-inf limit, constant
        per-channel gate closed form, brute-force triple loop on tiny sizes,
        the independently derived quadratic form (gla_parallel), flip symmetry,
        chunk-size invariance / state passing, linearity in v.
  * gla_parallel                         -- pinned against the brute-force loop
        and against gla_recurrent (independent derivation).
  * gla_chunked                          -- pinned by chunk-size invariance and
        explicit zero-padding equivalence (L=196/197 vs padded inputs).
  * dirgate_reference                    -- torch.nn.functional.logsigmoid plus an
        index-by-index layout brute force.
  * locality_* / rmsnorm_reference       -- torch.nn.functional.conv2d and the
        reference's own closed formula; layout brute force.
  * locality_sigmoid_gate_reference      -- tests/test_oracle_model.py: the library
        convolution on an explicitly rearranged [B, C, h, w] tensor, an index-by-index
        brute force on a 3 x 4 grid with H != Dv, zero / centre-tap / one-sided weights.
  * layernorm_reference                  -- torch.nn.functional.layer_norm (+ silu)
        in float64, and the mean-0 / variance-1 invariant.
  * naive_recurrent_gla_f32              -- float32 torch port of the reference's
        CPU-runnable routine; pinned against gla_recurrent (fp64) to 1e-5.
The reference holds no golden vectors for this path (its tests are GPU-only
kernel-vs-kernel comparisons), so nothing here is pinned by reference fixtures;
the composed eval-mode model forward is restated in vig_model_ref.py and pinned there.
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# a1: the recurrence
# --------------------------------------------------------------------------


def gla_recurrent(q, k, v, g, scale=None, reverse=False, initial_state=None,
                  return_state=False):
    """One-direction recurrent GLA in float64.

    Follows fla/ops/gla/naive.py:33-41 (forward sweep) and :48-56 (reverse
    sweep): S_t = diag(exp(g_t)) S_{t-1} + k_t v_t^T ; o_t = (scale*q_t)^T S_t.
    The reference hard-casts to float32 (naive.py:23); this restatement works in
    float64 so it can serve as ground truth for both fp32 and bf16 kernels.

    q, k, g: [B, H, L, Dk]; v: [B, H, L, Dv]; log-gates g <= 0 (natural log).
    reverse=True walks tokens L-1..0 (the gate of token t decays the state that
    arrives from t+1).  Returns o [B, H, L, Dv] (and the final state).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if scale is None or scale == -1:
        scale = Dk ** -0.5
    S = np.zeros((B, H, Dk, Dv), dtype=np.float64)
    if initial_state is not None:
        S = S + np.asarray(initial_state, dtype=np.float64)
    o = np.zeros((B, H, L, Dv), dtype=np.float64)
    order = range(L - 1, -1, -1) if reverse else range(L)
    a = np.exp(g)
    for t in order:
        S = S * a[:, :, t, :, None] + k[:, :, t, :, None] * v[:, :, t, None, :]
        o[:, :, t] = np.einsum("bhk,bhkv->bhv", q[:, :, t] * scale, S)
    if return_state:
        return o, S
    return o


def bidir_gla_recurrent(q, k, v, g_fwd, g_bwd, scale=None, out_scale=1.0):
    """Bidirectional GLA with independent per-direction gates, natural token order.

    o = out_scale * (o_fwd + o_bwd).  This is what the reference's merged
    inference kernel computes (fla/ops/gla/recurrent_fuse.py:19-148, forward
    pointers from token 0, reverse pointers from token T-1, reverse gates taken
    from the second half of the gate batch :79-80) with out_scale = 1/2 applied at
    recurrent_fuse.py:442, and what the training glue computes by flip-concat
    (classification/models/vig.py:407-409,425-426; chunk_fuse.py:574-596).
    The diagonal term scale*(q_i.k_i) v_i is counted in both directions.
    """
    of = gla_recurrent(q, k, v, g_fwd, scale=scale, reverse=False)
    ob = gla_recurrent(q, k, v, g_bwd, scale=scale, reverse=True)
    return out_scale * (of + ob)


def gla_recurrent_backward(q, k, v, g, do, scale=None, reverse=False):
    """Gradients of gla_recurrent's output contracted with `do`, float64, by the adjoint recurrences.

    Same derivatives as the reference's chunked backward (fla/ops/gla/chunk_fuse.py:413-518 with the
    gate gradient of :505-518, `dg = q*dq - k*dk` followed by a reversed cumulative sum), written per token:
        dS_t = (scale*q_t) do_t^T + diag(exp(g_{t'})) dS_{t'}      (t' = the token walked after t)
        dq_t = scale * S_t do_t ;  dk_t = dS_t v_t ;  dv_t = dS_t^T k_t
        dG_t = q_t*dq_t - k_t*dk_t ;  dg_t = sum of dG over t and every token walked after it.
    Returns dq, dk, dv, dg with the shapes of q, k, v, g.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    do = np.asarray(do, dtype=np.float64)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if scale is None or scale == -1:
        scale = Dk ** -0.5
    a = np.exp(g)
    order = list(range(L - 1, -1, -1) if reverse else range(L))
    dq = np.zeros_like(q)
    S = np.zeros((B, H, Dk, Dv))
    for t in order:
        S = S * a[:, :, t, :, None] + k[:, :, t, :, None] * v[:, :, t, None, :]
        dq[:, :, t] = scale * np.einsum("bhkv,bhv->bhk", S, do[:, :, t])
    dk = np.zeros_like(k)
    dv = np.zeros_like(v)
    dg = np.zeros_like(g)
    dS = np.zeros((B, H, Dk, Dv))
    run = np.zeros((B, H, Dk))
    prev = None
    for t in reversed(order):
        if prev is not None:
            dS = dS * a[:, :, prev, :, None]
        dS = dS + scale * q[:, :, t, :, None] * do[:, :, t, None, :]
        dk[:, :, t] = np.einsum("bhkv,bhv->bhk", dS, v[:, :, t])
        dv[:, :, t] = np.einsum("bhkv,bhk->bhv", dS, k[:, :, t])
        run = run + q[:, :, t] * dq[:, :, t] - k[:, :, t] * dk[:, :, t]
        dg[:, :, t] = run
        prev = t
    return dq, dk, dv, dg


def bidir_gla_backward(q, k, v, g_fwd, g_bwd, do, scale=None, out_scale=1.0):
    """Gradients of bidir_gla_recurrent: (dq, dk, dv, dg_fwd, dg_bwd); dq, dk, dv are summed over the directions."""
    do = out_scale * np.asarray(do, dtype=np.float64)
    fq, fk, fv, fg = gla_recurrent_backward(q, k, v, g_fwd, do, scale=scale, reverse=False)
    if g_bwd is None:
        return fq, fk, fv, fg, None
    bq, bk, bv, bg = gla_recurrent_backward(q, k, v, g_bwd, do, scale=scale, reverse=True)
    return fq + bq, fk + bk, fv + bv, fg, bg


def gla_parallel(q, k, v, g, scale=None, reverse=False):
    """Quadratic ("parallel") form, derived independently of the recurrence.

    A_ij = scale * sum_d q_id k_jd exp(G_id - G_jd) for j <= i, with G the
    inclusive prefix sum of g over tokens (reverse: j >= i, G the inclusive
    suffix sum); o = A v.  The exponent is formed before exponentiation so no
    overflow occurs.  O(L^2 Dk) memory: for L <= 256 only.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, H, L, Dk = q.shape
    if scale is None or scale == -1:
        scale = Dk ** -0.5
    if reverse:
        G = np.flip(np.cumsum(np.flip(g, axis=2), axis=2), axis=2)
    else:
        G = np.cumsum(g, axis=2)
    # E[b,h,i,j,d] = G_i - G_j   (<= 0 on the kept triangle)
    E = G[:, :, :, None, :] - G[:, :, None, :, :]
    idx = np.arange(L)
    keep = (idx[None, :] >= idx[:, None]) if reverse else (idx[None, :] <= idx[:, None])
    E = np.where(keep[None, None, :, :, None], E, -np.inf)
    A = scale * np.einsum("bhid,bhjd,bhijd->bhij", q, k, np.exp(E))
    return np.einsum("bhij,bhjv->bhiv", A, v)


def gla_bruteforce(q, k, v, g, scale=None, reverse=False):
    """Literal triple loop over the unrolled sum; tiny sizes only.

    o_i = scale * sum_{j<=i} sum_d q_id k_jd exp(sum_{t=j+1..i} g_td) v_j
    (reverse: j >= i and the decay uses t = i..j-1).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if scale is None or scale == -1:
        scale = Dk ** -0.5
    o = np.zeros((B, H, L, Dv))
    for b in range(B):
        for h in range(H):
            for i in range(L):
                js = range(i, L) if reverse else range(0, i + 1)
                for j in js:
                    for d in range(Dk):
                        if reverse:
                            dec = sum(g[b, h, t, d] for t in range(i, j))
                        else:
                            dec = sum(g[b, h, t, d] for t in range(j + 1, i + 1))
                        o[b, h, i] += scale * q[b, h, i, d] * k[b, h, j, d] * np.exp(dec) * v[b, h, j]
    return o


# --------------------------------------------------------------------------
# a2-a6: the chunked algebra (forward direction) used by the fused-chunk op
# --------------------------------------------------------------------------


def gla_chunked(q, k, v, g, chunk=16, scale=None, initial_state=None, return_state=False):
    """Chunked forward GLA in float64, mirroring the reference's fused-chunk op.

    Follows fla/ops/gla/chunk_fuse.py:554-572 (default scale, zero-pad the tail
    to a multiple of the chunk, slice the output), chunk_util.py:9-78 (chunk-local
    inclusive cumsum G, q~ = scale*q*exp(G), k~ = k*exp(G_last-G)),
    chunk_fuse.py:76-97 (o_inter = q~ S_prev ; S = S*exp(G_last) + k~^T v) and
    chunk_fuse.py:245-254 (A_ij = sum_d q_i k_j exp(G_i-G_j), j <= i).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if scale is None or scale == -1:
        scale = Dk ** -0.5
    T = -(-L // chunk) * chunk
    pad = T - L

    def padL(x):
        return np.pad(x, ((0, 0), (0, 0), (0, pad), (0, 0))) if pad else x

    q, k, v, g = map(padL, (q, k, v, g))
    S = np.zeros((B, H, Dk, Dv))
    if initial_state is not None:
        S = S + np.asarray(initial_state, dtype=np.float64)
    o = np.zeros((B, H, T, Dv))
    tri = np.tril(np.ones((chunk, chunk), dtype=bool))
    for c0 in range(0, T, chunk):
        sl = slice(c0, c0 + chunk)
        G = np.cumsum(g[:, :, sl], axis=2)
        Glast = G[:, :, -1:, :]
        qt = scale * q[:, :, sl] * np.exp(G)
        kt = k[:, :, sl] * np.exp(Glast - G)
        E = G[:, :, :, None, :] - G[:, :, None, :, :]
        E = np.where(tri[None, None, :, :, None], E, -np.inf)
        A = scale * np.einsum("bhid,bhjd,bhijd->bhij", q[:, :, sl], k[:, :, sl], np.exp(E))
        o[:, :, sl] = np.einsum("bhik,bhkv->bhiv", qt, S) + np.einsum("bhij,bhjv->bhiv", A, v[:, :, sl])
        S = S * np.exp(Glast[:, :, 0, :, None]) + np.einsum("bhjk,bhjv->bhkv", kt, v[:, :, sl])
    o = o[:, :, :L]
    if return_state:
        return o, S
    return o


# --------------------------------------------------------------------------
# a7: direction-wise gate preparation
# --------------------------------------------------------------------------


def dirgate_reference(gk_lin, num_heads, normalizer=16.0, clamp_min=None):
    """Gate preparation of the eval path, float64.

    Follows classification/models/vig.py:432-441: gk_lin [B, L, 2*H*Dk]; the
    first H*Dk channels are the forward gates and the last H*Dk the backward
    gates (chunk(2, dim=2)); each is laid out 'b n (h d) -> b h n d'; the result
    is logsigmoid(.)/normalizer with an optional lower clamp.  Returns
    [2, B, H, L, Dk] (index 0 = forward, 1 = backward), natural token order --
    i.e. the reference's cat([fw, bw], dim=0) viewed as [2, B, ...].
    """
    x = np.asarray(gk_lin, dtype=np.float64)
    B, L, C2 = x.shape
    Dk = C2 // (2 * num_heads)
    x = x.reshape(B, L, 2, num_heads, Dk).transpose(2, 0, 3, 1, 4)
    # logsigmoid(x) = -softplus(-x) = min(x,0) - log1p(exp(-|x|))
    y = np.minimum(x, 0.0) - np.log1p(np.exp(-np.abs(x)))
    y = y / normalizer
    if clamp_min is not None:
        y = np.maximum(y, clamp_min)
    return np.ascontiguousarray(y)


# --------------------------------------------------------------------------
# a8: 2D locality injection
# --------------------------------------------------------------------------


def dwconv3x3_reference(x_blc, weight, hw, bias=None, silu=False):
    """3x3 depthwise conv (zero pad 1) on the token grid, float64.

    Follows classification/models/vig.py:291-294,428-430: x [B, L, C] with
    L = h*w row-major is viewed as [B, C, h, w], convolved per channel with
    weight [C, 1, 3, 3] (cross-correlation, as torch.nn.Conv2d), optional bias
    and SiLU, and returned as [B, L, C].
    """
    x = np.asarray(x_blc, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64).reshape(-1, 3, 3)
    B, L, C = x.shape
    h, wd = hw
    assert L == h * wd
    x2 = x.reshape(B, h, wd, C)
    xp = np.pad(x2, ((0, 0), (1, 1), (1, 1), (0, 0)))
    y = np.zeros_like(x2)
    for di in range(3):
        for dj in range(3):
            y += xp[:, di:di + h, dj:dj + wd, :] * w[None, None, None, :, di, dj]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    if silu:
        y = y / (1.0 + np.exp(-y))
    return y.reshape(B, L, C)


def locality_sigmoid_gate_reference(o_bhld, weight, hw):
    """Synthetic locality gate of the ViG-B benchmark shape, float64.

    y = o * sigmoid(dwconv3x3(u)) with u = o rearranged 'b h l d -> b l (h d)'
    on the h x w token grid; output in the [B, H, L, Dv] layout of o.
    """
    o = np.asarray(o_bhld, dtype=np.float64)
    B, H, L, D = o.shape
    u = o.transpose(0, 2, 1, 3).reshape(B, L, H * D)
    c = dwconv3x3_reference(u, weight, hw)
    gate = 1.0 / (1.0 + np.exp(-c))
    y = u * gate
    return y.reshape(B, L, H, D).transpose(0, 2, 1, 3)


def rmsnorm_reference(x, weight, eps=1e-6):
    """x * rsqrt(mean(x^2, -1) + eps) * weight  (fla/modules/rmsnorm.py:38-52)."""
    x = np.asarray(x, dtype=np.float64)
    r = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    return x * r * np.asarray(weight, dtype=np.float64)


def layernorm_reference(x, weight, bias, eps=1e-5, silu=False, round_to=None):
    """LayerNorm over the last axis, float64, biased variance (torch.nn.functional.layer_norm as called by
    LayerNorm2d, classification/models/vig.py:619-624); silu applies x*sigmoid(x) to the result after round_to (a
    function float64 array -> float64 array: the separate activation of vig.py:653 reads stored values)."""
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mu) / np.sqrt(var + eps) * np.asarray(weight, dtype=np.float64) + np.asarray(bias, dtype=np.float64)
    if silu:
        if round_to is not None:
            y = round_to(y)
        y = y / (1.0 + np.exp(-y))
    return y


def rmsnorm_residual_reference(x, weight, eps=1e-6, residual=None, round_to=None):
    """Residual-add + RMS norm, float64: s = x + residual; y = s*rsqrt(mean(s^2)+eps)*weight; returns (y, s)
    (fla/modules/rmsnorm.py:98-125 with IS_RMS_NORM, HAS_RESIDUAL, STORE_RESIDUAL_OUT).  round_to, a function
    float64 array -> float64 array, rounds s to a storage type before it is normalised (what norm(x + residual) on
    stored tensors computes, classification/models/vig.py:598,606)."""
    s = np.asarray(x, dtype=np.float64)
    if residual is not None:
        s = s + np.asarray(residual, dtype=np.float64)
    if round_to is not None:
        s = round_to(s)
    return rmsnorm_reference(s, weight, eps), s


def split_heads_reference(qkv_blw, num_heads, dk, dv):
    """qkv [B, L, H*dk | H*dk | H*dv] -> q, k [B,H,L,dk], v [B,H,L,dv] (classification/models/vig.py:401-409)."""
    x = np.asarray(qkv_blw)
    B, L, _ = x.shape
    H = num_heads
    K = H * dk
    q = x[..., :K].reshape(B, L, H, dk).transpose(0, 2, 1, 3)
    k = x[..., K:2 * K].reshape(B, L, H, dk).transpose(0, 2, 1, 3)
    v = x[..., 2 * K:].reshape(B, L, H, dv).transpose(0, 2, 1, 3)
    return q, k, v


def swiglu_reference(gate_up):
    """(gate | up) halves of the last dimension -> gate * up / (1 + exp(-gate)), float64
    (flash-linear-attention/fla/modules/activations.py:109-113)."""
    x = np.asarray(gate_up, dtype=np.float64)
    I = x.shape[-1] // 2
    g, u = x[..., :I], x[..., I:]
    return g * u / (1.0 + np.exp(-g))


def locality_blend_reference(o_bhld, local_blc, glin_blc, w_g, w_l, eps=1e-6, silu_out=False):
    """Block epilogue before o_proj, float64.

    Follows classification/models/vig.py:444-457: o [B,H,L,Dv] -> [B,L,H,Dv];
    local_out [B,L,(H Dv)] -> [B,L,H,Dv]; both RMS-normalised over Dv with
    weights w_g / w_l; gamma = sigmoid(g_lin); y = o^ * gamma + l^ * (1-gamma);
    optional SiLU; returned as [B, L, H*Dv].
    """
    o = np.asarray(o_bhld, dtype=np.float64).transpose(0, 2, 1, 3)
    B, L, H, D = o.shape
    loc = np.asarray(local_blc, dtype=np.float64).reshape(B, L, H, D)
    gam = 1.0 / (1.0 + np.exp(-np.asarray(glin_blc, dtype=np.float64).reshape(B, L, H, D)))
    y = rmsnorm_reference(o, w_g, eps) * gam + rmsnorm_reference(loc, w_l, eps) * (1.0 - gam)
    if silu_out:
        y = y / (1.0 + np.exp(-y))
    return y.reshape(B, L, H * D)


# --------------------------------------------------------------------------
# CPU baseline: float32 torch port of the reference's only CPU-runnable routine
# --------------------------------------------------------------------------


def naive_recurrent_gla_f32(q, k, v, gk, reverse=False):
    """float32 torch port of fla/ops/gla/naive.py:13-58 (one sweep).

    Same operation order per token as the reference loop (scale q, exp the gate,
    outer product, decay-and-add, reduce over Dk).  Used only as the timed CPU
    baseline and in oracle self-checks.
    """
    import torch

    q, k, v, gk = (x.float() for x in (q, k, v, gk))
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    h = torch.zeros(B, H, Dk, Dv, dtype=torch.float32)
    o = torch.zeros_like(v)
    scale = Dk ** -0.5
    order = range(L - 1, -1, -1) if reverse else range(L)
    for i in order:
        q_i = q[:, :, i, :] * scale
        k_i = k[:, :, i]
        v_i = v[:, :, i, :]
        gk_i = gk[:, :, i].exp()
        kv_i = k_i[..., None] * v_i[..., None, :]
        h = h * gk_i[..., None] + kv_i
        o[:, :, i] = (q_i[..., None] * h).sum(-2)
    return o


def bidir_naive_recurrent_gla_f32(q, k, v, g_fwd, g_bwd):
    """Two float32 sweeps with independent gates, outputs summed (CPU baseline)."""
    return naive_recurrent_gla_f32(q, k, v, g_fwd, False) + naive_recurrent_gla_f32(q, k, v, g_bwd, True)
