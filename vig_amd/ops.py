"""Op-level Python interface: the reference's GLA call signatures over the HIP library.

Mirrors (same names, positional order, defaults and return convention):
  fused_chunk_gla              flash-linear-attention/fla/ops/gla/chunk_fuse.py:554-572
  batch_bid_fused_chunk_gla    fla/ops/gla/chunk_fuse.py:574-596
  bid_fused_recurrent_gla      fla/ops/gla/recurrent_fuse.py:659-676
  fused_recurrent_gla          fla/ops/gla/recurrent_fuse.py:631-657
The ops are differentiable: when autograd is recording and an input requires a
gradient, the backward runs the library's backward kernels (the reference's own
merged bidirectional op has no working backward, recurrent_fuse.py:443,456).
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple

import torch

from . import _lib

_DT = {torch.float32: _lib.VIG_F32, torch.bfloat16: _lib.VIG_BF16}


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; float32 and bfloat16 are built") from None


def _dense(t: torch.Tensor) -> torch.Tensor:
    """t contiguous and on a 16-byte boundary (the kernels move 16 bytes per access and the library refuses
    anything else): a view that starts in mid-row of its storage is copied."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


def _check_cuda(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise _lib.VigGlaError("vig_amd ops run on the GPU only (tensor is on %s); there is no CPU path" % t.device)
        if t.device != ts[0].device:
            raise ValueError("all tensors must be on the same device")


def gla_bidir_forward(q, k, v, g_fwd, g_bwd=None, scale: float = -1, out_scale: float = 1.0,
                      exact: bool = False, out: Optional[torch.Tensor] = None,
                      strong_gates: bool = False) -> torch.Tensor:
    """o = out_scale * (fwd(q,k,v,g_fwd) + bwd(q,k,v,g_bwd)), natural token order.

    q, k, g_*: [B,H,L,Dk]; v: [B,H,L,Dv].  g_bwd=None gives the causal op.
    `exact=True` forces the fp32-arithmetic recurrent kernel.  `strong_gates=True` (inference calls only) tells the
    matrix-core kernel to start with its wide-range score variant (vig_gla_bidir_fwd_wide): worth it when most slabs
    have a channel whose gates sum below about -8 over 64 tokens.
    Differentiable: when autograd is recording and an input requires grad, the backward runs vig_gla_bidir_bwd.
    """
    tensors = (q, k, v, g_fwd) + ((g_bwd,) if g_bwd is not None else ())
    if torch.is_grad_enabled() and any(t.requires_grad for t in tensors):
        if out is not None:
            raise ValueError("`out` cannot be given when a gradient is recorded")
        if scale == -1 or scale is None:
            scale = q.shape[-1] ** -0.5
        return _GLABidirFunction.apply(q, k, v, g_fwd, g_bwd, float(scale), float(out_scale), bool(exact))
    return _gla_bidir_forward_raw(q, k, v, g_fwd, g_bwd, scale, out_scale, exact, out, strong_gates)


def gla_bidir_backward(q, k, v, g_fwd, g_bwd, d_o, scale: float = -1, out_scale: float = 1.0,
                       exact: bool = False):
    """Gradients of gla_bidir_forward contracted with d_o: (dq, dk, dv, dg_fwd, dg_bwd or None).

    bf16 tensors and gates with Dk in {32, 64} and Dv = 64 run on the matrix cores, bidirectional or causal, any L (sequences
    longer than 256 tokens as segments chained through their states; bf16 operands,
    fp32 accumulation); everything else, and `exact=True`, on the fp32-arithmetic token-recurrent kernel.  Head widths
    of 128 are taken block by block (64 x 64 blocks, summed here).
    """
    lib = _lib.load()
    _check_cuda(q, k, v, g_fwd, g_bwd, d_o)
    q, k, v, g_fwd, d_o = (_dense(t) for t in (q, k, v, g_fwd, d_o))
    if g_bwd is not None:
        g_bwd = _dense(g_bwd)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if d_o.shape != v.shape or d_o.dtype != q.dtype:
        raise ValueError("d_o must match the output in shape and dtype")
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    if (Dk > 64 or Dv > 64) and Dk % 64 == 0 and Dv % 64 == 0:
        return _gla_bidir_backward_blocks(q, k, v, g_fwd, g_bwd, d_o, float(scale), out_scale, exact)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dgf = torch.empty_like(g_fwd)
    dgb = torch.empty_like(g_bwd) if g_bwd is not None else None
    if exact:
        ws_bytes = lib.vig_gla_bidir_bwd_workspace(B, H, L, Dk, Dv, int(g_bwd is not None))
    else:  # the workspace of the dispatched path (HierViG's head shape rides the matrix cores zero-padded)
        ws_bytes = lib.vig_gla_bidir_bwd_workspace_for(B, H, L, Dk, Dv, _dt(q), _dt(g_fwd), int(g_bwd is not None))
    if ws_bytes == 0:
        raise _lib.VigGlaError(f"vig_gla_bidir_bwd: shape Dk={Dk}, Dv={Dv} is not built")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        fn = lib.vig_gla_bidir_bwd_exact if exact else lib.vig_gla_bidir_bwd
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(),
                                   g_bwd.data_ptr() if g_bwd is not None else None, d_o.data_ptr(),
                                   dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dgf.data_ptr(),
                                   dgb.data_ptr() if dgb is not None else None, ws.data_ptr(), ws_bytes,
                                   B, H, L, Dk, Dv, float(scale), float(out_scale), _dt(q), _dt(g_fwd), _stream_ptr(q))
    _lib.check(rc, "vig_gla_bidir_bwd")
    return dq, dk, dv, dgf, dgb


def _gla_bidir_backward_blocks(q, k, v, g_fwd, g_bwd, d_o, scale, out_scale, exact):
    """Head widths beyond 64 (the reference's own op tests use Dk = Dv = 128, tests/ops/test_gla.py:10-77): the op is a
    sum over key channels and acts on every value channel separately, so its backward is the backward of the 64 x 64
    blocks: dq, dk and the gate gradients of a key block summed over the value blocks, dv of a value block summed over
    the key blocks (in fp32; each block call rounds to the tensors' dtype once)."""
    Dk, Dv = q.shape[-1], v.shape[-1]
    kb = [slice(i, i + 64) for i in range(0, Dk, 64)]
    vb = [slice(i, i + 64) for i in range(0, Dv, 64)]
    f32 = lambda t: torch.zeros(t.shape, dtype=torch.float32, device=t.device)
    dq, dk, dv, dgf = f32(q), f32(k), f32(v), f32(g_fwd)
    dgb = f32(g_bwd) if g_bwd is not None else None
    for a in kb:
        qa, ka, gfa = (t[..., a].contiguous() for t in (q, k, g_fwd))
        gba = g_bwd[..., a].contiguous() if g_bwd is not None else None
        for b in vb:
            r = gla_bidir_backward(qa, ka, v[..., b].contiguous(), gfa, gba, d_o[..., b].contiguous(), scale, out_scale,
                                   exact)
            dq[..., a] += r[0].float()
            dk[..., a] += r[1].float()
            dv[..., b] += r[2].float()
            dgf[..., a] += r[3].float()
            if dgb is not None:
                dgb[..., a] += r[4].float()
    return (dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), dgf.to(g_fwd.dtype),
            dgb.to(g_bwd.dtype) if dgb is not None else None)


class _GLABidirFunction(torch.autograd.Function):
    """Autograd node of the bidirectional op (the reference's FusedChunkGLAFunction, chunk_fuse.py:315-518)."""

    @staticmethod
    def forward(ctx, q, k, v, g_fwd, g_bwd, scale, out_scale, exact):
        o = _gla_bidir_forward_raw(q, k, v, g_fwd, g_bwd, scale, out_scale, exact, None)
        ctx.save_for_backward(q, k, v, g_fwd, g_bwd)
        ctx.scale, ctx.out_scale, ctx.exact = scale, out_scale, exact
        return o

    @staticmethod
    def backward(ctx, d_o):
        q, k, v, g_fwd, g_bwd = ctx.saved_tensors
        # (a caller that asked for fp32 arithmetic gets it in both directions of the graph)
        dq, dk, dv, dgf, dgb = gla_bidir_backward(q, k, v, g_fwd, g_bwd, d_o, ctx.scale, ctx.out_scale, exact=ctx.exact)
        return dq, dk, dv, dgf, dgb, None, None, None


def _head_view_strides(t):
    """(batch, head, token) element strides of a [B,H,L,D] view whose channels are contiguous and whose rows start on
    16-byte boundaries, or None: what vig_gla_bidir_fwd_strided reads in place."""
    sb, sh, st, sd = t.stride()
    if t.is_contiguous() or sd != 1 or min(sb, sh, st) <= 0 or sb % 8 or sh % 8 or st % 8 or st > (1 << 20):
        return None
    return (sb, sh, st) if t.data_ptr() % 16 == 0 else None


def _gla_bidir_forward_strided(q, k, v, g_fwd, g_bwd, scale, out_scale, out):
    """The op on head-split views of wider token rows (e.g. column blocks of a projection output), read in place by
    the matrix-core slab kernel; None when the call is not of that kind."""
    if not (q.dtype == torch.bfloat16 and g_fwd.dtype == torch.bfloat16 and q.dim() == 4 and q.shape[2] <= 256
            and q.shape[3] in (32, 64) and v.shape[-1] == 64):
        return None
    if k.shape != q.shape or g_fwd.shape != q.shape or v.shape[:3] != q.shape[:3] or k.dtype != q.dtype or v.dtype != q.dtype:
        return None
    B, H, L, Dk = q.shape
    # the same refusals as the dense path, before anything is handed to a kernel that trusts its arguments
    if g_bwd is not None and (g_bwd.dtype != g_fwd.dtype or g_bwd.shape != g_fwd.shape):
        raise ValueError("g_bwd must match g_fwd in dtype and shape")
    if out is not None and not (out.is_contiguous() and out.data_ptr() % 16 == 0 and out.shape == (B, H, L, 64)
                                and out.dtype == q.dtype and out.device == q.device):
        raise ValueError("bad `out` tensor")
    strides = []
    for t, D in ((q, Dk), (k, Dk), (v, 64)):
        st = _head_view_strides(t)
        if st is None:
            if not t.is_contiguous() or t.data_ptr() % 16:
                return None
            st = (H * L * D, L * D, D)
        strides.append((ctypes.c_longlong * 3)(*st))
    if all(t.is_contiguous() for t in (q, k, v)):
        return None
    lib = _lib.load()
    g_fwd = _dense(g_fwd)
    g_bwd = _dense(g_bwd) if g_bwd is not None else None
    if out is None:
        out = torch.empty(B, H, L, 64, dtype=q.dtype, device=q.device)
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    with torch.cuda.device(q.device):
        rc = lib.vig_gla_bidir_fwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(),
                                           g_bwd.data_ptr() if g_bwd is not None else None, out.data_ptr(),
                                           B, H, L, Dk, 64, ctypes.addressof(strides[0]), ctypes.addressof(strides[1]),
                                           ctypes.addressof(strides[2]), float(scale), float(out_scale),
                                           _lib.VIG_BF16, _lib.VIG_BF16, _stream_ptr(q))
    _lib.check(rc, "vig_gla_bidir_fwd_strided")
    return out


def _gla_bidir_forward_raw(q, k, v, g_fwd, g_bwd, scale, out_scale, exact, out, strong_gates=False):
    lib = _lib.load()
    _check_cuda(q, k, v, g_fwd, g_bwd)
    if not exact and not strong_gates and (out is None or (out.is_contiguous() and out.data_ptr() % 16 == 0)):
        o = _gla_bidir_forward_strided(q, k, v, g_fwd, g_bwd, scale, out_scale, out)
        if o is not None:
            return o
    q, k, v, g_fwd = (_dense(t) for t in (q, k, v, g_fwd))
    if g_bwd is not None:
        g_bwd = _dense(g_bwd)
        if g_bwd.dtype != g_fwd.dtype or g_bwd.shape != g_fwd.shape:
            raise ValueError("g_bwd must match g_fwd in dtype and shape")
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if k.shape != q.shape or g_fwd.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError("shape mismatch between q, k, v, g")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share a dtype")
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    io_dt, g_dt = _dt(q), _dt(g_fwd)
    if out is None:
        out = torch.empty(B, H, L, Dv, dtype=q.dtype, device=q.device)
    elif not (out.is_contiguous() and out.data_ptr() % 16 == 0 and out.shape == (B, H, L, Dv)
              and out.dtype == q.dtype):
        raise ValueError("bad `out` tensor")
    fn = lib.vig_gla_bidir_fwd_exact if exact else (lib.vig_gla_bidir_fwd_wide if strong_gates else lib.vig_gla_bidir_fwd)
    if exact:  # the token-recurrent kernel parks the first direction's fp32 sums when the tensors are narrower
        ws_bytes = B * H * L * Dv * 4 if (g_bwd is not None and io_dt != _lib.VIG_F32) else 0
    else:
        ws_bytes = lib.vig_gla_bidir_fwd_workspace_for(B, H, L, Dk, Dv, io_dt, g_dt, int(g_bwd is not None))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    with torch.cuda.device(q.device):
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(),
                g_bwd.data_ptr() if g_bwd is not None else None, out.data_ptr(),
                ws.data_ptr() if ws is not None else None, ws_bytes,
                B, H, L, Dk, Dv, float(scale), float(out_scale), io_dt, g_dt, _stream_ptr(q))
    _lib.check(rc, "vig_gla_bidir_fwd")
    return out


def _split_bid_gates(q, g):
    B = q.shape[0]
    if g.shape[0] != 2 * B:
        raise ValueError(f"bidirectional gates must be [2B,H,L,Dk]; got batch {g.shape[0]} for B={B}")
    return g[:B], g[B:]


def gla_causal_state_forward(q, k, v, g, initial_state=None, output_final_state: bool = False, scale: float = -1,
                             exact: bool = False):
    """The causal op with a state carried in and / or out: (o, final_state or None).

    initial_state [B,H,Dk,Dv] (any float dtype; used as fp32, detached as in chunk_fuse.py:565-566) is the state
    before the first token; final_state is fp32 [B,H,Dk,Dv] (chunk_fuse.py:353-356).  A call that records a gradient
    goes through _causal_state_recording."""
    lib = _lib.load()
    _check_cuda(q, k, v, g, initial_state)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v, g)):
        return _causal_state_recording(q, k, v, g, initial_state, output_final_state, scale, exact)
    q, k, v, g = (_dense(t) for t in (q, k, v, g))
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if k.shape != q.shape or g.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError("shape mismatch between q, k, v, g")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share a dtype")
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    s0 = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (B, H, Dk, Dv):
            raise ValueError(f"initial_state must be [B,H,Dk,Dv] = {(B, H, Dk, Dv)}; got {tuple(initial_state.shape)}")
        s0 = _dense(initial_state.detach().float())
    final = torch.empty(B, H, Dk, Dv, dtype=torch.float32, device=q.device) if output_final_state else None
    out = torch.empty(B, H, L, Dv, dtype=q.dtype, device=q.device)
    io_dt, g_dt = _dt(q), _dt(g)
    ptrs = (q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), out.data_ptr(),
            s0.data_ptr() if s0 is not None else None, final.data_ptr() if final is not None else None)
    tail = (B, H, L, Dk, Dv, float(scale), 1.0, io_dt, g_dt, _stream_ptr(q))
    with torch.cuda.device(q.device):
        if exact:
            rc = lib.vig_gla_causal_state_fwd_exact(*ptrs, *tail)
        else:
            ws_bytes = lib.vig_gla_causal_state_fwd_workspace(B, H, L, Dk, Dv, io_dt, g_dt)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
            rc = lib.vig_gla_causal_state_fwd(*ptrs, ws.data_ptr() if ws is not None else None, ws_bytes, *tail)
    _lib.check(rc, "vig_gla_causal_state_fwd")
    return out, final


def _causal_state_recording(q, k, v, g, initial_state, output_final_state, scale, exact):
    """The causal op with a state in and / or out while autograd records.  As in the reference the initial state is a
    constant (chunk_fuse.py:565-566 detaches it) and the final state carries no gradient (chunk_fuse.py:413: its
    cotangent is ignored), so what is needed are the gradients of q, k, v, g with the initial state's share in them.
    The library's backward kernels start from a zero state; a state S0 is what 2*Dk gate-free tokens in front of the
    sequence leave behind (keys = unit vectors, values = the rows of S0 as a high and a low part in the tensors' dtype,
    queries zero), so the plain differentiable op on the lengthened sequence gives outputs and gradients alike."""
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    final = None
    if output_final_state:
        with torch.no_grad():
            final = gla_causal_state_forward(q.detach(), k.detach(), v.detach(), g.detach(), initial_state, True, scale,
                                             exact)[1]
    if initial_state is None:
        return gla_bidir_forward(q, k, v, g, None, scale, 1.0, exact=exact), final
    if tuple(initial_state.shape) != (B, H, Dk, Dv):
        raise ValueError(f"initial_state must be [B,H,Dk,Dv] = {(B, H, Dk, Dv)}; got {tuple(initial_state.shape)}")
    s0 = initial_state.detach().float()
    hi = s0.to(v.dtype)
    lo = (s0 - hi.float()).to(v.dtype)
    eye = torch.eye(Dk, dtype=k.dtype, device=k.device).expand(B, H, Dk, Dk)
    zq = torch.zeros(B, H, 2 * Dk, Dk, dtype=q.dtype, device=q.device)
    zg = torch.zeros(B, H, 2 * Dk, Dk, dtype=g.dtype, device=g.device)
    o = gla_bidir_forward(torch.cat([zq, q], 2), torch.cat([eye, eye, k], 2), torch.cat([hi, lo, v], 2),
                          torch.cat([zg, g], 2), None, scale, 1.0, exact=exact)
    return o[:, :, 2 * Dk:], final


def fused_chunk_gla(q, k, v, g, scale: int = -1, initial_state=None, output_final_state: bool = False
                    ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Causal GLA on [B,H,L,D] tensors; returns (o, final_state) with final_state None unless asked for
    (chunk_fuse.py:554-572)."""
    if initial_state is not None or output_final_state:
        return gla_causal_state_forward(q, k, v, g, initial_state, output_final_state, scale)
    return gla_bidir_forward(q, k, v, g, None, scale, 1.0), None


def fused_recurrent_gla(q, k, v, gk=None, gv=None, scale: int = -1, initial_state=None,
                        output_final_state: bool = False, causal: bool = True):
    """Causal recurrent GLA (fp32 state arithmetic); causal=False returns [o, o_reversed] with shared gates."""
    if gv is not None:
        raise NotImplementedError("value gates (gv) are not used by ViG and not built")
    if gk is None:
        gk = torch.zeros_like(q)
    if initial_state is not None or output_final_state:
        if not causal:  # (recurrent_fuse.py:650-652 asserts the same)
            raise NotImplementedError("bidirectional GLA takes no initial/final state")
        return gla_causal_state_forward(q, k, v, gk, initial_state, output_final_state, scale, exact=True)
    o = gla_bidir_forward(q, k, v, gk, None, scale, 1.0, exact=True)
    if causal:
        return o, None
    f = lambda x: x.flip(dims=[2])
    o_rev = f(gla_bidir_forward(f(q), f(k), f(v), f(gk), None, scale, 1.0, exact=True))
    return [o, o_rev]


def batch_bid_fused_chunk_gla(q, k, v, g, scale: int = -1, initial_state=None, output_final_state: bool = False
                              ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q,k,v [B,H,L,D]; g [2B,H,L,Dk] = cat(fwd gates, bwd gates), both in natural order; o=(o_f+o_b)/2."""
    if initial_state is not None or output_final_state:
        raise NotImplementedError("bidirectional GLA takes no initial/final state")
    gf, gb = _split_bid_gates(q, g)
    return gla_bidir_forward(q, k, v, gf, gb, scale, 0.5), None


def bid_fused_recurrent_gla(q, k, v, gk=None, gv=None, scale: int = -1, initial_state=None,
                            output_final_state: bool = False, causal: bool = True
                            ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Merged bidirectional inference op: gk [2B,H,L,Dk] natural order; o=(o_f+o_b)/2."""
    if gv is not None:
        raise NotImplementedError("value gates (gv) are not used by ViG and not built")
    if initial_state is not None or output_final_state:
        raise NotImplementedError("bidirectional GLA takes no initial/final state")
    if not causal:
        raise NotImplementedError("causal=False on the merged op is unused by ViG and not built")
    if gk is None:
        gk = torch.zeros((2 * q.shape[0],) + tuple(q.shape[1:]), dtype=q.dtype, device=q.device)
    gf, gb = _split_bid_gates(q, gk)
    return gla_bidir_forward(q, k, v, gf, gb, scale, 0.5), None


# ---------------------------------------------------------------------------
# neighbours
# ---------------------------------------------------------------------------

def dirgate(gk_lin: torch.Tensor, num_heads: int, gate_logit_normalizer: float = 16.0,
            clamp_min: Optional[float] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """gk_lin [B,L,2*H*Dk] -> [2,B,H,L,Dk] = logsigmoid/normalizer (vig.py:432-441).
    Differentiable (vig_dirgate_bwd) when autograd is recording and gk_lin requires grad."""
    if torch.is_grad_enabled() and gk_lin.requires_grad:
        return _DirGateFunction.apply(gk_lin, num_heads, float(gate_logit_normalizer), clamp_min, out_dtype)
    return _dirgate_raw(gk_lin, num_heads, gate_logit_normalizer, clamp_min, out_dtype)


class _DirGateFunction(torch.autograd.Function):
    """Autograd node of the direction-wise gate preparation."""

    @staticmethod
    def forward(ctx, gk_lin, H, normalizer, clamp_min, out_dtype):
        gk_lin = _dense(gk_lin)
        ctx.save_for_backward(gk_lin)
        ctx.args = (H, normalizer, clamp_min)
        return _dirgate_raw(gk_lin, H, normalizer, clamp_min, out_dtype)

    @staticmethod
    def backward(ctx, d_g):
        (gk_lin,) = ctx.saved_tensors
        H, normalizer, clamp_min = ctx.args
        lib = _lib.load()
        d_g = _dense(d_g)
        B, L, C2 = gk_lin.shape
        d_in = torch.empty_like(gk_lin)
        with torch.cuda.device(gk_lin.device):
            rc = lib.vig_dirgate_bwd(gk_lin.data_ptr(), d_g.data_ptr(), d_in.data_ptr(), B, L, H, C2 // (2 * H),
                                     1.0 / normalizer, float("nan") if clamp_min is None else float(clamp_min),
                                     _dt(gk_lin), _dt(d_g), _stream_ptr(gk_lin))
        _lib.check(rc, "vig_dirgate_bwd")
        return d_in, None, None, None, None


def _dirgate_raw(gk_lin, num_heads, gate_logit_normalizer=16.0, clamp_min=None, out_dtype=None):
    lib = _lib.load()
    _check_cuda(gk_lin)
    gk_lin = _dense(gk_lin)
    B, L, C2 = gk_lin.shape
    Dk = C2 // (2 * num_heads)
    out_dtype = out_dtype or gk_lin.dtype
    out = torch.empty(2, B, num_heads, L, Dk, dtype=out_dtype, device=gk_lin.device)
    with torch.cuda.device(gk_lin.device):
        rc = lib.vig_dirgate_fwd(gk_lin.data_ptr(), out.data_ptr(), B, L, num_heads, Dk,
                                 1.0 / float(gate_logit_normalizer),
                                 float("nan") if clamp_min is None else float(clamp_min),
                                 _dt(gk_lin), _DT[out_dtype], _stream_ptr(gk_lin))
    _lib.check(rc, "vig_dirgate_fwd")
    return out


GATE_RANK = 16  # the low-rank width vig_dirgate_lowrank_fwd is built for (gate_low_rank_dim of every shipped config)


def dirgate_lowrank(gk_low: torch.Tensor, w_up: torch.Tensor, b_up: torch.Tensor, num_heads: int,
                    gate_logit_normalizer: float = 16.0, clamp_min: Optional[float] = None,
                    out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """gk_low [B,L,16] (may be a column block of a wider tensor), w_up [2*H*Dk,16], b_up [2*H*Dk] ->
    [2,B,H,L,Dk] = logsigmoid(gk_low @ w_up.T + b_up)/normalizer: the second gk_proj layer (vig.py:296-297) and
    vig.py:432-441 in one kernel; the pre-activation is rounded to gk_low's dtype as the separate layer stores it."""
    lib = _lib.load()
    _check_cuda(gk_low, w_up, b_up)
    gk_low, ld = _token_rows(gk_low)
    B, L, R = gk_low.shape
    w_up, b_up = _dense(w_up.detach()), _dense(b_up.detach())
    C2 = w_up.shape[0]
    if w_up.shape != (C2, R) or b_up.shape != (C2,) or C2 % (2 * num_heads):
        raise ValueError("w_up must be [2*H*Dk, rank] and b_up [2*H*Dk]")
    if w_up.dtype != gk_low.dtype or b_up.dtype != gk_low.dtype:
        raise TypeError("gk_low, w_up and b_up must share a dtype")
    Dk = C2 // (2 * num_heads)
    out_dtype = out_dtype or gk_low.dtype
    out = torch.empty(2, B, num_heads, L, Dk, dtype=out_dtype, device=gk_low.device)
    with torch.cuda.device(gk_low.device):
        rc = lib.vig_dirgate_lowrank_fwd(gk_low.data_ptr(), ld, w_up.data_ptr(), b_up.data_ptr(), out.data_ptr(),
                                         B, L, num_heads, Dk, R, 1.0 / float(gate_logit_normalizer),
                                         float("nan") if clamp_min is None else float(clamp_min),
                                         _dt(gk_low), _DT[out_dtype], _stream_ptr(gk_low))
    _lib.check(rc, "vig_dirgate_lowrank_fwd")
    return out


def dwconv3x3(x: torch.Tensor, weight: torch.Tensor, hw, bias: Optional[torch.Tensor] = None,
              silu: bool = False) -> torch.Tensor:
    """x [B,L,C] on the (h,w) token grid; weight [C,1,3,3] or [C,3,3]; returns [B,L,C].
    Differentiable: when autograd is recording and x, weight or bias requires grad, the input gradient is the same
    stencil kernel run with the taps mirrored, the weight and bias gradients come from vig_dwconv3x3_bwd_weight."""
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, weight, bias)):
        y = _DWConv3x3Function.apply(x, weight, bias, tuple(hw))
        return torch.nn.functional.silu(y) if silu else y
    return _dwconv3x3_raw(x, weight, hw, bias, silu)


class _DWConv3x3Function(torch.autograd.Function):
    """Autograd node of the depthwise 3x3 convolution on the token grid (vig.py:291-294), without the activation."""

    @staticmethod
    def forward(ctx, x, weight, bias, hw):
        ctx.save_for_backward(x, weight)
        ctx.hw = hw
        ctx.bias_dtype = bias.dtype if bias is not None else None
        return _dwconv3x3_raw(x, weight, hw, bias, False)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        (h, w), (B, L, C) = ctx.hw, x.shape
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            # dx[p] = sum_t w[t] dy[p - t]: the same stencil with the taps mirrored through the centre
            dx = _dwconv3x3_raw(dy, weight.detach().reshape(C, 9).flip(-1), ctx.hw, None, False)
        if ctx.needs_input_grad[1] or (ctx.bias_dtype is not None and ctx.needs_input_grad[2]):
            lib = _lib.load()
            x, dy = _dense(x), _dense(dy)
            both = torch.empty(C * 10, dtype=torch.float32, device=x.device)
            ws_bytes = lib.vig_dwconv3x3_bwd_weight_workspace(B, C)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
            with torch.cuda.device(x.device):
                rc = lib.vig_dwconv3x3_bwd_weight(x.data_ptr(), dy.data_ptr(), both.data_ptr(), ws.data_ptr(), ws_bytes,
                                                  B, h, w, C, _dt(x), _stream_ptr(x))
            _lib.check(rc, "vig_dwconv3x3_bwd_weight")
            if ctx.needs_input_grad[1]:
                dw = both[:C * 9].reshape(weight.shape).to(weight.dtype)
            if ctx.bias_dtype is not None and ctx.needs_input_grad[2]:
                db = both[C * 9:].to(ctx.bias_dtype)
        return dx, dw, db, None


def _dwconv3x3_raw(x, weight, hw, bias, silu):
    lib = _lib.load()
    _check_cuda(x, weight, bias)
    x = _dense(x)
    B, L, C = x.shape
    h, w = hw
    if L != h * w:
        raise ValueError("L must equal h*w")
    wt = _dense(weight.detach().reshape(C, 9).float())
    bs = _dense(bias.detach().float()) if bias is not None else None
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = lib.vig_dwconv3x3_fwd(x.data_ptr(), wt.data_ptr(), bs.data_ptr() if bs is not None else None,
                                   y.data_ptr(), B, h, w, C, int(silu), _dt(x), _stream_ptr(x))
    _lib.check(rc, "vig_dwconv3x3_fwd")
    return y


def locality_gate(o: torch.Tensor, weight: torch.Tensor, hw) -> torch.Tensor:
    """y = o * sigmoid(dwconv3x3(o)) on [B,H,L,Dv] with channel = head*Dv + d."""
    lib = _lib.load()
    _check_cuda(o, weight)
    o = _dense(o)
    B, H, L, Dv = o.shape
    h, w = hw
    if L != h * w:
        raise ValueError("L must equal h*w")
    wt = _dense(weight.detach().reshape(H * Dv, 9).float())
    y = torch.empty_like(o)
    with torch.cuda.device(o.device):
        rc = lib.vig_locality_gate_fwd(o.data_ptr(), wt.data_ptr(), y.data_ptr(), B, H, h, w, Dv, _dt(o),
                                       _stream_ptr(o))
    _lib.check(rc, "vig_locality_gate_fwd")
    return y


def gla_bidir_locality_gate(q, k, v, g_fwd, g_bwd, weight: torch.Tensor, hw, scale: float = -1,
                            out_scale: float = 1.0) -> torch.Tensor:
    """locality_gate(gla_bidir_forward(q, k, v, g_fwd, g_bwd), weight, hw), bit for bit.

    Shapes the one-kernel form is built for (bf16, Dk in {32,64}, Dv=64, L=h*w<=256) never write the ungated
    output to memory; every other shape makes the two calls.  Inference only.
    """
    lib = _lib.load()
    _check_cuda(q, k, v, g_fwd, g_bwd, weight)
    B, H, L, Dk = q.shape
    Dv = v.shape[-1]
    h, w = hw
    if L != h * w:
        raise ValueError("L must equal h*w")
    if scale == -1 or scale is None:
        scale = Dk ** -0.5
    fusable = (g_bwd is not None and q.dtype == torch.bfloat16 and g_fwd.dtype == torch.bfloat16 and Dk in (32, 64)
               and Dv == 64 and L <= 256 and w + 2 <= 64 and h + 2 <= 8 * (64 // (w + 2)))
    if not fusable:
        return locality_gate(gla_bidir_forward(q, k, v, g_fwd, g_bwd, scale, out_scale), weight, hw)
    q, k, v, g_fwd, g_bwd = (_dense(t.detach()) for t in (q, k, v, g_fwd, g_bwd))
    if k.shape != q.shape or g_fwd.shape != q.shape or g_bwd.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError("shape mismatch between q, k, v, g")
    if k.dtype != q.dtype or v.dtype != q.dtype or g_bwd.dtype != g_fwd.dtype:
        raise TypeError("q, k, v must share a dtype, and so must the gates")
    wt = _dense(weight.detach().reshape(H * Dv, 9).float())
    y = torch.empty(B, H, L, Dv, dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.vig_gla_bidir_locgate_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(),
                                           g_bwd.data_ptr(), wt.data_ptr(), y.data_ptr(), B, H, L, Dk, Dv, h, w,
                                           float(scale), float(out_scale), _dt(q), _dt(g_fwd), _stream_ptr(q))
    _lib.check(rc, "vig_gla_bidir_locgate_fwd")
    return y


def _token_rows(t: torch.Tensor):
    """t [B, L, C] as (tensor, elements between token rows): a column block of a contiguous wider [B, L, W] tensor
    is passed as it lies when its rows keep the 16-byte alignment of the vector loads, anything else is packed."""
    if t.dim() == 3 and not t.is_contiguous():
        B, L, C = t.shape
        sb, sl, sc = t.stride()
        if sc == 1 and sl >= C and sb == L * sl and (sl * t.element_size()) % 16 == 0 and t.data_ptr() % 16 == 0:
            return t, sl
    t = _dense(t)
    return t, t.shape[-1]


def locality_blend(o: torch.Tensor, local: torch.Tensor, g_lin: torch.Tensor, w_g: torch.Tensor,
                   w_l: torch.Tensor, eps: float = 1e-6, silu_out: bool = False) -> torch.Tensor:
    """Block epilogue (vig.py:444-457): o [B,H,L,Dv]; local, g_lin [B,L,H*Dv] -> y [B,L,H*Dv].
    g_lin may be a block of columns of a wider [B, L, W] tensor (it is read in place).
    Differentiable (vig_locality_blend_bwd) when autograd is recording and an input or a norm weight requires grad."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in (o, local, g_lin, w_g, w_l)):
        return _LocalityBlendFunction.apply(o, local, g_lin, w_g, w_l, float(eps), bool(silu_out))
    return _locality_blend_raw(o, local, g_lin, w_g, w_l, eps, silu_out)


class _LocalityBlendFunction(torch.autograd.Function):
    """Autograd node of the block epilogue: forward and backward each one kernel of the library."""

    @staticmethod
    def forward(ctx, o, local, g_lin, w_g, w_l, eps, silu_out):
        o, local, g_lin = _dense(o), _dense(local), _dense(g_lin)
        ctx.save_for_backward(o, local, g_lin, w_g, w_l)
        ctx.eps, ctx.silu_out = eps, silu_out
        return _locality_blend_raw(o, local, g_lin, w_g, w_l, eps, silu_out)

    @staticmethod
    def backward(ctx, dy):
        o, local, g_lin, w_g, w_l = ctx.saved_tensors
        lib = _lib.load()
        B, H, L, Dv = o.shape
        dy = _dense(dy)
        d_o, d_local, d_glin = torch.empty_like(o), torch.empty_like(local), torch.empty_like(g_lin)
        dw = torch.empty(2, Dv, dtype=torch.float32, device=o.device)
        ws_bytes = lib.vig_locality_blend_bwd_workspace(B, L, Dv)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=o.device)
        wg, wl = _dense(w_g.detach().float()), _dense(w_l.detach().float())
        with torch.cuda.device(o.device):
            rc = lib.vig_locality_blend_bwd(o.data_ptr(), local.data_ptr(), g_lin.data_ptr(), wg.data_ptr(),
                                            wl.data_ptr(), dy.data_ptr(), d_o.data_ptr(), d_local.data_ptr(),
                                            d_glin.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws_bytes, B, H, L, Dv,
                                            H * Dv, ctx.eps, int(ctx.silu_out), _dt(o), _stream_ptr(o))
        _lib.check(rc, "vig_locality_blend_bwd")
        return d_o, d_local, d_glin, dw[0].to(w_g.dtype), dw[1].to(w_l.dtype), None, None


def _locality_blend_raw(o, local, g_lin, w_g, w_l, eps, silu_out):
    lib = _lib.load()
    _check_cuda(o, local, g_lin, w_g, w_l)
    o, local = _dense(o), _dense(local)
    g_lin, ldg = _token_rows(g_lin)
    B, H, L, Dv = o.shape
    if local.shape != (B, L, H * Dv) or g_lin.shape != (B, L, H * Dv):
        raise ValueError("local and g_lin must be [B, L, H*Dv]")
    if local.dtype != o.dtype or g_lin.dtype != o.dtype:
        raise TypeError("o, local, g_lin must share a dtype")
    y = torch.empty_like(local)
    wg = _dense(w_g.detach().float())
    wl = _dense(w_l.detach().float())
    with torch.cuda.device(o.device):
        rc = lib.vig_locality_blend_fwd(o.data_ptr(), local.data_ptr(), g_lin.data_ptr(), wg.data_ptr(),
                                        wl.data_ptr(), y.data_ptr(), B, H, L, Dv, ldg, float(eps), int(silu_out),
                                        _dt(o), _stream_ptr(o))
    _lib.check(rc, "vig_locality_blend_fwd")
    return y


def locality_blend_linear_supported(o: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether locality_blend_linear takes this block (bf16 on the GPU, 64-channel heads, square o_proj of width 384 or
    192)."""
    return (o.is_cuda and o.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and o.dim() == 4
            and o.shape[-1] == 64 and weight.dim() == 2 and weight.shape[0] == weight.shape[1] == o.shape[1] * 64
            and weight.shape[0] in (384, 192))


def locality_blend_linear(o: torch.Tensor, local: torch.Tensor, g_lin: torch.Tensor, w_g: torch.Tensor,
                          w_l: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6,
                          silu_out: bool = False) -> torch.Tensor:
    """o_proj(locality_blend(...)) in one kernel (vig.py:444-463): the blended [B, L, H*Dv] tensor, rounded to bf16
    as locality_blend stores it, feeds the matrix instructions from on-chip memory and is never written.
    Inference only (no autograd node)."""
    lib = _lib.load()
    _check_cuda(o, local, g_lin, w_g, w_l, weight)
    o, local, w = _dense(o), _dense(local), _dense(weight.detach())
    g_lin, ldg = _token_rows(g_lin)
    B, H, L, Dv = o.shape
    if local.shape != (B, L, H * Dv) or g_lin.shape != (B, L, H * Dv):
        raise ValueError("local and g_lin must be [B, L, H*Dv]")
    if not (local.dtype == g_lin.dtype == w.dtype == o.dtype):
        raise TypeError("o, local, g_lin and weight must share a dtype")
    C = w.shape[0]
    out = torch.empty(B, L, C, dtype=o.dtype, device=o.device)
    wg = _dense(w_g.detach().float())
    wl = _dense(w_l.detach().float())
    with torch.cuda.device(o.device):
        rc = lib.vig_locality_blend_linear_fwd(o.data_ptr(), local.data_ptr(), g_lin.data_ptr(), wg.data_ptr(),
                                               wl.data_ptr(), w.data_ptr(), out.data_ptr(), B, H, L, Dv, C, ldg,
                                               float(eps), int(silu_out), _dt(o), _stream_ptr(o))
    _lib.check(rc, "vig_locality_blend_linear_fwd")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, residual: Optional[torch.Tensor] = None,
            prenorm: bool = False, round_sum: bool = False):
    """Residual-add + RMS norm over the last dimension (fla/modules/rmsnorm.py:69-125 semantics).

    Returns y, or (y, x + residual) with prenorm=True.  round_sum=True normalises the sum after rounding it to the
    storage dtype, i.e. what `norm(x + residual)` on stored tensors computes.
    """
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, residual, weight)):
        if residual is None:
            y = _RMSNormFunction.apply(x, None, weight, float(eps), False)
            return (y, x) if prenorm else y
        y, total = _RMSNormFunction.apply(x, residual, weight, float(eps), bool(round_sum))
        return (y, total) if prenorm else y
    return _rmsnorm_raw(x, weight, eps, residual, prenorm, round_sum)


class _RMSNormFunction(torch.autograd.Function):
    """Autograd node of the residual-add + RMS norm (LayerNormFn in its RMS mode, fla/modules/rmsnorm.py:390-471):
    forward and backward on the library's kernels.  With a residual it returns (y, x + residual)."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps, round_sum):
        y, total = _rmsnorm_raw(x, weight, eps, residual, True, round_sum)
        ctx.save_for_backward(total, weight)
        ctx.set_materialize_grads(False)  # an unused output hands backward None instead of a tensor of zeros
        ctx.eps, ctx.has_residual = eps, residual is not None
        return y if residual is None else (y, total)

    @staticmethod
    def backward(ctx, dy, d_total=None):
        total, weight = ctx.saved_tensors
        lib = _lib.load()
        C = total.shape[-1]
        rows = total.numel() // C
        dy = _dense(dy) if dy is not None else torch.zeros_like(total)
        if d_total is not None:
            d_total = _dense(d_total)
        w = _dense(weight.detach().float())
        ds = torch.empty_like(total)
        dw = ws = None
        ws_bytes = 0
        if ctx.needs_input_grad[2]:
            dw = torch.empty(C, dtype=torch.float32, device=total.device)
            ws_bytes = lib.vig_rmsnorm_bwd_workspace(rows, C)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=total.device)
        with torch.cuda.device(total.device):
            rc = lib.vig_rmsnorm_bwd(total.data_ptr(), w.data_ptr(), dy.data_ptr(),
                                     d_total.data_ptr() if d_total is not None else None, ds.data_ptr(),
                                     dw.data_ptr() if dw is not None else None,
                                     ws.data_ptr() if ws is not None else None, ws_bytes, rows, C, ctx.eps,
                                     _dt(total), _stream_ptr(total))
        _lib.check(rc, "vig_rmsnorm_bwd")
        if dw is not None:
            dw = dw.to(weight.dtype).reshape(weight.shape)
        return ds, (ds if ctx.has_residual else None), dw, None, None


def _rmsnorm_raw(x, weight, eps, residual, prenorm, round_sum):
    lib = _lib.load()
    _check_cuda(x, weight)
    x = _dense(x)
    C = x.shape[-1]
    rows = x.numel() // C
    if residual is not None:
        _check_cuda(residual)
        residual = _dense(residual)
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("residual must match x in shape and dtype")
    w = weight.detach()
    w = _dense(w.float())
    y = torch.empty_like(x)
    res_out = torch.empty_like(x) if (prenorm and residual is not None) else None
    with torch.cuda.device(x.device):
        rc = lib.vig_rmsnorm_fwd(x.data_ptr(), residual.data_ptr() if residual is not None else None, w.data_ptr(),
                                 y.data_ptr(), res_out.data_ptr() if res_out is not None else None, rows, C,
                                 float(eps), int(round_sum), _dt(x), _stream_ptr(x))
    _lib.check(rc, "vig_rmsnorm_fwd")
    if prenorm:
        return y, (res_out if res_out is not None else x)
    return y


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5,
              silu: bool = False, pre_bias: Optional[torch.Tensor] = None,
              post_add: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm over the last dimension of a contiguous tensor, optionally followed by SiLU on the stored value
    (LayerNorm2d and the swish behind it, vig.py:619-624,650-655, on channels-last data).  pre_bias [C] is added to
    x first (the bias of the convolution in front); post_add [P, C], P dividing the row count, is added to the
    result row-periodically (the position table, vig.py:858-865)."""
    lib = _lib.load()
    _check_cuda(x, weight, bias, pre_bias, post_add)
    x = _dense(x)
    C = x.shape[-1]
    rows = x.numel() // C
    w = _dense(weight.detach().float())
    b = _dense(bias.detach().float())
    if w.shape != (C,) or b.shape != (C,):
        raise ValueError("weight and bias must be [C]")
    pb = None
    if pre_bias is not None:
        pb = _dense(pre_bias.detach().float())
        if pb.shape != (C,):
            raise ValueError("pre_bias must be [C]")
    pa, prow = None, 0
    if post_add is not None:
        pa = _dense(post_add.detach().reshape(-1, C))
        prow = pa.shape[0]
        if pa.dtype != x.dtype or rows % prow:
            raise ValueError("post_add must have x's dtype and a row count that divides x's")
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = lib.vig_layernorm_fwd(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), rows, C,
                                   float(eps), int(silu), pb.data_ptr() if pb is not None else None,
                                   pa.data_ptr() if pa is not None else None, prow, _dt(x), _stream_ptr(x))
    _lib.check(rc, "vig_layernorm_fwd")
    return y


def split_heads(qkv: torch.Tensor, num_heads: int, head_qk_dim: int, head_v_dim: int):
    """qkv [B, L, H*Dk | H*Dk | H*Dv] -> q, k [B,H,L,Dk], v [B,H,L,Dv] (vig.py:401-409).
    qkv may be a block of columns of a wider [B, L, W] tensor (it is read in place).
    Differentiable (vig_split_heads_bwd) when autograd is recording and qkv requires grad."""
    if torch.is_grad_enabled() and qkv.requires_grad:
        return _SplitHeadsFunction.apply(qkv, num_heads, head_qk_dim, head_v_dim)
    return _split_heads_raw(qkv, num_heads, head_qk_dim, head_v_dim)


class _SplitHeadsFunction(torch.autograd.Function):
    """Autograd node of the head split: the backward gathers dq, dk, dv into token-major rows in one pass."""

    @staticmethod
    def forward(ctx, qkv, H, Dk, Dv):
        ctx.dims = (H, Dk, Dv)
        return _split_heads_raw(qkv, H, Dk, Dv)

    @staticmethod
    def backward(ctx, dq, dk, dv):
        lib = _lib.load()
        H, Dk, Dv = ctx.dims
        dq, dk, dv = _dense(dq), _dense(dk), _dense(dv)
        B, _, L, _ = dq.shape
        d_qkv = torch.empty(B, L, H * (2 * Dk + Dv), dtype=dq.dtype, device=dq.device)
        with torch.cuda.device(dq.device):
            rc = lib.vig_split_heads_bwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), d_qkv.data_ptr(), B, L, H, Dk,
                                         Dv, _dt(dq), _stream_ptr(dq))
        _lib.check(rc, "vig_split_heads_bwd")
        return d_qkv, None, None, None


def _split_heads_raw(qkv, num_heads, head_qk_dim, head_v_dim):
    lib = _lib.load()
    _check_cuda(qkv)
    qkv, ld = _token_rows(qkv)
    B, L, W = qkv.shape
    H = num_heads
    if W != H * (2 * head_qk_dim + head_v_dim):
        raise ValueError("last dimension must be H*(2*Dk+Dv)")
    q = torch.empty(B, H, L, head_qk_dim, dtype=qkv.dtype, device=qkv.device)
    k = torch.empty_like(q)
    v = torch.empty(B, H, L, head_v_dim, dtype=qkv.dtype, device=qkv.device)
    with torch.cuda.device(qkv.device):
        rc = lib.vig_split_heads_fwd(qkv.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), B, L, H, head_qk_dim,
                                     head_v_dim, ld, _dt(qkv), _stream_ptr(qkv))
    _lib.check(rc, "vig_split_heads_fwd")
    return q, k, v


def pack_patch_conv_weight(weight: torch.Tensor) -> torch.Tensor:
    """[Cout, Cin, KH, KW] -> [Cout, Cin*KH, 16]: kernel rows zero-padded to the 16 columns vig_patch_conv_fwd reads."""
    Cout, Cin, KH, KW = weight.shape
    if KW > 16:
        raise ValueError("kernel width above 16")
    return torch.nn.functional.pad(weight.detach(), (0, 16 - KW)).reshape(Cout, Cin * KH, 16).contiguous()


def patch_conv_supported(x: torch.Tensor, weight: torch.Tensor, stride: int, padding: int) -> bool:
    """Whether patch_conv takes this convolution (the reference's stem shape in bf16); else use torch's."""
    Cout, Cin, KH, KW = weight.shape
    return (x.dtype == torch.bfloat16 and x.is_cuda and x.dim() == 4 and stride == 8 and padding == 1 and KW <= 16
            and Cin * KH == 27 and x.shape[1] == Cin and x.shape[3] % 8 == 0 and x.shape[3] <= 248
            and Cout % 32 == 0 and 64 <= Cout <= 256 and (x.shape[3] + 2 - KW) // 8 + 1 <= 32)


def patch_conv(x: torch.Tensor, w_packed: torch.Tensor, kernel_hw, stride: int = 8, padding: int = 1) -> torch.Tensor:
    """x [B, Cin, H, W] bf16 -> [B, OH, OW, Cout] (channels-last rows) = conv2d without bias (vig.py:651);
    w_packed from pack_patch_conv_weight."""
    lib = _lib.load()
    _check_cuda(x, w_packed)
    x = _dense(x)
    B, Cin, H, W = x.shape
    KH, KW = kernel_hw
    Cout = w_packed.shape[0]
    if (w_packed.shape != (Cout, Cin * KH, 16) or w_packed.dtype != x.dtype or not w_packed.is_contiguous()
            or w_packed.data_ptr() % 16):
        raise ValueError("w_packed must be the contiguous [Cout, Cin*KH, 16] tensor of pack_patch_conv_weight, in x's dtype")
    OH, OW = (H + 2 * padding - KH) // stride + 1, (W + 2 * padding - KW) // stride + 1
    y = torch.empty(B, OH, OW, Cout, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.vig_patch_conv_fwd(x.data_ptr(), w_packed.data_ptr(), y.data_ptr(), B, Cin, H, W, KH, KW, stride,
                                    padding, Cout, _dt(x), _stream_ptr(x))
    _lib.check(rc, "vig_patch_conv_fwd")
    return y


def linear_swiglu_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether linear_swiglu takes this layer (bf16 on the GPU, contraction 384 or 192, 32-aligned halves)."""
    return (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] in (384, 192) and x.shape[-1] == weight.shape[1] and weight.shape[0] % 64 == 0)


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """swiglu(x @ weight.T) with weight [2*I, K] = (gate rows | up rows): gate_proj and the SwiGLU product
    (vig.py:492-495) in one kernel, no [.., 2*I] intermediate."""
    lib = _lib.load()
    _check_cuda(x, weight)
    x = _dense(x)
    w = _dense(weight.detach())
    K, I = w.shape[1], w.shape[0] // 2
    y = torch.empty(*x.shape[:-1], I, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.vig_linear_swiglu_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), x.numel() // K, K, I, _dt(x),
                                       _stream_ptr(x))
    _lib.check(rc, "vig_linear_swiglu_fwd")
    return y


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """gate_up [..., 2*I] = (gate | up) -> gate * up / (1 + exp(-gate))  (fla/modules/activations.py:109-113).
    Differentiable (vig_swiglu_bwd) when autograd is recording and gate_up requires grad."""
    if torch.is_grad_enabled() and gate_up.requires_grad:
        return _SwiGLUFunction.apply(gate_up)
    return _swiglu_raw(gate_up)


class _SwiGLUFunction(torch.autograd.Function):
    """Autograd node of the SwiGLU product (SwiGLUFunction, fla/modules/activations.py:137-148)."""

    @staticmethod
    def forward(ctx, gate_up):
        gate_up = _dense(gate_up)
        ctx.save_for_backward(gate_up)
        return _swiglu_raw(gate_up)

    @staticmethod
    def backward(ctx, dy):
        (gate_up,) = ctx.saved_tensors
        lib = _lib.load()
        dy = _dense(dy)
        I = gate_up.shape[-1] // 2
        rows = gate_up.numel() // (2 * I)
        d_in = torch.empty_like(gate_up)
        with torch.cuda.device(gate_up.device):
            rc = lib.vig_swiglu_bwd(gate_up.data_ptr(), dy.data_ptr(), d_in.data_ptr(), rows, I, _dt(gate_up),
                                    _stream_ptr(gate_up))
        _lib.check(rc, "vig_swiglu_bwd")
        return d_in


def _swiglu_raw(gate_up: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    _check_cuda(gate_up)
    gate_up = _dense(gate_up)
    I = gate_up.shape[-1] // 2
    rows = gate_up.numel() // (2 * I)
    out = torch.empty(*gate_up.shape[:-1], I, dtype=gate_up.dtype, device=gate_up.device)
    with torch.cuda.device(gate_up.device):
        rc = lib.vig_swiglu_fwd(gate_up.data_ptr(), out.data_ptr(), rows, I, _dt(gate_up), _stream_ptr(gate_up))
    _lib.check(rc, "vig_swiglu_fwd")
    return out
