"""Block- and model-level host side: the reference's module interfaces over the HIP ops.

`GatedLinearAttention` keeps the constructor arguments, forward signature and parameter names of
classification/models/vig.py:241-464, so a reference state_dict loads unchanged.  The three GEMMs
(qkv_proj, gk_proj, g_proj, o_proj) stay in torch (hipBLASLt); everything between them runs in this
package's kernels:
    3x3 depthwise conv on the token grid   -> vig_dwconv3x3_fwd      (vig.py:291-294,428-430)
    direction-wise gate preparation        -> vig_dirgate_fwd        (vig.py:432-441)
    bidirectional GLA                      -> vig_gla_bidir_fwd      (vig.py:442-443)
    RMS-norm x2 + sigmoid blend (+SiLU)    -> vig_locality_blend_fwd (vig.py:444-457)
    split + three head rearranges          -> vig_split_heads_fwd    (vig.py:401-409)
    residual add + RMSNorm (prenorm)       -> vig_rmsnorm_fwd        (rmsnorm.py:69-125; vig.py:598,602-606,896)
    SwiGLU product                         -> vig_swiglu_fwd         (activations.py:109-113; vig.py:492-495)
The surrounding ViG shell (patch embedding, MLP GEMMs, head) is plain torch and follows
vig.py:469-497,530-618,625-672,705-912 for the options the shipped configs use.  There is no CPU path: every
library op raises on tensors that are not on the GPU.

Two ways through every module.  In eval mode, or whenever gradients are not being recorded, the forward runs on the
library's fused inference kernels and leaves no autograd graph.  In training mode with gradients enabled
(`model.train()` outside `torch.no_grad()`) the block records one: the GEMMs and the patch embedding are torch's
differentiable operations, and everything between them -- depthwise conv, head split, gate preparation, the
bidirectional GLA, the norm/blend epilogue, the residual RMS norms and the SwiGLU product -- runs on the library's
kernels in both directions through the autograd nodes of `ops` (the reference's training branch, vig.py:354-426,
with its flips and concatenations folded into the op).
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _ext, ops


def _f32(owner: nn.Module, tag: str, t: Optional[torch.Tensor], shape=None):
    """fp32 contiguous copy of parameter `t` (the kernels take fp32 weights), kept on `owner` under `tag` and refreshed
    when the parameter is replaced, moved, cast or written in place: no conversion kernel per forward."""
    if t is None:
        return None
    key = (t.data_ptr(), t._version, t.dtype, t.device)
    cache = owner.__dict__.setdefault("_f32_cache", {})
    hit = cache.get(tag)
    if hit is None or hit[0] != key:
        v = t.detach().float()
        cache[tag] = hit = (key, (v.reshape(shape) if shape is not None else v).contiguous())
    return hit[1]


_CACHE_ATTRS = ("_f32_cache", "_w32_key", "_w32_cache", "_w1_packed")


def invalidate_caches(model: nn.Module) -> None:
    """Drops the fp32, stacked and packed weight copies every module of `model` keeps for its kernels.  The copies are
    refreshed by themselves when a parameter is replaced, moved, cast or written through torch's in-place operations;
    a write through `.data` (p.data.mul_(..), module.weight.data[...] = ..) changes neither the pointer nor the version
    counter they are keyed on, so code that writes that way calls this afterwards.  load_state_dict and train() /
    eval() switches of these modules call it by themselves."""
    for m in model.modules():
        for a in _CACHE_ATTRS:
            m.__dict__.pop(a, None)
        if "_in_cat" in m.__dict__:
            m.__dict__["_in_cat"] = None


class _CacheMixin:
    """For the modules that keep derived weight copies: the copies do not outlive a state-dict load or a switch
    between training and evaluation (the usual places where weights change behind the version counter)."""

    def train(self, mode: bool = True):
        invalidate_caches(self)
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        invalidate_caches(self)
        return super()._load_from_state_dict(*args, **kwargs)


def _recording(module: nn.Module) -> bool:
    """True when this call has to leave an autograd graph: training mode with gradients enabled."""
    return module.training and torch.is_grad_enabled()


class RMSNorm(_CacheMixin, nn.Module):
    """x * rsqrt(mean(x^2) + eps) * weight, arithmetic in fp32 (fla/modules/rmsnorm.py:38-52,491-512).

    forward(x, residual=None, prenorm=False): with a residual the sum is normalised and, with
    prenorm=True, also returned (rmsnorm.py:94-106) -- the wiring GLABlock relies on.
    """

    def __init__(self, hidden_size: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def _w32(self):
        """fp32 copy of the weight, refreshed when the parameter changes (the kernels take fp32 weights)."""
        w = self.weight
        key = (w.data_ptr(), w._version, w.dtype, w.device)
        if getattr(self, "_w32_key", None) != key:
            self._w32_cache = w.detach().float().contiguous()
            self._w32_key = key
        return self._w32_cache

    def forward(self, x, residual=None, prenorm: bool = False, round_sum: bool = False):
        if _recording(self):  # the op's autograd node: forward and backward on the library's kernels
            if residual is not None and residual.dtype != x.dtype:  # autocast: a bf16 branch meets the fp32 stream
                dt = torch.promote_types(x.dtype, residual.dtype)
                x, residual = x.to(dt), residual.to(dt)
            return ops.rmsnorm(x, self.weight, self.eps, residual=residual, prenorm=prenorm, round_sum=round_sum)
        ext = _ext.load()
        if (ext is not None and x.is_cuda and not _recording(self) and x.is_contiguous()
                and (residual is None or (residual.is_contiguous() and residual.dtype == x.dtype))):
            # (operator library: checks, allocation and launch in one C++ call)
            y, total = ext.rmsnorm_fwd(x, residual, self._w32(), self.eps, round_sum)
            return (y, x if total is None else total) if prenorm else y
        return ops.rmsnorm(x, self._w32(), self.eps, residual=residual, prenorm=prenorm, round_sum=round_sum)


class GatedLinearAttention(_CacheMixin, nn.Module):
    """ViG's bidirectional GLA token mixer (classification/models/vig.py:241-464)."""

    def __init__(self, d_model: int = 1024, expand_v: float = 2.0, expand_k: float = 1.0, num_heads: int = 4,
                 gate_fn: str = "swish", layernorm_eps: float = 1e-5, gate_logit_normalizer: int = 16,
                 gate_low_rank_dim: int = 16, mode: str = "fused_chunk", clamp_min: Optional[float] = None,
                 fuse_norm: bool = True, use_dirpe: bool = False, use_out_act: bool = False,
                 use_out_gate: bool = True, rope_mode: str = "none", use_act_in_conv: bool = True,
                 use_bias_in_dwconv: bool = False, *args, **kwargs):
        super().__init__()
        if mode not in ("chunk", "fused_recurrent", "fused_chunk", "bid_fused_chunk", "bidv2_fused_chunk"):
            raise AssertionError(f"Not suppoerted mode `{mode}`.")
        if rope_mode != "none":
            raise NotImplementedError("rope modes other than 'none' are not used by the shipped ViG configs")
        if use_dirpe:
            raise NotImplementedError("use_dirpe is not used by the shipped ViG configs")
        if gate_fn not in ("swish", "silu"):
            raise NotImplementedError("only the swish/SiLU gate function is built")
        self.d_model = d_model
        self.mode = mode
        self.value_dim = int(d_model * expand_v)
        self.key_dim = int(d_model * expand_k)
        self.clamp_min = clamp_min
        assert self.key_dim % num_heads == 0, f"key dim must be divisible by num_heads of {num_heads}"
        assert self.value_dim % num_heads == 0, f"value dim must be divisible by num_heads of {num_heads}"
        self.num_heads = num_heads
        self.head_qk_dim = self.key_dim // num_heads
        self.head_v_dim = self.value_dim // num_heads
        self.use_out_gate = use_out_gate  # stored, never read (as in the reference, vig.py:285)
        self.use_out_act = use_out_act
        # inference switch (not a parameter of the reference): this layer's gates are known to be strong, so the GLA
        # op starts with its wide-range form (calibrate_strong_gates sets it from a sample batch)
        self.strong_gates = False
        self.use_act_in_conv = use_act_in_conv
        self.layernorm_eps = layernorm_eps
        self.gate_logit_normalizer = gate_logit_normalizer

        self.in_proj = nn.Sequential(
            nn.Conv2d(d_model, d_model, kernel_size=3, padding=1, groups=d_model, bias=use_bias_in_dwconv),
            nn.SiLU() if use_act_in_conv else nn.Identity(),
        )
        self.qkv_proj = nn.Linear(d_model, 2 * self.key_dim + self.value_dim, bias=False)
        self.gk_proj = nn.Sequential(nn.Linear(d_model, gate_low_rank_dim, bias=False),
                                     nn.Linear(gate_low_rank_dim, self.key_dim * 2, bias=True))
        self.o_proj = nn.Linear(self.value_dim, d_model, bias=False)
        self.g_norm = RMSNorm(self.head_v_dim, eps=layernorm_eps)
        self.l_norm = RMSNorm(self.head_v_dim, eps=layernorm_eps)
        self.g_proj = nn.Linear(d_model, self.value_dim, bias=True)
        self._in_cat = None  # (key, weight, bias) of the concatenated input projection, built on first use
        self.reset_parameters()

    def reset_parameters(self):
        gain = 2 ** -2.5
        nn.init.xavier_uniform_(self.qkv_proj.weight, gain=gain)
        nn.init.xavier_uniform_(self.in_proj[0].weight, gain=gain)
        nn.init.xavier_uniform_(self.g_proj.weight, gain=gain)
        nn.init.xavier_uniform_(self.o_proj.weight, gain=gain)
        nn.init.xavier_uniform_(self.gk_proj[0].weight, gain=gain)
        nn.init.xavier_uniform_(self.gk_proj[1].weight, gain=gain)

    def _input_projections(self, xs):
        """qkv_proj, g_proj and the first (low-rank) gk_proj layer all read xs: they run as ONE matrix product with
        the three weights stacked (rows padded with zeros to a multiple of 128, which the GEMM tiles prefer), and the
        consumers read their column blocks of the result in place.  Every output column is the same dot product (and
        bias add) as in the separate layers.  The stacked copy follows the parameters: it is rebuilt when one of them
        is replaced, moved, cast or written in place."""
        w, b = self._stacked_in()
        z = F.linear(xs, w, b)
        n0 = self.qkv_proj.weight.shape[0]
        n1 = n0 + self.value_dim
        return z[..., :n0], z[..., n0:n1], z[..., n1:n1 + self.gk_proj[0].weight.shape[0]]

    def _stacked_in(self):
        """(weight, bias) of the stacked input projection: rows qkv | g | low-rank gate, zero-padded to a multiple of 128."""
        srcs = (self.qkv_proj.weight, self.g_proj.weight, self.g_proj.bias, self.gk_proj[0].weight)
        key = tuple((t.data_ptr(), t._version, t.dtype, t.device) for t in srcs)
        if self._in_cat is None or self._in_cat[0] != key:
            wq, wg, bg, wr = (t.detach() for t in srcs)
            n = wq.shape[0] + wg.shape[0] + wr.shape[0]
            w = wq.new_zeros((n + 127) // 128 * 128, wq.shape[1])
            b = wq.new_zeros(w.shape[0])
            w[:n] = torch.cat((wq, wg, wr), 0)
            b[wq.shape[0]:wq.shape[0] + wg.shape[0]] = bg
            self._in_cat = (key, w, b)
        return self._in_cat[1], self._in_cat[2]

    def _mix(self, x, hw, out_scale):
        """The token mixer on x [B, L, C] with L = h*w tokens in row-major grid order."""
        H = self.num_heads
        conv = self.in_proj[0]
        ext = _ext.load()
        if (ext is not None and x.is_cuda and x.is_contiguous() and self.gk_proj[0].weight.shape[0] == ops.GATE_RANK
                and x.dtype == self.qkv_proj.weight.dtype and not self.strong_gates):
            # the whole mixer as one operator of the library (csrc/torch_ext.cpp: the same kernel sequence as below)
            w_in, b_in = self._stacked_in()
            up = self.gk_proj[1]
            return ext.gla_block_mix(x, hw[0], hw[1], _f32(self, "conv_w_flat", conv.weight, (-1,)),
                                     _f32(self, "conv_b", conv.bias), self.use_act_in_conv, w_in, b_in, H,
                                     self.head_qk_dim, self.head_v_dim, up.weight, up.bias, self.gate_logit_normalizer,
                                     self.clamp_min, self.g_norm._w32(), self.l_norm._w32(), self.layernorm_eps,
                                     self.use_out_act, self.o_proj.weight, out_scale)
        # local_out, already in the [B, L, C] layout the projections consume
        xs = ops.dwconv3x3(x, _f32(self, "conv_w", conv.weight, (-1, 3, 3)), hw, bias=_f32(self, "conv_b", conv.bias),
                           silu=self.use_act_in_conv)
        qkv, g_lin, gk_low = self._input_projections(xs)
        dk, dv = self.head_qk_dim, self.head_v_dim
        if qkv.dtype == torch.bfloat16 and qkv.shape[1] <= 256 and dk in (32, 64) and dv == 64 and qkv.stride(1) % 8 == 0:
            # head-split views of the projection's rows: the matrix-core slab kernel reads them in place
            q, k, v = (t.unflatten(-1, (H, d)).transpose(1, 2)
                       for t, d in zip(qkv.split((H * dk, H * dk, H * dv), -1), (dk, dk, dv)))
        else:
            q, k, v = ops.split_heads(qkv, H, dk, dv)
        up = self.gk_proj[1]
        if gk_low.shape[-1] == ops.GATE_RANK:  # the rank-16 up-projection runs inside the gate kernel
            gates = ops.dirgate_lowrank(gk_low, up.weight, up.bias, H, self.gate_logit_normalizer, self.clamp_min)
        else:
            gates = ops.dirgate(up(gk_low), H, self.gate_logit_normalizer, self.clamp_min)
        self._last_gates = gates if getattr(self, "_keep_gates", False) else None
        o = ops.gla_bidir_forward(q, k, v, gates[0], gates[1], scale=-1, out_scale=out_scale,
                                  strong_gates=self.strong_gates)
        if ops.locality_blend_linear_supported(o, self.o_proj.weight):  # ViG-S / ViG-T widths: no blended intermediate
            return ops.locality_blend_linear(o, xs, g_lin, self.g_norm._w32(), self.l_norm._w32(), self.o_proj.weight,
                                             eps=self.layernorm_eps, silu_out=self.use_out_act)
        y = ops.locality_blend(o, xs, g_lin, self.g_norm._w32(), self.l_norm._w32(),
                               eps=self.layernorm_eps, silu_out=self.use_out_act)
        return self.o_proj(y)

    def _mix_autograd(self, x, hw, out_scale):
        """_mix with an autograd graph (the reference's training branch, vig.py:354-426,444-463: its flipped copies of
        q, k, v and of the backward gates are what the op's second direction reads in place).  The projections are
        torch's differentiable GEMMs; everything between them is the library's kernels both ways, through the ops'
        autograd nodes."""
        H = self.num_heads
        conv = self.in_proj[0]
        if torch.is_autocast_enabled():  # what autocast would hand a convolution
            x = x.to(torch.get_autocast_dtype("cuda"))
        xs = ops.dwconv3x3(x, conv.weight, hw, bias=conv.bias, silu=self.use_act_in_conv)  # differentiable, [B, L, C]
        q, k, v = ops.split_heads(self.qkv_proj(xs), H, self.head_qk_dim, self.head_v_dim)
        gates = ops.dirgate(self.gk_proj(xs), H, self.gate_logit_normalizer, self.clamp_min)
        g_fwd, g_bwd = gates.unbind(0)
        o = ops.gla_bidir_forward(q, k, v, g_fwd, g_bwd, scale=-1, out_scale=out_scale)
        # both head norms, the sigmoid blend and the output activation: one kernel each way
        y = ops.locality_blend(o, xs, self.g_proj(xs), self.g_norm.weight, self.l_norm.weight,
                               eps=self.layernorm_eps, silu_out=self.use_out_act)
        return self.o_proj(y)

    def forward(self, x, lower_bound=0, **kwargs):
        if kwargs.get("token_position", None) is not None:
            raise NotImplementedError("class-token splicing is not built (the shipped configs use IF_CLS_TOKEN False)")
        # training glue averages the directions (vig.py:425-426); the eval path halves twice
        # (recurrent_fuse.py:442, then vig.py:443)
        hw = tuple(kwargs["patch_resolution"])
        if _recording(self):
            return self._mix_autograd(x, hw, 0.5)
        with torch.no_grad():
            return self._mix(x, hw, 0.5 if self.training else 0.25)


def calibrate_strong_gates(model: nn.Module, *sample_inputs, share: float = 0.25, tile: int = 32,
                           limit: float = 6.9) -> dict:
    """Sets `strong_gates` on every GatedLinearAttention of `model` from one eval forward on a sample batch: a layer is
    marked when more than `share` of its (batch, head) sequences hold a 32-token tile whose summed log-gate falls
    below -`limit` in some channel (the range of the GLA kernel's fp16 form: such a sequence is computed twice by the
    default entry point, at about four times the cost, while the wide-range form costs 1.65 times).  Returns
    {module name: share of such sequences}.  One-off: it synchronises and runs the unfused block path."""
    mods = {n: m for n, m in model.named_modules() if isinstance(m, GatedLinearAttention)}
    was_training = model.training
    model.eval()
    saved = {}
    for n, m in mods.items():
        saved[n] = m.strong_gates
        m.strong_gates, m._keep_gates = True, True  # (the unfused path, which exposes the gates)
    out = {}
    try:
        with torch.no_grad():
            model(*sample_inputs)
        for n, m in mods.items():
            g = getattr(m, "_last_gates", None)
            if g is None:
                out[n] = 0.0
                continue
            worst = None
            for gd in (g[0], g[1]):  # [B, H, L, Dk] natural-log gates of one direction
                L = gd.shape[2]
                pad = (-L) % tile
                t = F.pad(gd.float(), (0, 0, 0, pad)).unflatten(2, (-1, tile)).sum(3)  # [B, H, tiles, Dk]
                w = t.amin(dim=(2, 3))
                worst = w if worst is None else torch.minimum(worst, w)
            out[n] = float((worst < -limit).float().mean().item())
    finally:
        for n, m in mods.items():
            m._keep_gates, m._last_gates = False, None
            m.strong_gates = saved[n]
        model.train(was_training)
    for n, m in mods.items():
        m.strong_gates = out[n] > share
    return out


class GLA2D(GatedLinearAttention):
    """HierViG's token mixer (classification/models/vig_h.py:338-606): the same block on a feature map,
    x [B, H, W, C] (or [B, C, H, W] with channel_first), same parameter names (its Linear2d keeps nn.Linear's weight
    shape, vig_h.py:202-209).  Both branches of the reference average the two directions once (training glue
    vig_h.py:531-532; eval bid_fused_recurrent_gla with the second halving commented out, vig_h.py:578-579)."""

    def __init__(self, d_model: int = 1024, expand_v: float = 2.0, expand_k: float = 1.0, num_heads: int = 4,
                 gate_fn: str = "swish", layernorm_eps: float = 1e-5, gate_logit_normalizer: int = 16,
                 gate_low_rank_dim: int = 16, mode: str = "fused_chunk", clamp_min: Optional[float] = None,
                 fuse_norm: bool = True, use_dirpe: bool = False, use_out_act: bool = False,
                 use_act_in_conv: bool = True, rope_mode: str = "none", channel_first: bool = False, *args, **kwargs):
        super().__init__(d_model=d_model, expand_v=expand_v, expand_k=expand_k, num_heads=num_heads, gate_fn=gate_fn,
                         layernorm_eps=layernorm_eps, gate_logit_normalizer=gate_logit_normalizer,
                         gate_low_rank_dim=gate_low_rank_dim, mode=mode, clamp_min=clamp_min, fuse_norm=fuse_norm,
                         use_dirpe=use_dirpe, use_out_act=use_out_act, rope_mode=rope_mode,
                         use_act_in_conv=use_act_in_conv, use_bias_in_dwconv=False)
        self.channel_first = channel_first
        self.d_group = 2

    def forward(self, x, **kwargs):
        if self.channel_first:
            B, C, H, W = x.shape
            x = x.permute(0, 2, 3, 1)
        else:
            B, H, W, C = x.shape
        if _recording(self):
            y = self._mix_autograd(x.reshape(B, H * W, C), (H, W), 0.5)
        else:
            with torch.no_grad():
                y = self._mix(x.reshape(B, H * W, C), (H, W), 0.5)
        if self.channel_first:
            return y.permute(0, 2, 1).reshape(B, -1, H, W)
        return y.reshape(B, H, W, -1)


class GLAMLP(nn.Module):
    """SwiGLU MLP (vig.py:469-497; swiglu = x*sigmoid(x)*y, fla/modules/activations.py:109-113)."""

    def __init__(self, hidden_size: int, hidden_ratio: Optional[int] = None, intermediate_size: Optional[int] = None,
                 hidden_act: str = "swish"):
        super().__init__()
        if hidden_ratio is None:
            hidden_ratio = 4
        if intermediate_size is None:
            intermediate_size = int(hidden_size * hidden_ratio * 2 / 3)
            intermediate_size = 256 * ((intermediate_size + 256 - 1) // 256)
        self.hidden_size, self.hidden_ratio, self.intermediate_size = hidden_size, hidden_ratio, intermediate_size
        self.gate_proj = nn.Linear(hidden_size, intermediate_size * 2, bias=False)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False)

    def forward(self, x):
        if _recording(self):  # the SwiGLU product's autograd node runs on the library's kernels both ways
            return self.down_proj(ops.swiglu(self.gate_proj(x)))
        w = self.gate_proj.weight
        if ops.linear_swiglu_supported(x, w):  # ViG-S / ViG-T widths in bf16: no [.., 2*I] intermediate
            ext = _ext.load()
            if ext is not None and x.is_contiguous():
                return self.down_proj(ext.linear_swiglu_fwd(x, w))
            return self.down_proj(ops.linear_swiglu(x, w))
        return self.down_proj(ops.swiglu(self.gate_proj(x)))


class DropPath(nn.Module):
    """Stochastic depth: in training mode a branch is dropped per sample with probability drop_prob and the kept
    ones are scaled by 1 / (1 - drop_prob); identity otherwise (timm's DropPath as used at vig.py:533,606-608)."""

    def __init__(self, drop_prob: float = 0.0, scale_by_keep: bool = True):
        super().__init__()
        self.drop_prob, self.scale_by_keep = float(drop_prob), scale_by_keep

    def forward(self, x):
        if self.drop_prob == 0.0 or not self.training:
            return x
        keep = 1.0 - self.drop_prob
        mask = x.new_empty((x.shape[0],) + (1,) * (x.dim() - 1)).bernoulli_(keep)
        if keep > 0.0 and self.scale_by_keep:
            mask.div_(keep)
        return x * mask

    def extra_repr(self):
        return f"drop_prob={self.drop_prob:0.3f}"


class GLABlock(nn.Module):
    """attn_norm -> GLA -> (residual add + mlp_norm, prenorm) -> MLP -> residual (vig.py:530-618), no layer scale;
    drop_path is the stochastic-depth rate of both branches (vig.py:533,606-608)."""

    def __init__(self, hidden_size: int, num_heads: int, expand_k: float, expand_v: float, eps: float = 1e-6,
                 use_out_act: bool = False, use_act_in_conv: bool = True, use_bias_in_dwconv: bool = False,
                 intermediate_size: Optional[int] = None, mode: str = "fused_chunk", drop_path: float = 0.0):
        super().__init__()
        self.drop_path = DropPath(drop_path) if drop_path > 0.0 else nn.Identity()
        self.attn_norm = RMSNorm(hidden_size, eps=eps)
        self.attn = GatedLinearAttention(d_model=hidden_size, expand_k=expand_k, expand_v=expand_v,
                                         num_heads=num_heads, layernorm_eps=eps, mode=mode, use_out_act=use_out_act,
                                         use_act_in_conv=use_act_in_conv, use_bias_in_dwconv=use_bias_in_dwconv)
        self.mlp_norm = RMSNorm(hidden_size, eps=eps)
        self.mlp = GLAMLP(hidden_size, intermediate_size=intermediate_size)

    def forward(self, hidden_states, **kwargs):
        residual = hidden_states
        h = self.attn(self.attn_norm(hidden_states), **kwargs)
        h, residual = self.mlp_norm(self.drop_path(h), residual, True)
        return (residual + self.drop_path(self.mlp(h)),)

    def forward_carry(self, branch, residual, **kwargs):
        """Same block, with the closing `residual + mlp(h)` of the previous block folded into this block's first norm:
        takes (branch, residual) with hidden_states = residual + branch and returns the next such pair."""
        ext = _ext.load()
        at = self.attn
        if (ext is not None and not _recording(self) and not self.training and branch.is_cuda and branch.is_contiguous()
                and type(at) is GatedLinearAttention and at.gk_proj[0].weight.shape[0] == ops.GATE_RANK
                and not at.strong_gates
                and branch.dtype == at.qkv_proj.weight.dtype and kwargs.get("token_position", None) is None
                and (residual is None or (residual.is_contiguous() and residual.dtype == branch.dtype))
                # (the operator takes one eps for both norms and the eval-mode output scale)
                and self.mlp_norm.eps == self.attn_norm.eps and not at.training):
            # the whole block as one operator of the library (csrc/torch_ext.cpp: the same kernel sequence as below)
            hw = tuple(kwargs["patch_resolution"])
            conv, up = at.in_proj[0], at.gk_proj[1]
            w_in, b_in = at._stacked_in()
            with torch.no_grad():
                return ext.gla_block_carry(
                    branch, residual, self.attn_norm._w32(), self.attn_norm.eps, hw[0], hw[1],
                    _f32(at, "conv_w_flat", conv.weight, (-1,)), _f32(at, "conv_b", conv.bias), at.use_act_in_conv, w_in,
                    b_in, at.num_heads, at.head_qk_dim, at.head_v_dim, up.weight, up.bias, at.gate_logit_normalizer,
                    at.clamp_min, at.g_norm._w32(), at.l_norm._w32(), at.layernorm_eps, at.use_out_act, at.o_proj.weight,
                    0.25, self.mlp_norm._w32(), self.mlp.gate_proj.weight, self.mlp.down_proj.weight)
        if residual is None:
            h, hidden = self.attn_norm(branch), branch
        else:  # the explicit add stores a rounded sum and attn_norm normalises that (vig.py:598,606)
            h, hidden = self.attn_norm(branch, residual, True, round_sum=True)
        h = self.attn(h, **kwargs)
        h, residual = self.mlp_norm(self.drop_path(h), hidden, True)
        return self.drop_path(self.mlp(h)), residual


class LayerNorm2d(_CacheMixin, nn.LayerNorm):
    """LayerNorm over the channels of a [B, C, H, W] map (vig.py:619-624).  The patch embedding keeps its maps in
    channels-last memory, where the permuted view is a plain [B*H*W, C] row matrix for the row kernel; `silu`
    folds the swish that follows the first norm (vig.py:653) into the same pass."""

    def forward(self, x, silu: bool = False, pre_bias=None, post_add=None):
        rows = x.permute(0, 2, 3, 1)  # a view; contiguous when x is channels-last
        if _recording(self):
            if pre_bias is not None:
                rows = rows + pre_bias.to(rows.dtype)
            y = F.layer_norm(rows, (rows.shape[-1],), self.weight, self.bias, self.eps)
            if silu:
                y = F.silu(y)
            if post_add is not None:
                y = (y.flatten(1, 2) + post_add).reshape(y.shape)
            return y.permute(0, 3, 1, 2)
        return ops.layernorm(rows, _f32(self, "w", self.weight), _f32(self, "b", self.bias), self.eps, silu=silu,
                             pre_bias=pre_bias, post_add=post_add).permute(0, 3, 1, 2)


class V2PatchEmbed(_CacheMixin, nn.Module):
    """Two strided convs with LayerNorm2d (vig.py:625-672), use_act_in_patch False."""

    def __init__(self, patch_size=16, in_chans=3, embed_dim=768, use_bias_in_patch=True):
        super().__init__()
        stride = patch_size // 2
        self.proj = nn.Sequential(
            nn.Conv2d(in_chans, embed_dim // 2, kernel_size=stride + 1, stride=stride, padding=1, bias=use_bias_in_patch),
            LayerNorm2d(embed_dim // 2),
            nn.SiLU(),
            nn.Conv2d(embed_dim // 2, embed_dim, kernel_size=3, stride=2, padding=1, bias=use_bias_in_patch),
            LayerNorm2d(embed_dim),
        ).to(memory_format=torch.channels_last)  # conv weights stored the way the channels-last kernels read them

    def forward(self, x, pos_embed=None, pos_shape=None):
        """pos_embed [1, h*w, C] on the grid pos_shape, if given, is added to the tokens (resized to the actual grid)
        inside the last norm's kernel."""
        # channels-last throughout: the convolutions run in that layout, the norms see row matrices, and the final
        # 'b c h w -> b (h w) c' is a view; each convolution's bias add rides in the norm kernel behind it
        if _recording(self):  # plain modules, differentiable (LayerNorm2d and the convolutions record their graph)
            x = self.proj(x)
            hw = tuple(x.shape[-2:])
            x = x.flatten(2).transpose(1, 2)
            if pos_embed is not None:
                x = x + resize_pos_embed(pos_embed, pos_shape, hw).to(x.dtype)
            return x, hw
        conv1, norm1, act, conv2, norm2 = self.proj
        if (conv1.stride[0] == conv1.stride[1] and conv1.padding[0] == conv1.padding[1] and conv1.groups == 1
                and conv1.dilation == (1, 1)
                and ops.patch_conv_supported(x, conv1.weight, conv1.stride[0], conv1.padding[0])):
            # the stem's shape: the library's implicit-GEMM kernel reads the images as they are and writes rows
            x = ops.patch_conv(x, self._packed_w1(), conv1.kernel_size, conv1.stride[0], conv1.padding[0])
            x = x.permute(0, 3, 1, 2)  # [B, C, H, W] view of channels-last memory
        else:
            x = self._conv_nobias(conv1, x.contiguous(memory_format=torch.channels_last))
        x = norm1(x, silu=isinstance(act, nn.SiLU), pre_bias=_f32(self, "b1", conv1.bias))
        if not isinstance(act, nn.SiLU):
            x = act(x)
        x = self._conv_nobias(conv2, x)
        hw = tuple(x.shape[-2:])
        if pos_embed is not None:
            pos_embed = resize_pos_embed(pos_embed, pos_shape, hw).to(x.dtype)
        x = norm2(x, pre_bias=_f32(self, "b2", conv2.bias), post_add=pos_embed)
        return x.flatten(2).transpose(1, 2), hw

    def _packed_w1(self):
        """The first convolution's weight in the kernel's packed form, rebuilt when the parameter changes."""
        w = self.proj[0].weight
        key = (w.data_ptr(), w._version, w.dtype, w.device)
        hit = self.__dict__.get("_w1_packed")
        if hit is None or hit[0] != key:
            self.__dict__["_w1_packed"] = hit = (key, ops.pack_patch_conv_weight(w))
        return hit[1]

    @staticmethod
    def _conv_nobias(conv, x):
        return F.conv2d(x, conv.weight, None, conv.stride, conv.padding, conv.dilation, conv.groups)


def resize_pos_embed(pos_embed, src_shape, dst_shape):
    """Bicubic resize of a [1, h*w, C] table (vig.py:915-958), no extra tokens."""
    if tuple(src_shape) == tuple(dst_shape):
        return pos_embed
    _, L, C = pos_embed.shape
    w = pos_embed.reshape(1, src_shape[0], src_shape[1], C).permute(0, 3, 1, 2)
    w = F.interpolate(w.float(), size=dst_shape, align_corners=False, mode="bicubic")
    return torch.flatten(w, 2).transpose(1, 2).to(pos_embed.dtype)


class ViG(nn.Module):
    """Non-hierarchical ViG with the options of the shipped vig-{t,s,b}.yaml (vig.py:705-912): v2 patch embedding,
    absolute position table, no class token, SwiGLU MLP, average-pool head."""

    def __init__(self, img_size=224, patch_size=16, depth=12, num_heads=6, embed_dim=384, channels=3,
                 num_classes=1000, expand_k=0.5, expand_v=1.0, use_out_act=False, use_act_in_conv=False,
                 use_bias_in_dwconv=False, rms_norm_eps=1e-6, initializer_range=0.02, drop_path_rate=0.1):
        super().__init__()
        self.embed_dim = embed_dim
        dpr = [x.item() for x in torch.linspace(0, drop_path_rate, depth)]  # stochastic depth decay rule (vig.py:805)
        self.patch_embed = V2PatchEmbed(patch_size=patch_size, in_chans=channels, embed_dim=embed_dim)
        self.patch_resolution = (img_size // patch_size, img_size // patch_size)
        self.pos_embed = nn.Parameter(torch.zeros(1, self.patch_resolution[0] * self.patch_resolution[1], embed_dim))
        self.head = nn.Linear(embed_dim, num_classes)
        self.blocks = nn.ModuleList([
            GLABlock(embed_dim, num_heads, expand_k, expand_v, eps=rms_norm_eps, use_out_act=use_out_act,
                     use_act_in_conv=use_act_in_conv, use_bias_in_dwconv=use_bias_in_dwconv, drop_path=dpr[i])
            for i in range(depth)])
        self.norm = RMSNorm(embed_dim, eps=rms_norm_eps)
        # init order of the reference (vig.py:825-837,332-349): every Linear N(0, 0.02) with zero bias, then the
        # GLA projections xavier-uniform with gain 2^-2.5; convs of the patch embedding keep torch's default
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, mean=0.0, std=initializer_range)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
        for m in self.modules():
            if isinstance(m, GatedLinearAttention):
                m.reset_parameters()
        nn.init.trunc_normal_(self.pos_embed, std=0.02)

    def forward_features(self, x):
        B = x.shape[0]
        x, hw = self.patch_embed(x, self.pos_embed, self.patch_resolution)
        branch, residual = x, None
        for blk in self.blocks:
            branch, residual = blk.forward_carry(branch, residual, patch_resolution=hw, token_position=None)
        x = self.norm(branch, residual, round_sum=True) if residual is not None else self.norm(branch)
        return x.reshape(B, hw[0] * hw[1], -1).mean(dim=1)

    def forward(self, x):
        if _recording(self):
            return self.head(self.forward_features(x))
        with torch.no_grad():
            return self.head(self.forward_features(x))


def vig_small(**kw):
    """vig-s.yaml: dim 384, 6 heads (Dk 32, Dv 64), depth 12, drop-path rate 0.2."""
    kw.setdefault("drop_path_rate", 0.2)
    return ViG(depth=12, num_heads=6, embed_dim=384, use_out_act=False, use_act_in_conv=False, **kw)


def vig_tiny(**kw):
    """vig-t.yaml: dim 192, 3 heads, depth 12, SiLU after the dwconv and on the blend output."""
    return ViG(depth=12, num_heads=3, embed_dim=192, use_out_act=True, use_act_in_conv=True, **kw)


def vig_base(**kw):
    """vig-b.yaml: dim 768, 12 heads, depth 12, drop-path rate 0.5."""
    kw.setdefault("drop_path_rate", 0.5)
    return ViG(depth=12, num_heads=12, embed_dim=768, use_out_act=False, use_act_in_conv=False, **kw)
