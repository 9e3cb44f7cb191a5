"""CPU restatement (float64 torch) of the ViG eval-mode forward, for logits checks.

TEST INFRASTRUCTURE ONLY (see gla_oracle.py).  It consumes a state_dict with the reference's
parameter names and follows the eval branch of the reference model:
  classification/models/vig.py:427-463  (GatedLinearAttention, eval path: natural-order gates,
      bid_fused_recurrent_gla -> (o_f+o_b)/2, then o /= 2, RMS norms, sigmoid blend, out_act, o_proj)
  classification/models/vig.py:582-618  (GLABlock: attn_norm, residual add + mlp_norm with prenorm, MLP, residual)
  classification/models/vig.py:469-497  (GLAMLP, swiglu = silu(gate) * y)
  classification/models/vig.py:625-672  (V2PatchEmbed), :843-912 (forward_features, avgpool head)
  flash-linear-attention/fla/modules/rmsnorm.py:38-52 (RMS norm formula)
The reference cannot be imported here (missing timm / causal_conv1d / Triton-only modules) and ships no
golden logits.  Pinning: each primitive (conv2d, linear, logsigmoid, the GLA recurrence) is pinned in
tests/test_oracle.py; the composition (op order, which norm takes which branch and weight, the channel map
of 'b (h d) l -> b l h d', the second halving in front of g_norm, the un-normalised residual, the prenorm
MLP input, row-major token order, pooling and head) by tests/test_oracle_model.py through special cases
whose answers do not need the composed formula: saturated blend gates, zeroed output projections, eps = 0
scale invariance against eps > 0 on small outputs, channel-constant biases in the stem, a single hot cell.
What stays unpinned is only what no arithmetic check can reach: that the published checkpoints' keys mean
what classification/models/vig.py says they mean (no weights are available offline).
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

from . import gla_oracle as O


def _rms(x, w, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def _ln2d(x, w, b, eps=1e-5):
    return F.layer_norm(x.permute(0, 2, 3, 1), (x.shape[1],), w, b, eps).permute(0, 3, 1, 2)


def bidir_gla_torch(q, k, v, gf, gb, scale=None, out_scale=1.0):
    """The bidirectional GLA as its unrolled double sum (the closed form of naive.py:33-41,48-56), in differentiable
    torch operations: autograd through it gives the gradients the training path is checked against.  [B, H, L, D]
    float64 tensors, moderate gate sums only (the decays are factored as e^{G_i} e^{-G_j}).  The forward is pinned
    against the token recurrence in tests/test_oracle.py."""
    L = q.shape[2]
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    G = torch.cumsum(gf, dim=2)                                  # inclusive prefix sums: decay j -> i (j <= i) = G_i - G_j
    Hs = torch.flip(torch.cumsum(torch.flip(gb, [2]), 2), [2])   # inclusive suffix sums: decay j -> i (j >= i) = H_i - H_j
    lower = torch.tril(torch.ones(L, L, dtype=q.dtype))
    a_f = torch.einsum("bhid,bhjd->bhij", q * torch.exp(G), k * torch.exp(-G)) * lower
    a_b = torch.einsum("bhid,bhjd->bhij", q * torch.exp(Hs), k * torch.exp(-Hs)) * lower.T
    return out_scale * scale * torch.einsum("bhij,bhjd->bhid", a_f + a_b, v)


def gla_block_attn(sd, pre, x, hw, num_heads, eps=1e-6, act_in_conv=False, out_act=False, normalizer=16.0,
                   second_halving=True, differentiable=False):
    """Eval-mode GatedLinearAttention.forward on x [B, L, C] (float64).  second_halving=False gives HierViG's
    GLA2D (classification/models/vig_h.py:536-606), whose `o /= 2` after the op is commented out (:579), and the
    training branch (vig.py:425-426: one average of the two directions).  differentiable=True runs the GLA as
    bidir_gla_torch, so that autograd reaches x and the parameters."""
    B, L, C = x.shape
    h, w = hw
    x2 = x.reshape(B, h, w, C).permute(0, 3, 1, 2)
    bias = sd.get(pre + "in_proj.0.bias")
    local = F.conv2d(x2, sd[pre + "in_proj.0.weight"], bias, padding=1, groups=C).flatten(2)  # [B, C, L]
    if act_in_conv:
        local = F.silu(local)
    xs = local.permute(0, 2, 1)
    qkv = xs @ sd[pre + "qkv_proj.weight"].T
    value_dim = sd[pre + "o_proj.weight"].shape[1]
    key_dim = (qkv.shape[-1] - value_dim) // 2
    q, k, v = torch.split(qkv, [key_dim, key_dim, value_dim], dim=2)
    gk = (xs @ sd[pre + "gk_proj.0.weight"].T) @ sd[pre + "gk_proj.1.weight"].T + sd[pre + "gk_proj.1.bias"]
    fw, bw = gk.chunk(2, dim=2)
    H = num_heads
    heads = lambda t: t.reshape(B, L, H, -1).permute(0, 2, 1, 3)
    gf = F.logsigmoid(heads(fw)) / normalizer
    gb = F.logsigmoid(heads(bw)) / normalizer
    if differentiable:
        o = bidir_gla_torch(heads(q), heads(k), heads(v), gf, gb, out_scale=0.5)
    else:
        o = O.bidir_gla_recurrent(heads(q).numpy(), heads(k).numpy(), heads(v).numpy(), gf.numpy(), gb.numpy(),
                                  out_scale=0.5)
        o = torch.from_numpy(o)
    if second_halving:
        o = o / 2  # the second halving of the eval path (vig.py:443)
    o = o.permute(0, 2, 1, 3)  # b l h d
    Dv = value_dim // H
    loc = local.reshape(B, H, Dv, L).permute(0, 3, 1, 2)  # 'b (h d) l -> b l h d'
    loc = _rms(loc, sd[pre + "l_norm.weight"], eps)
    o = _rms(o, sd[pre + "g_norm.weight"], eps)
    g = torch.sigmoid(xs @ sd[pre + "g_proj.weight"].T + sd[pre + "g_proj.bias"]).reshape(B, L, H, Dv)
    y = (o * g + loc * (1 - g)).reshape(B, L, H * Dv)
    if out_act:
        y = F.silu(y)
    return y @ sd[pre + "o_proj.weight"].T


def vig_forward(state_dict, images, num_heads, depth, eps=1e-6, act_in_conv=False, out_act=False, train=False):
    """Logits [B, num_classes] of the eval-mode ViG (v2 patch embedding, no class token, avgpool head).
    train=True follows the training branch instead (directions averaged once) and stays differentiable: the caller
    passes float64 CPU leaf tensors and reads their .grad after a backward."""
    sd = state_dict if train else {k: v.detach().double().cpu() for k, v in state_dict.items()}
    x = images.double().cpu()
    pe = "patch_embed.proj."
    x = F.conv2d(x, sd[pe + "0.weight"], sd.get(pe + "0.bias"), stride=sd[pe + "0.weight"].shape[-1] - 1, padding=1)
    x = F.silu(_ln2d(x, sd[pe + "1.weight"], sd[pe + "1.bias"]))
    x = F.conv2d(x, sd[pe + "3.weight"], sd.get(pe + "3.bias"), stride=2, padding=1)
    x = _ln2d(x, sd[pe + "4.weight"], sd[pe + "4.bias"])
    hw = tuple(x.shape[-2:])
    x = x.flatten(2).transpose(1, 2)
    x = x + sd["pos_embed"]  # same grid as the table (no resize in this restatement)
    for i in range(depth):
        p = f"blocks.{i}."
        residual = x
        hsn = _rms(x, sd[p + "attn_norm.weight"], eps)
        a = gla_block_attn(sd, p + "attn.", hsn, hw, num_heads, eps, act_in_conv, out_act,
                           second_halving=not train, differentiable=train)
        residual = a + residual
        hn = _rms(residual, sd[p + "mlp_norm.weight"], eps)
        gate, y = (hn @ sd[p + "mlp.gate_proj.weight"].T).chunk(2, -1)
        x = residual + (F.silu(gate) * y) @ sd[p + "mlp.down_proj.weight"].T
    x = _rms(x, sd["norm.weight"], eps)
    feat = x.mean(dim=1)
    return feat @ sd["head.weight"].T + sd["head.bias"]
