"""Pins the two composed restatements of the oracle that no reference fixture covers (no GPU):

  * locality_sigmoid_gate_reference (the sigmoid locality gate of the ViG-B benchmark shape), against the library
    convolution on an explicitly rearranged tensor and against an index-by-index brute force;
  * oracle/vig_model_ref.py (eval-mode block and model forward, classification/models/vig.py:427-463,582-608,
    625-672,843-912), by special cases whose answers the mathematics fixes without running the composed formula:
    saturated blend gates, zeroed output projections, the eps = 0 scale invariance of the head norms, spatially
    constant inputs, a single hot token.

Each case is chosen so that one plausible slip in the restatement (a swapped (h, d) channel map, the two norms or
their weights exchanged, the blend taken before the norm, the second halving after instead of before the norm, the
residual taken after the norm instead of before, a transposed token grid) fails it.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gla_oracle as O
from oracle import vig_model_ref as M

torch.manual_seed(0)


# ---------------------------------------------------------------------------------------------------------------
# locality_sigmoid_gate_reference
# ---------------------------------------------------------------------------------------------------------------

def test_sigmoid_locality_gate_against_library_conv(rng):
    B, H, D, h, w = 2, 3, 4, 5, 6
    L, C = h * w, H * D
    o = rng.standard_normal((B, H, L, D))
    wt = rng.standard_normal((C, 1, 3, 3)) / 3
    got = O.locality_sigmoid_gate_reference(o, wt, (h, w))
    # the same thing written with tensor rearrangements and the library convolution: channel c = head * D + d,
    # channel-first image [B, C, h, w] with token l = y * w + x
    ot = torch.from_numpy(o)
    img = ot.permute(0, 1, 3, 2).reshape(B, C, h, w)
    gate = torch.sigmoid(F.conv2d(img, torch.from_numpy(wt), padding=1, groups=C))
    want = (img * gate).reshape(B, H, D, L).permute(0, 1, 3, 2).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-13)


def test_sigmoid_locality_gate_bruteforce_indices(rng):
    # 3 x 4 grid (not square: a transposed grid fails), H != D (a swapped (h, d) channel map fails)
    B, H, D, h, w = 1, 2, 3, 3, 4
    o = rng.standard_normal((B, H, h * w, D))
    wt = rng.standard_normal((H * D, 3, 3))
    got = O.locality_sigmoid_gate_reference(o, wt, (h, w))
    for hd in range(H):
        for d in range(D):
            c = hd * D + d
            for y in range(h):
                for x in range(w):
                    acc = 0.0
                    for di in (-1, 0, 1):
                        for dj in (-1, 0, 1):
                            yy, xx = y + di, x + dj
                            if 0 <= yy < h and 0 <= xx < w:
                                acc += wt[c, di + 1, dj + 1] * o[0, hd, yy * w + xx, d]
                    want = o[0, hd, y * w + x, d] / (1.0 + np.exp(-acc))
                    assert abs(got[0, hd, y * w + x, d] - want) < 1e-13


def test_sigmoid_locality_gate_special_weights(rng):
    B, H, D, h, w = 1, 2, 2, 4, 3
    o = rng.standard_normal((B, H, h * w, D))
    zero = np.zeros((H * D, 3, 3))
    np.testing.assert_allclose(O.locality_sigmoid_gate_reference(o, zero, (h, w)), 0.5 * o, rtol=1e-14)
    centre = zero.copy()
    centre[:, 1, 1] = 1.0  # conv = identity: y = o * sigmoid(o)
    np.testing.assert_allclose(O.locality_sigmoid_gate_reference(o, centre, (h, w)), o / (1 + np.exp(-o)), rtol=1e-13)
    right = zero.copy()
    right[:, 1, 2] = 50.0  # tap (0, +1): the gate opens where the right-hand neighbour is positive, 0.5 at the last column
    y = O.locality_sigmoid_gate_reference(o, right, (h, w))
    img = o.reshape(B, H, h, w, D)
    want = np.empty_like(img)
    want[:, :, :, :-1] = img[:, :, :, :-1] / (1 + np.exp(-50.0 * img[:, :, :, 1:]))
    want[:, :, :, -1] = 0.5 * img[:, :, :, -1]
    np.testing.assert_allclose(y.reshape(img.shape), want, rtol=1e-12, atol=1e-300)


# ---------------------------------------------------------------------------------------------------------------
# the composed block and model forward
# ---------------------------------------------------------------------------------------------------------------

def _block_sd(C, H, pre="", key_ratio=0.5, rank=4, conv_bias=False, gen=None):
    g = gen or torch.Generator().manual_seed(7)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    Kd = int(C * key_ratio)
    sd = {
        pre + "in_proj.0.weight": r(C, 1, 3, 3) / 3,
        pre + "qkv_proj.weight": r(2 * Kd + C, C) / C ** 0.5,
        pre + "gk_proj.0.weight": r(rank, C) / C ** 0.5,
        pre + "gk_proj.1.weight": r(2 * Kd, rank),
        pre + "gk_proj.1.bias": r(2 * Kd),
        pre + "g_proj.weight": r(C, C) / C ** 0.5,
        pre + "g_proj.bias": r(C),
        pre + "o_proj.weight": r(C, C) / C ** 0.5,
        pre + "g_norm.weight": 1 + 0.3 * r(C // H),
        pre + "l_norm.weight": 1 + 0.3 * r(C // H),
    }
    if conv_bias:
        sd[pre + "in_proj.0.bias"] = r(C)
    return sd


def _gla_inputs_of_block(sd, x, hw, H):
    """q, k, v, g_fwd, g_bwd [B, H, L, D] as the block hands them to the op, from library routines only."""
    B, L, C = x.shape
    img = x.reshape(B, hw[0], hw[1], C).permute(0, 3, 1, 2)
    local = F.conv2d(img, sd["in_proj.0.weight"], sd.get("in_proj.0.bias"), padding=1, groups=C)  # [B, C, h, w]
    xs = local.flatten(2).transpose(1, 2)
    Kd = (sd["qkv_proj.weight"].shape[0] - C) // 2
    qkv = F.linear(xs, sd["qkv_proj.weight"])
    heads = lambda t: t.reshape(B, L, H, -1).transpose(1, 2)
    q, k, v = heads(qkv[..., :Kd]), heads(qkv[..., Kd:2 * Kd]), heads(qkv[..., 2 * Kd:])
    gk = F.linear(F.linear(xs, sd["gk_proj.0.weight"]), sd["gk_proj.1.weight"], sd["gk_proj.1.bias"])
    gf, gb = heads(F.logsigmoid(gk[..., :Kd]) / 16), heads(F.logsigmoid(gk[..., Kd:]) / 16)
    return local, xs, q, k, v, gf, gb


@pytest.mark.parametrize("conv_bias", [False, True])
def test_block_saturated_gate_selects_one_branch(conv_bias):
    """g_proj.bias = +40: sigmoid = 1 to 1e-17, the block is o_proj(RMSNorm_g(o)) whatever l_norm holds;
    g_proj.bias = -40: the block is o_proj(RMSNorm_l(local)) whatever the GLA branch holds (vig.py:447-463)."""
    B, H, C, hw = 2, 2, 8, (3, 4)
    L, Dv, eps = hw[0] * hw[1], C // H, 1e-6
    sd = _block_sd(C, H, conv_bias=conv_bias)
    x = torch.randn(B, L, C, dtype=torch.float64)
    local, xs, q, k, v, gf, gb = _gla_inputs_of_block(sd, x, hw, H)
    rms = lambda t, w: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w

    hi = dict(sd)
    hi["g_proj.bias"] = torch.full((C,), 40.0, dtype=torch.float64)
    hi["g_proj.weight"] = torch.zeros(C, C, dtype=torch.float64)
    got = M.gla_block_attn(hi, "", x, hw, H, eps)
    # the op's eval result is the mean of the directions halved once more (vig.py:442-443): a quarter of the sum
    o = torch.from_numpy(O.bidir_gla_recurrent(*(t.numpy() for t in (q, k, v, gf, gb)), out_scale=0.25))
    want = F.linear(rms(o.transpose(1, 2), sd["g_norm.weight"]).reshape(B, L, C), sd["o_proj.weight"])
    torch.testing.assert_close(got, want, rtol=1e-11, atol=1e-12)
    other = dict(hi)
    other["l_norm.weight"] = torch.randn(Dv, dtype=torch.float64)
    torch.testing.assert_close(M.gla_block_attn(other, "", x, hw, H, eps), got, rtol=0, atol=1e-14)

    lo = dict(sd)
    lo["g_proj.bias"] = torch.full((C,), -40.0, dtype=torch.float64)
    lo["g_proj.weight"] = torch.zeros(C, C, dtype=torch.float64)
    got = M.gla_block_attn(lo, "", x, hw, H, eps)
    # 'b (h d) l -> b l h d': channel c of the convolution output is (head c // Dv, d = c % Dv)
    loc = local.flatten(2).reshape(B, H, Dv, L).permute(0, 3, 1, 2)
    want = F.linear(rms(loc, sd["l_norm.weight"]).reshape(B, L, C), sd["o_proj.weight"])
    torch.testing.assert_close(got, want, rtol=1e-11, atol=1e-12)
    other = dict(lo)
    other["g_norm.weight"] = torch.randn(Dv, dtype=torch.float64)
    other["qkv_proj.weight"] = torch.randn_like(sd["qkv_proj.weight"])
    torch.testing.assert_close(M.gla_block_attn(other, "", x, hw, H, eps), got, rtol=0, atol=1e-14)


def test_block_blend_is_convex_in_the_gate():
    """With g_proj.weight = 0 the gate is the constant sigmoid(bias) per channel, so the block output is the
    bias-weighted mix of the two saturated answers, channel by channel, before o_proj."""
    B, H, C, hw = 1, 2, 8, (4, 3)
    L = hw[0] * hw[1]
    sd = _block_sd(C, H)
    sd["g_proj.weight"] = torch.zeros(C, C, dtype=torch.float64)
    sd["o_proj.weight"] = torch.eye(C, dtype=torch.float64)
    x = torch.randn(B, L, C, dtype=torch.float64)
    branch = {}
    for name, b in (("o", 40.0), ("l", -40.0)):
        s = dict(sd)
        s["g_proj.bias"] = torch.full((C,), b, dtype=torch.float64)
        branch[name] = M.gla_block_attn(s, "", x, hw, H)
    gam = torch.sigmoid(sd["g_proj.bias"])
    want = branch["o"] * gam + branch["l"] * (1 - gam)
    torch.testing.assert_close(M.gla_block_attn(sd, "", x, hw, H), want, rtol=1e-12, atol=1e-13)


def test_second_halving_sits_in_front_of_the_head_norm():
    """vig.py:443 halves the op's output BEFORE g_norm.  An RMS norm with eps = 0 is scale invariant, so there the
    halving cancels exactly; with eps > 0 and a small GLA output it does not, by the factor the formula gives."""
    B, H, C, hw = 1, 2, 8, (3, 3)
    L, Dv = 9, 4
    sd = _block_sd(C, H)
    sd["g_proj.weight"] = torch.zeros(C, C, dtype=torch.float64)
    sd["g_proj.bias"] = torch.full((C,), 40.0, dtype=torch.float64)
    sd["o_proj.weight"] = torch.eye(C, dtype=torch.float64)
    x = torch.randn(B, L, C, dtype=torch.float64)
    a = M.gla_block_attn(sd, "", x, hw, H, eps=0.0, second_halving=True)
    b = M.gla_block_attn(sd, "", x, hw, H, eps=0.0, second_halving=False)
    torch.testing.assert_close(a, b, rtol=1e-13, atol=1e-14)
    # small outputs: values scaled by 1e-3 make mean(o^2) comparable to eps
    small = dict(sd)
    small["qkv_proj.weight"] = sd["qkv_proj.weight"].clone()
    small["qkv_proj.weight"][-C:] *= 1e-3
    eps = 1e-6
    a = M.gla_block_attn(small, "", x, hw, H, eps=eps, second_halving=True)
    b = M.gla_block_attn(small, "", x, hw, H, eps=eps, second_halving=False)
    assert (a - b).abs().max() > 1e-2 * b.abs().max()
    # exact relation: with m = mean(o_half^2) per (token, head),  a = b * 0.5 * sqrt((m + eps) / (m / 4 + eps))
    _, _, q, k, v, gf, gb = _gla_inputs_of_block(small, x, hw, H)
    o_half = torch.from_numpy(O.bidir_gla_recurrent(*(t.numpy() for t in (q, k, v, gf, gb)), out_scale=0.5))
    m = (o_half * o_half).mean(-1, keepdim=True).transpose(1, 2)  # [B, L, H, 1]
    ratio = 0.5 * torch.sqrt((m + eps) / (m / 4 + eps))
    torch.testing.assert_close(a.reshape(B, L, H, Dv), b.reshape(B, L, H, Dv) * ratio, rtol=1e-11, atol=1e-14)


def _model_sd(C=8, H=2, depth=2, grid=(3, 4), classes=5, seed=3):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    sd = {
        "patch_embed.proj.0.weight": r(C // 2, 3, 5, 5) / 5, "patch_embed.proj.0.bias": r(C // 2),
        "patch_embed.proj.1.weight": 1 + 0.2 * r(C // 2), "patch_embed.proj.1.bias": r(C // 2),
        "patch_embed.proj.3.weight": r(C, C // 2, 3, 3) / 3, "patch_embed.proj.3.bias": r(C),
        "patch_embed.proj.4.weight": 1 + 0.2 * r(C), "patch_embed.proj.4.bias": r(C),
        "pos_embed": 0.1 * r(1, grid[0] * grid[1], C),
        "norm.weight": 1 + 0.2 * r(C), "head.weight": r(classes, C), "head.bias": r(classes),
    }
    for i in range(depth):
        p = f"blocks.{i}."
        sd.update(_block_sd(C, H, p + "attn.", gen=g))
        sd[p + "attn_norm.weight"] = 1 + 0.2 * r(C)
        sd[p + "mlp_norm.weight"] = 1 + 0.2 * r(C)
        sd[p + "mlp.gate_proj.weight"] = r(2 * 12, C) / C ** 0.5
        sd[p + "mlp.down_proj.weight"] = r(C, 12) / 12 ** 0.5
    return sd


def _images(grid, B=2, seed=5):
    # kernel 5 / stride 4 / padding 1 then kernel 3 / stride 2 / padding 1: an (8 gh) x (8 gw) image gives gh x gw tokens
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, 3, 8 * grid[0], 8 * grid[1], generator=g, dtype=torch.float64)


def _patch_tokens(sd, images):
    """The v2 patch embedding from library routines (vig.py:625-672, 858-865): tokens [B, L, C] with the table added."""
    pe = "patch_embed.proj."
    k = sd[pe + "0.weight"].shape[-1]
    x = F.conv2d(images, sd[pe + "0.weight"], sd[pe + "0.bias"], stride=k - 1, padding=1)
    x = F.layer_norm(x.permute(0, 2, 3, 1), (x.shape[1],), sd[pe + "1.weight"], sd[pe + "1.bias"]).permute(0, 3, 1, 2)
    x = F.silu(x)
    x = F.conv2d(x, sd[pe + "3.weight"], sd[pe + "3.bias"], stride=2, padding=1)
    x = F.layer_norm(x.permute(0, 2, 3, 1), (x.shape[1],), sd[pe + "4.weight"], sd[pe + "4.bias"])  # [B, h, w, C]
    return x.flatten(1, 2) + sd["pos_embed"], tuple(x.shape[1:3])


def test_model_with_zeroed_output_projections_is_embedding_plus_head():
    """o_proj = 0 and down_proj = 0 make every block the identity on the residual stream (vig.py:582-608), so the
    logits are head(mean_tokens(RMSNorm(patch tokens + table))) (vig.py:896-904): pins the stem, the final norm, the
    pooling and the head, and that nothing but the two projections feeds the stream."""
    grid = (3, 4)
    sd = _model_sd(grid=grid)
    for i in range(2):
        sd[f"blocks.{i}.attn.o_proj.weight"].zero_()
        sd[f"blocks.{i}.mlp.down_proj.weight"].zero_()
    images = _images(grid)
    tokens, hw = _patch_tokens(sd, images)
    assert hw == grid
    eps = 1e-6
    feat = (tokens / torch.sqrt((tokens * tokens).mean(-1, keepdim=True) + eps) * sd["norm.weight"]).mean(1)
    want = F.linear(feat, sd["head.weight"], sd["head.bias"])
    torch.testing.assert_close(M.vig_forward(sd, images, 2, 2, eps), want, rtol=1e-11, atol=1e-12)


def test_model_residual_wiring_one_block():
    """One block, o_proj and down_proj the identity-like maps that expose the wiring: with down_proj = 0 the stream
    after the block is x + attn(RMSNorm_attn(x)) (the residual is the UN-normalised input, vig.py:598-606); with
    o_proj = 0 it is x + mlp(RMSNorm_mlp(x))."""
    grid = (3, 4)
    sd = _model_sd(depth=1, grid=grid)
    images = _images(grid)
    tokens, hw = _patch_tokens(sd, images)
    eps = 1e-6
    rms = lambda t, w: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w
    head = lambda t: F.linear(rms(t, sd["norm.weight"]).mean(1), sd["head.weight"], sd["head.bias"])
    p = "blocks.0."
    a = dict(sd)
    a[p + "mlp.down_proj.weight"] = torch.zeros_like(sd[p + "mlp.down_proj.weight"])
    attn = M.gla_block_attn(sd, p + "attn.", rms(tokens, sd[p + "attn_norm.weight"]), hw, 2, eps)  # pinned above
    torch.testing.assert_close(M.vig_forward(a, images, 2, 1, eps), head(tokens + attn), rtol=1e-11, atol=1e-12)
    b = dict(sd)
    b[p + "attn.o_proj.weight"] = torch.zeros_like(sd[p + "attn.o_proj.weight"])
    hn = rms(tokens, sd[p + "mlp_norm.weight"])
    gate, up = F.linear(hn, sd[p + "mlp.gate_proj.weight"]).chunk(2, -1)
    mlp = F.linear(F.silu(gate) * up, sd[p + "mlp.down_proj.weight"])  # swiglu(gate, y) = silu(gate) * y (vig.py:492-495)
    torch.testing.assert_close(M.vig_forward(b, images, 2, 1, eps), head(tokens + mlp), rtol=1e-11, atol=1e-12)
    # both branches on: the MLP reads the stream AFTER the attention branch was added (prenorm residual)
    res = tokens + attn
    gate, up = F.linear(rms(res, sd[p + "mlp_norm.weight"]), sd[p + "mlp.gate_proj.weight"]).chunk(2, -1)
    want = head(res + F.linear(F.silu(gate) * up, sd[p + "mlp.down_proj.weight"]))
    torch.testing.assert_close(M.vig_forward(sd, images, 2, 1, eps), want, rtol=1e-11, atol=1e-12)


def test_patch_embedding_special_cases():
    """A zero image with a channel-constant first bias leaves LayerNorm 1 at its bias; a zero second convolution with a
    channel-constant bias leaves LayerNorm 2 at its bias: tokens = ln2.bias + table, whatever the image."""
    grid = (2, 3)
    sd = _model_sd(depth=0, grid=grid)
    sd["patch_embed.proj.3.weight"].zero_()
    sd["patch_embed.proj.3.bias"].fill_(0.7)
    images = _images(grid)
    tokens = sd["patch_embed.proj.4.bias"] + sd["pos_embed"]  # [1, L, C]
    eps = 1e-6
    feat = (tokens / torch.sqrt((tokens * tokens).mean(-1, keepdim=True) + eps) * sd["norm.weight"]).mean(1)
    want = F.linear(feat, sd["head.weight"], sd["head.bias"]).expand(images.shape[0], -1)
    torch.testing.assert_close(M.vig_forward(sd, images, 2, 0, eps), want, rtol=1e-11, atol=1e-12)


def test_token_order_is_row_major_over_the_grid():
    """A bump in one 8 x 8 cell of the image may only move the tokens whose receptive field covers it: its own cell
    (y, x) -> token y * w + x and the direct neighbours, not the transposed position x * h + y."""
    grid = (2, 5)
    sd = _model_sd(depth=0, grid=grid)
    # a table that marks one token: the head reads sum over tokens of rms(token) -- compare against the library stem
    images = torch.zeros(1, 3, 8 * grid[0], 8 * grid[1], dtype=torch.float64)
    base, _ = _patch_tokens(sd, images)
    y, x = 1, 3
    images[0, :, 8 * y + 3:8 * y + 6, 8 * x + 3:8 * x + 6] = 2.0
    tok, _ = _patch_tokens(sd, images)
    moved = ((tok - base).abs().amax(-1)[0] > 1e-9).nonzero().flatten().tolist()
    assert y * grid[1] + x in moved and all(abs(t // grid[1] - y) <= 1 and abs(t % grid[1] - x) <= 1 for t in moved)
    # and the restatement's logits agree with the library stem under a table that singles tokens out
    sd["pos_embed"] = torch.linspace(-1, 1, grid[0] * grid[1], dtype=torch.float64).reshape(1, -1, 1) * torch.ones(8, dtype=torch.float64)
    tok, _ = _patch_tokens(sd, images)
    eps = 1e-6
    feat = (tok / torch.sqrt((tok * tok).mean(-1, keepdim=True) + eps) * sd["norm.weight"]).mean(1)
    torch.testing.assert_close(M.vig_forward(sd, images, 2, 0, eps), F.linear(feat, sd["head.weight"], sd["head.bias"]),
                               rtol=1e-11, atol=1e-12)
