"""The differentiable (training-mode) path of the block and the model: outputs against the kernel path, gradients
against autograd through the float64 CPU restatement (whose GLA is pinned in tests/test_oracle.py)."""
import numpy as np
import pytest
import torch

from oracle import vig_model_ref as R
from vig_amd import layers

from .util import announce

pytestmark = pytest.mark.gpu

VARIANTS = {
    # name: (d_model, heads, block options) -- head shapes Dk 32 / Dv 64 and Dk 16 / Dv 32
    "s": (128, 2, dict(use_act_in_conv=False, use_out_act=False)),
    "t": (96, 3, dict(use_act_in_conv=True, use_out_act=True)),
}


def _block(variant):
    dim, H, kw = VARIANTS[variant]
    torch.manual_seed(0)
    m = layers.GatedLinearAttention(d_model=dim, expand_k=0.5, expand_v=1.0, num_heads=H, layernorm_eps=1e-6, **kw)
    with torch.no_grad():
        m.g_norm.weight.uniform_(0.5, 1.5)
        m.l_norm.weight.uniform_(0.5, 1.5)
        m.g_proj.bias.normal_(0, 0.5)
        m.gk_proj[1].bias.normal_(0, 1.0)
        for lin in (m.qkv_proj, m.g_proj, m.o_proj, m.gk_proj[0], m.gk_proj[1]):
            lin.weight.mul_(8.0)  # the 2^-2.5 init makes everything tiny
    return m, dim, H, kw


def _rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2)])  # measured 2e-7 / 5.3e-3
@pytest.mark.parametrize("variant", ["s", "t"])
def test_training_forward_matches_kernel_forward(dtype, tol, variant):
    announce(f"GatedLinearAttention train-mode forward, autograd path against kernel path, {variant}, {dtype}")
    m, dim, H, kw = _block(variant)
    m = m.to("cuda", dtype).train()
    x = torch.randn(2, 49, dim, device="cuda", dtype=dtype)
    y_graph = m(x, patch_resolution=(7, 7), token_position=None)
    assert y_graph.requires_grad
    with torch.no_grad():
        y_kernel = m(x, patch_resolution=(7, 7), token_position=None)  # the library's kernels, training scale
    assert not y_kernel.requires_grad
    err = _rel(y_graph.detach().double().cpu(), y_kernel.double().cpu())
    print(f"  max-rel difference {err:.3e}", flush=True)
    assert err <= tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 4e-2)])  # measured 7e-7 / 1.2e-2
@pytest.mark.parametrize("variant", ["s", "t"])
def test_block_gradients(dtype, tol, variant):
    announce(f"GatedLinearAttention gradients against the float64 restatement, {variant}, {dtype}")
    m, dim, H, kw = _block(variant)
    x = torch.randn(2, 49, dim)
    cot = torch.randn(2, 49, dim)
    sd = {k: v.detach().double().requires_grad_() for k, v in m.state_dict().items()}
    x64 = x.double().requires_grad_()
    want = R.gla_block_attn(sd, "", x64, (7, 7), H, 1e-6, kw["use_act_in_conv"], kw["use_out_act"],
                            second_halving=False, differentiable=True)
    (want * cot.double()).sum().backward()

    md = m.to("cuda", dtype).train()
    xg = x.to("cuda", dtype).requires_grad_()
    got = md(xg, patch_resolution=(7, 7), token_position=None)
    (got.float() * cot.cuda()).sum().backward()
    err = _rel(got.detach().double().cpu(), want.detach())
    print(f"  forward max-rel err {err:.3e}", flush=True)
    assert err <= tol
    worst = ("x", _rel(xg.grad.double().cpu(), x64.grad))
    for name, p in md.named_parameters():
        assert p.grad is not None, name
        e = _rel(p.grad.double().cpu(), sd[name].grad)
        if e > worst[1]:
            worst = (name, e)
    print(f"  worst gradient max-rel err {worst[1]:.3e} ({worst[0]})", flush=True)
    assert worst[1] <= tol, worst


def test_vig_training_step():
    """A small ViG in training mode: logits and every parameter's gradient against the float64 restatement of the
    training branch, then one SGD step lowers the loss."""
    announce("ViG (64x64 images, depth 2, dim 96) training step, fp32")
    torch.manual_seed(0)
    kw = dict(img_size=64, depth=2, num_heads=3, embed_dim=96, num_classes=10, drop_path_rate=0.0)
    model = layers.ViG(**kw)
    with torch.no_grad():
        for blk in model.blocks:
            for lin in (blk.attn.qkv_proj, blk.attn.g_proj, blk.attn.o_proj, blk.attn.gk_proj[0], blk.attn.gk_proj[1]):
                lin.weight.mul_(8.0)
    images = torch.randn(3, 3, 64, 64)
    target = torch.tensor([1, 7, 4])
    sd = {k: v.detach().double().requires_grad_() for k, v in model.state_dict().items()}
    want = R.vig_forward(sd, images.double(), num_heads=3, depth=2, train=True)
    torch.nn.functional.cross_entropy(want, target).backward()

    model = model.cuda().train()
    logits = model(images.cuda())
    loss = torch.nn.functional.cross_entropy(logits, target.cuda())
    loss.backward()
    e = _rel(logits.detach().double().cpu(), want.detach())
    print(f"  logits max-rel err {e:.3e}", flush=True)
    assert e <= 5e-4
    worst = ("", 0.0)
    for name, p in model.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
        e = _rel(p.grad.double().cpu(), sd[name].grad)
        if e > worst[1]:
            worst = (name, e)
    print(f"  worst gradient max-rel err {worst[1]:.3e} ({worst[0]})", flush=True)
    assert worst[1] <= 2e-3, worst
    with torch.no_grad():
        for p in model.parameters():
            p -= 0.05 * p.grad
    after = torch.nn.functional.cross_entropy(model(images.cuda()), target.cuda())
    print(f"  loss {loss.item():.4f} -> {after.item():.4f}", flush=True)
    assert after.item() < loss.item()


def test_vig_training_step_under_bf16_autocast():
    """The same small ViG with fp32 parameters under torch.autocast(bfloat16) -- how the bf16 training-step figure is
    measured: logits and every parameter gradient against the float64 restatement at the bf16 bar; the parameter
    gradients stay fp32 and finite (the dtype glue: bf16 branches meeting the fp32 residual stream in the norm nodes,
    the cast of the block input, gradient dtypes arriving at the library's autograd nodes)."""
    announce("ViG (64x64 images, depth 2, dim 96) training step under bf16 autocast")
    torch.manual_seed(0)
    kw = dict(img_size=64, depth=2, num_heads=3, embed_dim=96, num_classes=10, drop_path_rate=0.0)
    model = layers.ViG(**kw)
    with torch.no_grad():
        for blk in model.blocks:
            for lin in (blk.attn.qkv_proj, blk.attn.g_proj, blk.attn.o_proj, blk.attn.gk_proj[0], blk.attn.gk_proj[1]):
                lin.weight.mul_(8.0)
    images = torch.randn(3, 3, 64, 64)
    target = torch.tensor([1, 7, 4])
    sd = {k: v.detach().double().requires_grad_() for k, v in model.state_dict().items()}
    want = R.vig_forward(sd, images.double(), num_heads=3, depth=2, train=True)
    torch.nn.functional.cross_entropy(want, target).backward()

    model = model.cuda().train()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        logits = model(images.cuda())
        loss = torch.nn.functional.cross_entropy(logits.float(), target.cuda())
    loss.backward()
    e = _rel(logits.detach().double().cpu(), want.detach())
    print(f"  logits max-rel err {e:.3e}", flush=True)
    assert e <= 2e-2  # measured 4.1e-3
    worst = ("", 0.0)
    for name, p in model.named_parameters():
        assert p.dtype == torch.float32 and p.grad is not None and p.grad.dtype == torch.float32, name
        assert torch.isfinite(p.grad).all(), name
        e = _rel(p.grad.double().cpu(), sd[name].grad)
        if e > worst[1]:
            worst = (name, e)
    print(f"  worst gradient max-rel err {worst[1]:.3e} ({worst[0]})", flush=True)
    assert worst[1] <= 6e-2, worst  # measured 1.7e-2


@pytest.mark.parametrize("channel_first", [False, True])
def test_gla2d_training_path(channel_first):
    """HierViG's GLA2D in training mode: the recorded forward equals the kernel forward, and the input gradient equals
    autograd through the float64 restatement."""
    announce(f"GLA2D training path, channel_first={channel_first}")
    torch.manual_seed(1)
    dim, H, hw = 96, 3, (9, 13)
    m = layers.GLA2D(d_model=dim, expand_k=0.5, expand_v=1.0, num_heads=H, layernorm_eps=1e-6,
                     use_act_in_conv=False, use_out_act=False, channel_first=channel_first)
    with torch.no_grad():
        for lin in (m.qkv_proj, m.g_proj, m.o_proj, m.gk_proj[0], m.gk_proj[1]):
            lin.weight.mul_(8.0)
    x = torch.randn(2, dim, *hw) if channel_first else torch.randn(2, *hw, dim)
    cot = torch.randn_like(x)
    sd = {k: v.detach().double() for k, v in m.state_dict().items()}
    x64 = x.double().requires_grad_()
    rows = (x64.permute(0, 2, 3, 1) if channel_first else x64).reshape(2, hw[0] * hw[1], dim)
    want = R.gla_block_attn(sd, "", rows, hw, H, 1e-6, False, False, second_halving=False, differentiable=True)
    want = want.reshape(2, *hw, dim)
    if channel_first:
        want = want.permute(0, 3, 1, 2)
    (want * cot.double()).sum().backward()

    m = m.cuda().train()
    xg = x.cuda().requires_grad_()
    got = m(xg)
    (got * cot.cuda()).sum().backward()
    with torch.no_grad():
        kernel = m(x.cuda())
    assert _rel(got.detach().cpu(), kernel.cpu()) <= 2e-4
    assert _rel(got.detach().cpu(), want.detach()) <= 2e-4
    e = _rel(xg.grad.cpu(), x64.grad)
    print(f"  input-gradient max-rel err {e:.3e}", flush=True)
    assert e <= 2e-4


def test_drop_path():
    """Stochastic depth of the block's branches (vig.py:533,606-608): per-sample masks scaled by 1/keep in training
    mode with the linear rate rule over depth; identity in eval mode, so inference is unchanged."""
    announce("DropPath: masks, scaling, rate rule, eval identity")
    torch.manual_seed(0)
    dp = layers.DropPath(0.25).train()
    x = torch.ones(4000, 3, 5, device="cuda")
    y = dp(x)
    per_sample = y.reshape(4000, -1)
    assert bool(((per_sample == 0).all(1) | (per_sample == 1 / 0.75).all(1)).all())  # whole samples, kept ones scaled
    kept = float((per_sample[:, 0] != 0).float().mean())
    assert abs(kept - 0.75) < 0.03
    assert torch.equal(dp.eval()(x), x)
    model = layers.ViG(img_size=64, depth=4, num_heads=3, embed_dim=96, num_classes=10, drop_path_rate=0.3)
    rates = [getattr(b.drop_path, "drop_prob", 0.0) for b in model.blocks]
    assert rates[0] == 0.0 and abs(rates[-1] - 0.3) < 1e-6 and abs(rates[1] - 0.1) < 1e-6
    model = model.cuda()
    images = torch.randn(8, 3, 64, 64, device="cuda")
    a = model.eval()(images)
    assert torch.equal(a, model(images))  # eval: deterministic
    model.train()
    b, c = model(images), model(images)
    assert b.requires_grad and not torch.equal(b, c)  # training: masks differ from call to call
    b.sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())
