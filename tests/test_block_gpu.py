"""GPU parity of the row-wise block kernels: residual RMS norm, head split, SwiGLU product."""
import numpy as np
import pytest
import torch

import vig_amd
from oracle import gla_oracle as O

from .util import announce, f64

pytestmark = pytest.mark.gpu


def _randn(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _close(got, want, tol):
    """Elementwise |got - want| <= tol * max(1, |want|): bf16 outputs carry half an output ulp (2^-9 relative)."""
    return bool(np.all(np.abs(got - want) <= tol * np.maximum(1.0, np.abs(want))))


def _bf16_round(a):
    return torch.from_numpy(a).to(torch.bfloat16).double().numpy()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("rows,C", [((2, 196), 384), ((3, 5), 192), ((1, 7), 768), ((9,), 8), ((2, 3), 2048)])
def test_rmsnorm_residual_prenorm(dtype, tol, rows, C):
    announce(f"rmsnorm {dtype} rows{rows} C{C}")
    x, r = _randn((*rows, C), 1, dtype), _randn((*rows, C), 2, dtype, 2.0)
    w = _randn((C,), 3) + 1.0
    # no residual
    want, _ = O.rmsnorm_residual_reference(f64(x), f64(w), 1e-6)
    got = vig_amd.ops.rmsnorm(x.cuda(), w.cuda(), 1e-6)
    assert _close(f64(got), want, tol)
    # residual, prenorm: the fused arithmetic normalises the unrounded sum
    want, s = O.rmsnorm_residual_reference(f64(x), f64(w), 1e-6, residual=f64(r))
    got, res = vig_amd.ops.rmsnorm(x.cuda(), w.cuda(), 1e-6, residual=r.cuda(), prenorm=True)
    assert _close(f64(got), want, tol)
    assert _close(f64(res), s, tol)
    if dtype == torch.bfloat16:
        # round_sum: the stored (rounded) sum is what gets normalised, and it is returned bit-exactly
        want, s = O.rmsnorm_residual_reference(f64(x), f64(w), 1e-6, residual=f64(r), round_to=_bf16_round)
        got, res = vig_amd.ops.rmsnorm(x.cuda(), w.cuda(), 1e-6, residual=r.cuda(), prenorm=True, round_sum=True)
        assert np.array_equal(f64(res), s)
        assert np.array_equal(f64(res), f64(x + r))
        assert _close(f64(got), want, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("rows,C", [(1568, 192), (197, 384), (5, 8), (33, 264), (3, 768), (2, 2048), (1, 4096)])
def test_layernorm(dtype, tol, rows, C):
    """LayerNorm (+ SiLU on the stored value) against the fp64 oracle on the stored inputs; tolerance relative to
    max(1, |want|): one rounding of the output."""
    announce(f"layernorm {dtype} rows{rows} C{C}")
    x = _randn((rows, C), 31, dtype) * 3 + 0.5
    w = _randn((C,), 32) * 0.2 + 1
    b = _randn((C,), 33) * 0.3
    rnd = (lambda a: f64(torch.from_numpy(a).to(dtype)))
    for silu in (False, True):
        want = O.layernorm_reference(f64(x), f64(w), f64(b), 1e-5, silu=silu, round_to=rnd)
        got = f64(vig_amd.ops.layernorm(x.cuda(), w.cuda(), b.cuda(), 1e-5, silu=silu))
        err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
        assert err.max() <= (tol if not silu else 2 * tol), (silu, err.max())
    # a bias added in front (rounded sum, as a convolution would have stored it) and a row-periodic table behind
    if rows % 7 == 0 or rows < 7:
        period = 7 if rows % 7 == 0 else rows
        pb = _randn((C,), 34) * 0.5
        pa = _randn((period, C), 35, dtype)
        xin = rnd(f64(x) + f64(pb))
        want = rnd(O.layernorm_reference(xin, f64(w), f64(b), 1e-5)) + np.tile(f64(pa), (rows // period, 1))
        got = f64(vig_amd.ops.layernorm(x.cuda(), w.cuda(), b.cuda(), 1e-5, pre_bias=pb.cuda(), post_add=pa.cuda()))
        err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
        assert err.max() <= 3 * tol, err.max()


@pytest.mark.parametrize("rows,K,I", [(50176, 384, 1024), (1000, 384, 1024), (33, 384, 96), (1, 192, 32), (777, 192, 512),
                                      (64, 384, 288)])
def test_linear_swiglu(rows, K, I):
    """gate_proj + SwiGLU in one kernel against (a) the fp64 oracle applied to the stored (bf16-rounded) gate and up
    values of an fp64 product -- a gate or up that rounds the other way moves the output by one bf16 ulp of that factor,
    hence the relative tolerance -- and (b) the two library steps it replaces (torch GEMM, then vig_swiglu_fwd)."""
    announce(f"linear_swiglu rows{rows} K{K} I{I}")
    x = _randn((rows, K), 51, torch.bfloat16)
    w = _randn((2 * I, K), 52, torch.bfloat16) * (K ** -0.5)
    got = vig_amd.ops.linear_swiglu(x.cuda(), w.cuda())
    assert tuple(got.shape) == (rows, I)
    gu = f64(x) @ f64(w).T
    gu_stored = f64(torch.from_numpy(gu).to(torch.bfloat16))
    want = O.swiglu_reference(gu_stored)
    err = np.abs(f64(got) - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= 3 * 2.0 ** -8, err.max()
    two = vig_amd.ops.swiglu(torch.nn.functional.linear(x.cuda(), w.cuda()))
    err2 = (got.double() - two.double()).abs() / two.double().abs().clamp_min(1.0)
    assert err2.max().item() <= 3 * 2.0 ** -8, err2.max().item()


def test_linear_swiglu_refuses_other_shapes():
    x = torch.zeros(4, 256, dtype=torch.bfloat16).cuda()
    w = torch.zeros(128, 256, dtype=torch.bfloat16).cuda()
    assert not vig_amd.ops.linear_swiglu_supported(x, w)
    assert not vig_amd.ops.linear_swiglu_supported(x.float()[:, :192], w.float()[:, :192])
    with pytest.raises(vig_amd._lib.VigGlaError):
        vig_amd.ops.linear_swiglu(x, w)


@pytest.mark.parametrize("B,H,W,KW,Cout", [(3, 224, 224, 9, 192), (2, 64, 64, 9, 96), (1, 40, 248, 9, 256),
                                           (2, 17, 24, 9, 64), (1, 224, 224, 16, 64)])
def test_patch_conv(B, H, W, KW, Cout):
    """The stem convolution (kernel 9 rows x KW columns, stride 8, padding 1, 3 channels) against torch's conv2d in
    fp64 on the stored bf16 inputs; one rounding of the output plus the fp32 accumulation of 243+ products."""
    announce(f"patch_conv B{B} {H}x{W} KW{KW} Cout{Cout}")
    x = _randn((B, 3, H, W), 41, torch.bfloat16)
    w = _randn((Cout, 3, 9, KW), 42, torch.bfloat16) * 0.1
    assert vig_amd.ops.patch_conv_supported(x.cuda(), w.cuda(), 8, 1)
    got = vig_amd.ops.patch_conv(x.cuda(), vig_amd.ops.pack_patch_conv_weight(w.cuda()), (9, KW), 8, 1)
    want = torch.nn.functional.conv2d(x.double(), w.double(), None, 8, 1).permute(0, 2, 3, 1)
    assert tuple(got.shape) == tuple(want.shape)
    err = (got.double().cpu() - want).abs() / want.abs().clamp_min(1.0)
    assert err.max().item() <= 2.0 ** -8, err.max().item()


def test_patch_conv_refuses_other_shapes():
    x = torch.zeros(1, 3, 32, 36, dtype=torch.bfloat16).cuda()  # width not a multiple of 8
    w = torch.zeros(32, 3, 9, 9, dtype=torch.bfloat16).cuda()
    assert not vig_amd.ops.patch_conv_supported(x, w, 8, 1)
    assert not vig_amd.ops.patch_conv_supported(x[..., :32], w, 4, 1)
    assert not vig_amd.ops.patch_conv_supported(x[..., :32].float(), w.float(), 8, 1)
    with pytest.raises(vig_amd._lib.VigGlaError):
        vig_amd.ops.patch_conv(x, vig_amd.ops.pack_patch_conv_weight(w), (9, 9), 8, 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,Dk,Dv", [(2, 196, 6, 32, 64), (1, 197, 3, 64, 64), (3, 7, 2, 16, 32)])
def test_split_heads_is_exact(dtype, B, L, H, Dk, Dv):
    announce(f"split_heads {dtype} B{B} L{L} H{H} {Dk}/{Dv}")
    qkv = _randn((B, L, H * (2 * Dk + Dv)), 4, dtype)
    q, k, v = vig_amd.ops.split_heads(qkv.cuda(), H, Dk, Dv)
    wq, wk, wv = O.split_heads_reference(f64(qkv), H, Dk, Dv)
    assert np.array_equal(f64(q), wq) and np.array_equal(f64(k), wk) and np.array_equal(f64(v), wv)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,Dk,Dv,W", [(2, 196, 6, 32, 64, 1280), (3, 7, 2, 16, 32, 136), (1, 50, 3, 64, 64, 588)])
def test_split_heads_reads_a_column_block_in_place(dtype, B, L, H, Dk, Dv, W):
    """qkv as the leading columns of a wider projection output: same result as on a packed copy; a row distance
    that breaks the 16-byte alignment (the views that start at column 1, and W = 588 with bf16) is packed
    by the wrapper."""
    announce(f"split_heads strided {dtype} B{B} L{L} H{H} {Dk}/{Dv} W{W}")
    n = H * (2 * Dk + Dv)
    wide = _randn((B, L, W), 5, dtype).cuda()
    for view in (wide[..., :n], wide[..., 8:8 + n], wide[..., 1:1 + n]):
        q, k, v = vig_amd.ops.split_heads(view, H, Dk, Dv)
        wq, wk, wv = O.split_heads_reference(f64(view), H, Dk, Dv)
        assert np.array_equal(f64(q), wq) and np.array_equal(f64(k), wk) and np.array_equal(f64(v), wv)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("rows,I", [((2, 196), 1024), ((5,), 8), ((3, 4), 512)])
def test_swiglu(dtype, tol, rows, I):
    announce(f"swiglu {dtype} rows{rows} I{I}")
    gu = _randn((*rows, 2 * I), 5, dtype, 2.0)
    want = O.swiglu_reference(f64(gu))
    got = vig_amd.ops.swiglu(gu.cuda())
    assert got.shape == (*rows, I)
    assert _close(f64(got), want, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("rows,C", [(37, 384), (300, 64), (9, 1024), (20000, 768), (5000, 192)])
@pytest.mark.parametrize("residual", [False, True])
def test_rmsnorm_gradients(dtype, tol, rows, C, residual):
    """vig_rmsnorm_bwd through the op's autograd node against autograd through the float64 formula: gradients of x,
    of the residual and of the weight, with a gradient arriving at the returned sum as well."""
    announce(f"rmsnorm gradients rows={rows} C={C} residual={residual} {dtype}")
    torch.manual_seed(rows + C)
    x = torch.randn(rows, C).to(dtype)
    r = torch.randn(rows, C).to(dtype) if residual else None
    w = torch.rand(C) + 0.5
    cot_y, cot_s = torch.randn(rows, C), torch.randn(rows, C)
    x64, w64 = x.double().requires_grad_(), w.double().requires_grad_()
    r64 = r.double().requires_grad_() if residual else None
    s64 = x64 + r64 if residual else x64
    if residual and dtype == torch.bfloat16:
        # the op returns the sum rounded to bf16 and its backward recomputes from that stored sum
        s64 = s64 + (s64.detach().to(dtype).double() - s64.detach())
    y64 = s64 * torch.rsqrt(s64.pow(2).mean(-1, keepdim=True) + 1e-6) * w64
    ((y64 * cot_y.double()).sum() + ((s64 * cot_s.double()).sum() if residual else 0)).backward()

    xg, wg = x.cuda().requires_grad_(), w.cuda().requires_grad_()
    rg = r.cuda().requires_grad_() if residual else None
    if residual:
        y, s = vig_amd.ops.rmsnorm(xg, wg, 1e-6, residual=rg, prenorm=True)
        ((y.float() * cot_y.cuda()).sum() + (s.float() * cot_s.cuda()).sum()).backward()
    else:
        y = vig_amd.ops.rmsnorm(xg, wg, 1e-6)
        (y.float() * cot_y.cuda()).sum().backward()

    def rel(a, b):
        return ((a.double().cpu() - b).abs().max() / b.abs().max()).item()

    errs = dict(y=rel(y.detach(), y64.detach()), dx=rel(xg.grad, x64.grad), dw=rel(wg.grad, w64.grad))
    if residual:
        errs["dres"] = rel(rg.grad, r64.grad)
    print("  " + "  ".join(f"{k} {v:.2e}" for k, v in errs.items()), flush=True)
    assert max(errs.values()) <= tol, errs


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_swiglu_gradients(dtype, tol):
    announce(f"swiglu gradients {dtype}")
    torch.manual_seed(2)
    gu = (torch.randn(3, 50, 2 * 136) * 2).to(dtype)
    cot = torch.randn(3, 50, 136)
    g64 = gu.double().requires_grad_()
    a, b = g64.chunk(2, -1)
    ((torch.nn.functional.silu(a) * b) * cot.double()).sum().backward()
    gg = gu.cuda().requires_grad_()
    y = vig_amd.ops.swiglu(gg)
    (y.float() * cot.cuda()).sum().backward()
    err = ((gg.grad.double().cpu() - g64.grad).abs().max() / g64.grad.abs().max()).item()
    print(f"  d_gate_up max-rel err {err:.2e}", flush=True)
    assert err <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_split_heads_gradients(dtype):
    """vig_split_heads_bwd: the gradient of the split is the gather of the three head-major gradients (exact)."""
    announce(f"split_heads gradients {dtype}")
    torch.manual_seed(4)
    B, L, H, Dk, Dv = 2, 37, 3, 16, 32
    qkv = torch.randn(B, L, H * (2 * Dk + Dv), device="cuda").to(dtype).requires_grad_()
    cq, ck = torch.randn(B, H, L, Dk, device="cuda").to(dtype), torch.randn(B, H, L, Dk, device="cuda").to(dtype)
    cv = torch.randn(B, H, L, Dv, device="cuda").to(dtype)
    q, k, v = vig_amd.ops.split_heads(qkv, H, Dk, Dv)
    torch.autograd.backward((q, k, v), (cq, ck, cv))

    def rows(t):
        return t.permute(0, 2, 1, 3).reshape(B, L, -1)

    want = torch.cat((rows(cq), rows(ck), rows(cv)), dim=-1)
    assert torch.equal(qkv.grad, want)


def test_rmsnorm_gradients_with_an_unused_output():
    """Only one of the two outputs of the residual form is used: the other's gradient arrives as None."""
    announce("rmsnorm gradients, one output unused")
    torch.manual_seed(0)
    x, r = torch.randn(20, 64, device="cuda"), torch.randn(20, 64, device="cuda")
    w = torch.rand(64, device="cuda") + 0.5
    for use in ("y", "sum"):
        xg, rg, wg = x.clone().requires_grad_(), r.clone().requires_grad_(), w.clone().requires_grad_()
        y, s = vig_amd.ops.rmsnorm(xg, wg, 1e-6, residual=rg, prenorm=True)
        (y if use == "y" else s).sum().backward()
        x2, r2, w2 = x.clone().requires_grad_(), r.clone().requires_grad_(), w.clone().requires_grad_()
        s2 = x2 + r2
        y2 = s2 * torch.rsqrt(s2.pow(2).mean(-1, keepdim=True) + 1e-6) * w2
        (y2 if use == "y" else s2).sum().backward()
        assert torch.allclose(xg.grad, x2.grad, rtol=1e-4, atol=1e-5) and torch.equal(xg.grad, rg.grad)
        assert torch.allclose(wg.grad, w2.grad if w2.grad is not None else torch.zeros_like(w), rtol=1e-4, atol=1e-5)


def test_backward_entry_points_validate_arguments():
    """Null pointers, unsupported widths and short workspaces are refused with the documented codes before any launch."""
    announce("argument validation of the block's backward entry points")
    from vig_amd import _lib
    lib = _lib.load()
    x = torch.zeros(64, 384, device="cuda", dtype=torch.bfloat16)
    w = torch.ones(384, device="cuda")
    p, wp, st = x.data_ptr(), w.data_ptr(), torch.cuda.current_stream().cuda_stream
    bf = _lib.VIG_BF16
    assert lib.vig_swiglu_bwd(None, p, p, 64, 192, bf, st) == _lib.VIG_EINVAL
    assert lib.vig_swiglu_bwd(p, p, p, 64, 190, bf, st) == _lib.VIG_ENOTSUP
    assert lib.vig_rmsnorm_bwd(p, wp, None, None, p, None, None, 0, 64, 384, 1e-6, bf, st) == _lib.VIG_EINVAL
    assert lib.vig_rmsnorm_bwd(p, wp, p, None, p, None, None, 0, 64, 2048, 1e-6, bf, st) == _lib.VIG_ENOTSUP
    assert lib.vig_rmsnorm_bwd(p, wp, p, None, p, wp, p, 16, 64, 384, 1e-6, bf, st) == _lib.VIG_ENOSPC
    assert lib.vig_rmsnorm_bwd_workspace(64, 384) == 4 * 384 * 4 and lib.vig_rmsnorm_bwd_workspace(0, 384) == 0
    assert lib.vig_dirgate_bwd(p, None, p, 1, 64, 3, 64, 1 / 16, float("nan"), bf, bf, st) == _lib.VIG_EINVAL
    assert lib.vig_dirgate_bwd(p, p, p, 1, 64, 3, 12, 1 / 16, float("nan"), bf, bf, st) == _lib.VIG_ENOTSUP
    assert lib.vig_split_heads_bwd(p, p, None, p, 1, 64, 3, 32, 64, bf, st) == _lib.VIG_EINVAL
    assert lib.vig_dwconv3x3_bwd_weight(p, p, wp, p, 16, 1, 8, 8, 384, bf, st) == _lib.VIG_ENOSPC
    assert lib.vig_dwconv3x3_bwd_weight(p, p, wp, None, 0, 1, 8, 8, 380, bf, st) == _lib.VIG_ENOTSUP
    assert lib.vig_locality_blend_bwd(p, p, p, wp, wp, p, p, p, p, wp, p, 16, 1, 6, 64, 64, 0, 1e-6, 0, bf,
                                      st) == _lib.VIG_ENOSPC
    assert lib.vig_locality_blend_bwd(p, p, p, wp, wp, p, p, p, p, wp, p, 1 << 20, 1, 6, 64, 48, 0, 1e-6, 0, bf,
                                      st) == _lib.VIG_ENOTSUP
    assert lib.vig_locality_blend_bwd_workspace(2, 64, 48) == 0
    torch.cuda.synchronize()
