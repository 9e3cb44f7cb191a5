"""GPU parity of the GLA op's neighbours: gate preparation, 3x3 stencil, locality gate, blend epilogue."""
import numpy as np
import pytest
import torch

import vig_amd
from oracle import gla_oracle as O
from vig_amd.synthetic import make_locality_weight

from .util import announce, f64, max_abs, max_rel

pytestmark = pytest.mark.gpu


def _randn(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 2e-3)])
@pytest.mark.parametrize("B,L,H,Dk", [(2, 196, 6, 32), (1, 197, 3, 64), (3, 7, 2, 16)])
def test_dirgate(dtype, tol, B, L, H, Dk):
    announce(f"dirgate {dtype} B{B} L{L} H{H} Dk{Dk}")
    x = _randn((B, L, 2 * H * Dk), 1, dtype, 3.0)
    want = O.dirgate_reference(f64(x), H, 16.0)
    got = f64(vig_amd.dirgate(x.cuda(), H, 16.0))
    assert got.shape == want.shape
    assert max_abs(got, want) <= tol
    wantc = O.dirgate_reference(f64(x), H, 16.0, clamp_min=-0.03)
    gotc = f64(vig_amd.dirgate(x.cuda(), H, 16.0, clamp_min=-0.03))
    assert max_abs(gotc, wantc) <= tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 4e-3)])
@pytest.mark.parametrize("B,L,H,Dk,wide", [(2, 196, 6, 32, 1280), (1, 197, 3, 64, 16), (3, 7, 2, 16, 24),
                                           (2, 50, 12, 64, 40)])
def test_dirgate_lowrank(dtype, tol, B, L, H, Dk, wide):
    """The rank-16 up-projection inside the gate kernel against the fp64 restatement of the two steps (the
    pre-activation rounded to the storage type in between, as the separate layer stores it): a pre-activation that
    rounds the other way moves a gate by at most one storage ulp of the pre-activation / 16 (2^-9 for values in
    [4, 8)), on top of the rounding of the output."""
    announce(f"dirgate_lowrank {dtype} B{B} L{L} H{H} Dk{Dk} row width {wide}")
    C2 = 2 * H * Dk
    z = _randn((B, L, wide), 21, dtype)
    w = _randn((C2, 16), 22, dtype, 0.5)
    b = _randn((C2,), 23, dtype, 0.5)
    low = z[..., wide - 16:]
    pre = f64(low) @ f64(w).T + f64(b)
    pre = f64(torch.from_numpy(pre).to(dtype))  # stored pre-activation
    for clamp in (None, -0.03):
        want = O.dirgate_reference(pre, H, 16.0, clamp_min=clamp)
        got = vig_amd.ops.dirgate_lowrank(z.cuda()[..., wide - 16:], w.cuda(), b.cuda(), H, 16.0, clamp_min=clamp)
        assert got.shape == want.shape
        assert max_abs(f64(got), want) <= tol
        # and against the two library steps it replaces
        two = vig_amd.dirgate(torch.nn.functional.linear(low.cuda(), w.cuda(), b.cuda()), H, 16.0, clamp_min=clamp)
        assert max_abs(f64(got), f64(two)) <= tol


def test_dirgate_feeds_gla_layout():
    """g_out[0]/g_out[1] are directly the g_fwd/g_bwd operands (reference: cat([fw,bw],0) viewed as [2,B,...])."""
    announce("dirgate -> gla layout")
    B, L, H, Dk = 2, 30, 2, 32
    x = _randn((B, L, 2 * H * Dk), 2)
    g = vig_amd.dirgate(x.cuda(), H)
    ref = torch.nn.functional.logsigmoid(x) / 16
    fw, bw = ref.chunk(2, dim=2)
    cat = torch.cat([fw, bw], dim=0).reshape(2 * B, L, H, Dk).permute(0, 2, 1, 3)
    assert (g.reshape(2 * B, H, L, Dk).cpu() - cat).abs().max() < 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("silu", [False, True])
def test_dwconv3x3(dtype, tol, silu):
    announce(f"dwconv3x3 {dtype} silu={silu}")
    B, h, w, C = 3, 14, 14, 384
    x = _randn((B, h * w, C), 3, dtype)
    wt = make_locality_weight(C, 4)
    bias = _randn((C,), 5)
    want = O.dwconv3x3_reference(f64(x), f64(wt), (h, w), bias=f64(bias), silu=silu)
    got = f64(vig_amd.dwconv3x3(x.cuda(), wt.cuda(), (h, w), bias=bias.cuda(), silu=silu))
    assert max_abs(got, want) <= tol
    want_nb = O.dwconv3x3_reference(f64(x), f64(wt), (h, w), silu=silu)
    got_nb = f64(vig_amd.dwconv3x3(x.cuda(), wt.cuda(), (h, w), silu=silu))
    assert max_abs(got_nb, want_nb) <= tol


def test_dwconv3x3_nonsquare_grid():
    announce("dwconv3x3 5x9 grid")
    B, h, w, C = 2, 5, 9, 16
    x = _randn((B, h * w, C), 6)
    wt = make_locality_weight(C, 7)
    want = O.dwconv3x3_reference(f64(x), f64(wt), (h, w))
    got = f64(vig_amd.dwconv3x3(x.cuda(), wt.cuda(), (h, w)))
    assert max_abs(got, want) <= 1e-5


def test_dwconv3x3_large_grid_row_bands():
    """64x64 token grid (the 1024^2-image shape): the kernel walks it in row bands with halo rows."""
    announce("dwconv3x3 64x64 grid, bf16, C=192")
    B, h, w, C = 1, 64, 64, 192
    x = _randn((B, h * w, C), 21, torch.bfloat16)
    wt = make_locality_weight(C, 22)
    want = O.dwconv3x3_reference(f64(x), f64(wt), (h, w), silu=True)
    got = f64(vig_amd.dwconv3x3(x.cuda(), wt.cuda(), (h, w), silu=True))
    assert max_abs(got, want) <= 2e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_locality_gate(dtype, tol):
    announce(f"locality sigmoid gate {dtype}")
    B, H, h, w, Dv = 2, 12, 14, 14, 64
    o = _randn((B, H, h * w, Dv), 8, dtype)
    wt = make_locality_weight(H * Dv, 9)
    want = O.locality_sigmoid_gate_reference(f64(o), f64(wt), (h, w))
    got = f64(vig_amd.locality_gate(o.cuda(), wt.cuda(), (h, w)))
    assert max_abs(got, want) <= tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("H,Dv,L", [(6, 64, 196), (3, 32, 49), (5, 64, 7)])
def test_locality_blend(dtype, tol, H, Dv, L):
    announce(f"blend epilogue {dtype} H{H} Dv{Dv} L{L}")
    B = 2
    o = _randn((B, H, L, Dv), 10, dtype)
    loc = _randn((B, L, H * Dv), 11, dtype)
    gl = _randn((B, L, H * Dv), 12, dtype)
    wg = _randn((Dv,), 13) * 0.1 + 1
    wl = _randn((Dv,), 14) * 0.1 + 1
    for silu in (False, True):
        want = O.locality_blend_reference(f64(o), f64(loc), f64(gl), f64(wg), f64(wl), 1e-6, silu)
        got = vig_amd.locality_blend(o.cuda(), loc.cuda(), gl.cuda(), wg.cuda(), wl.cuda(), 1e-6, silu)
        assert max_abs(f64(got), want) <= tol
        # g_lin as a column block of a wider tensor is read in place: same bits as on the packed copy
        wide = torch.zeros(B, L, H * Dv + 24, dtype=dtype).cuda()
        wide[..., 16:16 + H * Dv] = gl.cuda()
        got2 = vig_amd.locality_blend(o.cuda(), loc.cuda(), wide[..., 16:16 + H * Dv], wg.cuda(), wl.cuda(), 1e-6, silu)
        assert torch.equal(got, got2)


@pytest.mark.parametrize("B,H,L", [(2, 6, 196), (1, 3, 49), (3, 6, 37), (256, 6, 196), (1, 6, 1)])
def test_locality_blend_linear(B, H, L):
    """The blend and o_proj in one kernel against (a) an fp64 product of the stored (bf16-rounded) blend with the
    weight -- the fused kernel feeds the matrix instructions exactly those values, so what remains is fp32 accumulation
    and one rounding of the output -- and (b) the two library steps it replaces (vig_locality_blend_fwd, torch GEMM);
    g_lin as a column block of a wider tensor gives the same bits."""
    announce(f"blend + o_proj in one kernel B{B} H{H} L{L}")
    Dv, C = 64, H * 64
    dt = torch.bfloat16
    o = _randn((B, H, L, Dv), 20, dt).cuda()
    loc = _randn((B, L, C), 21, dt).cuda()
    gl = _randn((B, L, C), 22, dt).cuda()
    wg = (_randn((Dv,), 23) * 0.1 + 1).cuda()
    wl = (_randn((Dv,), 24) * 0.1 + 1).cuda()
    w = (_randn((C, C), 25, dt) * (C ** -0.5)).cuda()
    assert vig_amd.ops.locality_blend_linear_supported(o, w)
    for silu in (False, True):
        got = vig_amd.ops.locality_blend_linear(o, loc, gl, wg, wl, w, 1e-6, silu)
        assert tuple(got.shape) == (B, L, C)
        y = vig_amd.locality_blend(o, loc, gl, wg, wl, 1e-6, silu)
        two = torch.nn.functional.linear(y, w)
        err2 = (got.double() - two.double()).abs() / two.double().abs().clamp_min(1.0)
        assert err2.max().item() <= 2 * 2.0 ** -8, err2.max().item()
        if B * L <= 1200:
            want = f64(y) @ f64(w).T
            err = np.abs(f64(got).reshape(-1, C) - want.reshape(-1, C)) / np.maximum(1.0, np.abs(want.reshape(-1, C)))
            assert err.max() <= 2.0 ** -8, err.max()
            ref = O.locality_blend_reference(f64(o), f64(loc), f64(gl), f64(wg), f64(wl), 1e-6, silu) @ f64(w).T
            assert max_abs(f64(got), ref) <= 3e-2
        wide = torch.zeros(B, L, C + 24, dtype=dt).cuda()
        wide[..., 16:16 + C] = gl
        assert torch.equal(vig_amd.ops.locality_blend_linear(o, loc, wide[..., 16:16 + C], wg, wl, w, 1e-6, silu), got)
    assert not vig_amd.ops.locality_blend_linear_supported(o.float(), w.float())
    assert not vig_amd.ops.locality_blend_linear_supported(o, w[:, :C - 64])


# ---- the locality gate fused into the GLA kernel (vig_gla_bidir_locgate_fwd) ----
def _gla_inputs(B, H, L, Dk, seed, gate_scale=None):
    from vig_amd.synthetic import make_gla_inputs
    kw = {} if gate_scale is None else {"gate_scale": gate_scale}
    q, k, v, gf, gb = make_gla_inputs(B, H, L, Dk, 64, seed=seed, dtype=torch.bfloat16, **kw)
    if gate_scale is not None:
        gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
    return q, k, v, gf, gb


def _assert_fused_equals_two_calls(got, two, plain):
    """The one-kernel gate against GLA kernel + stencil kernel: bit for bit, except under outputs of the GLA (`plain`)
    below 2^-14: the fused kernel stages them as fp16, whose grid there (steps of 2^-24) is coarser than bf16's, so
    such an output, and the gate's product with it, may move by that step."""
    differs = got != two
    assert not (differs & (plain.abs() >= 2.0 ** -14)).any()
    assert ((got.float() - two.float()).abs() <= 2.0 ** -24).all()
    assert differs.float().mean().item() <= 1e-4


@pytest.mark.parametrize("B,H,hw,Dk", [(2, 12, (14, 14), 64), (3, 2, (16, 16), 64), (5, 3, (7, 7), 32),
                                        (2, 2, (3, 5), 64), (1, 3, (1, 9), 64), (2, 1, (12, 1), 32),
                                        (1, 2, (6, 40), 64), (1, 1, (1, 1), 64)])
def test_fused_locality_gate_matches_two_calls_and_oracle(B, H, hw, Dk):
    """One kernel against (a) the GLA call followed by the stencil call, bit for bit, and (b) the fp64 oracle:
    recurrent GLA, then o * sigmoid(conv(o)), within the bf16 bound."""
    from .util import oracle_bidir
    announce(f"fused locality gate B{B} H{H} grid {hw} Dk{Dk}")
    L = hw[0] * hw[1]
    q, k, v, gf, gb = _gla_inputs(B, H, L, Dk, seed=300 + L)
    wt = make_locality_weight(H * 64, 31)
    dq, dk, dv, dgf, dgb = (t.cuda() for t in (q, k, v, gf, gb))
    got = vig_amd.gla_bidir_locality_gate(dq, dk, dv, dgf, dgb, wt.cuda(), hw)
    plain = vig_amd.gla_bidir_forward(dq, dk, dv, dgf, dgb)
    two = vig_amd.locality_gate(plain, wt.cuda(), hw)
    _assert_fused_equals_two_calls(got, two, plain)
    o = oracle_bidir(q, k, v, gf, gb)
    want = O.locality_sigmoid_gate_reference(o, f64(wt), hw)
    assert max_abs(f64(got), want) <= 2e-2


def test_fused_locality_gate_many_slabs_mixed_gate_strength():
    """More slabs than workgroups, every 5th with gates too strong for the fp16 score operands: the slab that is
    walked twice must not leave anything of its first walk in the output."""
    announce("fused locality gate, 420 slabs, every 5th with strong gates")
    B, H, hw = 70, 6, (14, 14)
    q, k, v, gf, gb = _gla_inputs(B, H, 196, 64, seed=51)
    _, _, _, sf, sb = _gla_inputs(B, H, 196, 64, seed=52, gate_scale=1.0)
    strong = (torch.arange(B * H).reshape(B, H) % 5 == 2)[:, :, None, None]
    gf, gb = torch.where(strong, sf, gf), torch.where(strong, sb, gb)
    wt = make_locality_weight(H * 64, 33)
    dq, dk, dv, dgf, dgb = (t.cuda() for t in (q, k, v, gf, gb))
    got = vig_amd.gla_bidir_locality_gate(dq, dk, dv, dgf, dgb, wt.cuda(), hw)
    plain = vig_amd.gla_bidir_forward(dq, dk, dv, dgf, dgb)
    two = vig_amd.locality_gate(plain, wt.cuda(), hw)
    assert torch.isfinite(got.float()).all()
    _assert_fused_equals_two_calls(got, two, plain)


def test_fused_locality_gate_other_shapes_take_two_calls():
    """Shapes outside the one-kernel form (long sequence, fp32) go through the two calls and still match the oracle."""
    from .util import oracle_bidir
    announce("fused locality gate wrapper on L=18x18 and on fp32")
    hw = (18, 18)
    q, k, v, gf, gb = _gla_inputs(1, 2, 324, 64, seed=61)
    wt = make_locality_weight(2 * 64, 35)
    got = vig_amd.gla_bidir_locality_gate(*(t.cuda() for t in (q, k, v, gf, gb)), wt.cuda(), hw)
    want = O.locality_sigmoid_gate_reference(oracle_bidir(q, k, v, gf, gb), f64(wt), hw)
    assert max_abs(f64(got), want) <= 2e-2
    q, k, v, gf, gb = (t.float() for t in _gla_inputs(1, 2, 49, 64, seed=62))
    got = vig_amd.gla_bidir_locality_gate(*(t.cuda() for t in (q, k, v, gf, gb)), wt.cuda(), (7, 7))
    want = O.locality_sigmoid_gate_reference(oracle_bidir(q, k, v, gf, gb), f64(wt), (7, 7))
    assert max_abs(f64(got), want) <= 1e-4 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("shape", [(3, 5, 7, 24), (2, 14, 14, 768), (1, 1, 40, 8)])
def test_dwconv3x3_gradients(dtype, tol, silu, shape):
    """Input, weight and bias gradients of the differentiable stencil op against autograd through torch's conv2d in
    float64 (on the same rounded inputs)."""
    announce(f"dwconv3x3 gradients {shape} {dtype} silu={silu}")
    torch.manual_seed(3)
    B, h, w, C = shape
    x = torch.randn(B, h * w, C).to(dtype)
    wt = (torch.randn(C, 1, 3, 3) / 3).to(dtype)
    bs = torch.randn(C).to(dtype)
    cot = torch.randn(B, h * w, C)
    x64, w64, b64 = (t.double().requires_grad_() for t in (x, wt, bs))
    y64 = torch.nn.functional.conv2d(x64.reshape(B, h, w, C).permute(0, 3, 1, 2), w64, b64, padding=1, groups=C)
    if silu:
        y64 = torch.nn.functional.silu(y64)
    y64 = y64.flatten(2).transpose(1, 2)
    (y64 * cot.double()).sum().backward()
    xg, wg, bg = (t.cuda().requires_grad_() for t in (x, wt, bs))
    y = vig_amd.ops.dwconv3x3(xg, wg, (h, w), bias=bg, silu=silu)
    (y.float() * cot.cuda()).sum().backward()

    def rel(a, b):
        return ((a.double().cpu() - b).abs().max() / b.abs().max()).item()

    errs = dict(y=rel(y.detach(), y64.detach()), dx=rel(xg.grad, x64.grad), dw=rel(wg.grad, w64.grad),
                db=rel(bg.grad, b64.grad))
    print("  " + "  ".join(f"{k} {v:.2e}" for k, v in errs.items()), flush=True)
    assert max(errs.values()) <= tol, errs


@pytest.mark.parametrize("silu_out", [False, True])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B,H,L,Dv", [(2, 6, 49, 64), (1, 3, 70, 32), (2, 12, 33, 64)])
def test_locality_blend_gradients(dtype, tol, silu_out, B, H, L, Dv):
    """vig_locality_blend_bwd through the op's autograd node against autograd through the float64 expression of the
    epilogue (vig.py:447-457), on the same rounded inputs: gradients of o, local, g_lin and both norm weights."""
    announce(f"locality_blend gradients B{B} H{H} L{L} Dv{Dv} {dtype} silu_out={silu_out}")
    torch.manual_seed(B * 100 + L)
    C = H * Dv
    o = torch.randn(B, H, L, Dv).to(dtype)
    loc = torch.randn(B, L, C).to(dtype)
    gl = torch.randn(B, L, C).to(dtype)
    wg, wl = torch.rand(Dv) + 0.5, torch.rand(Dv) + 0.5
    cot = torch.randn(B, L, C)
    t64 = [t.double().requires_grad_() for t in (o, loc, gl, wg, wl)]

    def rms(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

    on = rms(t64[0].permute(0, 2, 1, 3), t64[3])
    ln = rms(t64[1].reshape(B, L, H, Dv), t64[4])
    s = torch.sigmoid(t64[2]).reshape(B, L, H, Dv)
    y64 = (on * s + ln * (1 - s)).reshape(B, L, C)
    if silu_out:
        y64 = torch.nn.functional.silu(y64)
    (y64 * cot.double()).sum().backward()
    tg = [t.cuda().requires_grad_() for t in (o, loc, gl, wg, wl)]
    y = vig_amd.ops.locality_blend(*tg, eps=1e-6, silu_out=silu_out)
    (y.float() * cot.cuda()).sum().backward()

    def rel(a, b):
        return ((a.double().cpu() - b).abs().max() / b.abs().max()).item()

    errs = {n: rel(a.grad, b.grad) for n, a, b in zip(("do", "dlocal", "dglin", "dw_g", "dw_l"), tg, t64)}
    errs["y"] = rel(y.detach(), y64.detach())
    print("  " + "  ".join(f"{k} {v:.2e}" for k, v in errs.items()), flush=True)
    assert max(errs.values()) <= tol, errs


@pytest.mark.parametrize("clamp_min", [None, -0.05])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_dirgate_gradients(dtype, tol, clamp_min):
    """vig_dirgate_bwd against autograd through logsigmoid / normalizer / clamp / split / rearrange in float64."""
    announce(f"dirgate gradients {dtype} clamp_min={clamp_min}")
    torch.manual_seed(1)
    B, L, H, Dk = 2, 45, 3, 16
    x = (torch.randn(B, L, 2 * H * Dk) * 2).to(dtype)
    cot = torch.randn(2, B, H, L, Dk)
    x64 = x.double().requires_grad_()
    g64 = torch.nn.functional.logsigmoid(x64) / 16
    if clamp_min is not None:
        g64 = torch.clamp_min(g64, clamp_min)
    g64 = g64.reshape(B, L, 2, H, Dk).permute(2, 0, 3, 1, 4)
    (g64 * cot.double()).sum().backward()
    xg = x.cuda().requires_grad_()
    g = vig_amd.ops.dirgate(xg, H, 16.0, clamp_min)
    (g.float() * cot.cuda()).sum().backward()
    err = ((xg.grad.double().cpu() - x64.grad).abs().max() / x64.grad.abs().max()).item()
    print(f"  d_gk_lin max-rel err {err:.2e}", flush=True)
    assert err <= tol
