"""The PyTorch-ROCm operator library (torch.ops.vig_amd.*, csrc/torch_ext.cpp) against the ctypes binding of the same
C ABI: every forward operator bit for bit on the same inputs, argument checks as exceptions, and the eval-mode model
through the operators against the model on the ctypes binding."""
import numpy as np
import pytest
import torch

import vig_amd
from vig_amd import _ext, layers, ops
from vig_amd.synthetic import make_gla_inputs, make_locality_weight

from .util import announce

pytestmark = pytest.mark.gpu


def _ops():
    ext = _ext.load()
    assert ext is not None, f"operator library not loaded: {_ext.why_not()}"
    return ext


def _same(a, b):
    assert a.dtype == b.dtype and a.shape == b.shape
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gla_operators_match_the_ctypes_binding(dtype):
    ext = _ops()
    announce(f"torch.ops.vig_amd GLA operators {dtype}")
    for (B, H, L, Dk, Dv) in ((3, 2, 196, 64, 64), (2, 3, 700, 32, 64), (2, 2, 130, 16, 32), (1, 2, 50, 128, 64)):
        t = [x.cuda() for x in make_gla_inputs(B, H, L, Dk, Dv, seed=5, dtype=dtype)]
        _same(ext.gla_bidir_fwd(*t, -1.0, 0.5, 0), ops.gla_bidir_forward(*t, out_scale=0.5))
        _same(ext.gla_bidir_fwd(*t[:4], None, -1.0, 1.0, 0), ops.gla_bidir_forward(*t[:4], None))
        _same(ext.gla_bidir_fwd(*t, 0.3, 1.0, 2), ops.gla_bidir_forward(*t, scale=0.3, exact=True))
        if Dk in (32, 64) and Dv == 64:
            _same(ext.gla_bidir_fwd(*t, -1.0, 1.0, 1), ops.gla_bidir_forward(*t, strong_gates=True))
        s0 = torch.randn(B, H, Dk, Dv, device="cuda")
        o1, f1 = ext.gla_causal_state_fwd(*t[:4], s0, True, -1.0, False)
        o2, f2 = ops.gla_causal_state_forward(*t[:4], s0, True)
        _same(o1, o2)
        _same(f1, f2)
        o1, f1 = ext.gla_causal_state_fwd(*t[:4], None, False, -1.0, True)
        assert f1 is None
        _same(o1, ops.gla_causal_state_forward(*t[:4], None, False, exact=True)[0])
        if Dk <= 64 and Dv <= 64:
            d_o = torch.randn(B, H, L, Dv, device="cuda").to(dtype)
            for exact in (False, True):
                got = ext.gla_bidir_bwd(*t, d_o, -1.0, 1.0, exact)
                want = ops.gla_bidir_backward(*t, d_o, exact=exact)
                for a, b in zip(got, want):
                    _same(a, b)
            got = ext.gla_bidir_bwd(*t[:4], None, d_o, -1.0, 1.0, False)
            assert got[4] is None
    # fused locality gate
    t = [x.cuda() for x in make_gla_inputs(2, 3, 196, 64, 64, seed=6, dtype=torch.bfloat16)]
    w = make_locality_weight(3 * 64, seed=7).cuda()
    _same(ext.gla_bidir_locgate_fwd(*t, w.reshape(-1).contiguous(), 14, 14, -1.0, 1.0),
          ops.gla_bidir_locality_gate(*t, w, (14, 14)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_neighbour_operators_match_the_ctypes_binding(dtype):
    ext = _ops()
    announce(f"torch.ops.vig_amd neighbour operators {dtype}")
    g = torch.Generator(device="cuda").manual_seed(3)
    r = lambda *s: torch.randn(*s, device="cuda", generator=g).to(dtype)
    rf = lambda *s: torch.randn(*s, device="cuda", generator=g)
    B, L, H, Dk, Dv, hw = 3, 196, 6, 32, 64, (14, 14)
    C = H * Dv
    gk = r(B, L, 2 * H * Dk)
    _same(ext.dirgate_fwd(gk, H, 16.0, None), ops.dirgate(gk, H))
    _same(ext.dirgate_fwd(gk, H, 8.0, -0.05), ops.dirgate(gk, H, 8.0, -0.05))
    wide = r(B, L, 1280)
    low, w_up, b_up = wide[..., 1152:1168], r(2 * H * Dk, 16), r(2 * H * Dk)
    _same(ext.dirgate_lowrank_fwd(low, w_up, b_up, H, 16.0, None), ops.dirgate_lowrank(low, w_up, b_up, H))
    x = r(B, L, C)
    cw, cb = rf(C, 1, 3, 3) / 3, rf(C)
    _same(ext.dwconv3x3_fwd(x, cw.reshape(-1).contiguous(), cb, 14, 14, True), ops.dwconv3x3(x, cw, hw, cb, silu=True))
    _same(ext.dwconv3x3_fwd(x, cw.reshape(-1).contiguous(), None, 14, 14, False), ops.dwconv3x3(x, cw, hw))
    o = r(B, H, L, Dv)
    _same(ext.locality_gate_fwd(o, cw.reshape(-1).contiguous(), 14, 14), ops.locality_gate(o, cw, hw))
    wg, wl = rf(Dv).abs() + 0.5, rf(Dv).abs() + 0.5
    glin = wide[..., 768:768 + C]
    _same(ext.locality_blend_fwd(o, x, glin, wg, wl, 1e-6, True), ops.locality_blend(o, x, glin, wg, wl, 1e-6, True))
    wn = rf(C).abs() + 0.5
    res = r(B, L, C)
    y1, s1 = ext.rmsnorm_fwd(x, res, wn, 1e-6, True)
    y2, s2 = ops.rmsnorm(x, wn, 1e-6, residual=res, prenorm=True, round_sum=True)
    _same(y1, y2)
    _same(s1, s2)
    y1, s1 = ext.rmsnorm_fwd(x, None, wn, 1e-6, False)
    assert s1 is None
    _same(y1, ops.rmsnorm(x, wn, 1e-6))
    lb, pre, post = rf(C), rf(C), r(L, C)
    _same(ext.layernorm_fwd(x, wn, lb, 1e-5, True, pre, post), ops.layernorm(x, wn, lb, 1e-5, True, pre, post))
    _same(ext.layernorm_fwd(x, wn, lb, 1e-5, False, None, None), ops.layernorm(x, wn, lb))
    qkv = wide[..., :H * (2 * Dk + Dv)]
    for a, b in zip(ext.split_heads_fwd(qkv, H, Dk, Dv), ops.split_heads(qkv, H, Dk, Dv)):
        _same(a, b)
    gu = r(B, L, 2 * 1024)
    _same(ext.swiglu_fwd(gu), ops.swiglu(gu))
    if dtype == torch.bfloat16:
        wgp = r(2048, C)
        _same(ext.linear_swiglu_fwd(x, wgp), ops.linear_swiglu(x, wgp))
        img, wc = r(2, 3, 224, 224), r(192, 3, 9, 9) / 9
        packed = ops.pack_patch_conv_weight(wc)
        _same(ext.patch_conv_fwd(img, packed, 9, 9, 8, 1), ops.patch_conv(img, packed, (9, 9)))


def test_operator_argument_checks():
    ext = _ops()
    announce("torch.ops.vig_amd argument checks")
    t = [x.cuda() for x in make_gla_inputs(1, 2, 64, 64, 64, seed=1, dtype=torch.bfloat16)]
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ext.gla_bidir_fwd(t[0].cpu(), *t[1:], -1.0, 1.0, 0)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.gla_bidir_fwd(t[0].transpose(1, 2), *t[1:], -1.0, 1.0, 0)
    with pytest.raises(RuntimeError, match="share a dtype"):
        ext.gla_bidir_fwd(t[0].float(), *t[1:], -1.0, 1.0, 0)
    with pytest.raises(RuntimeError, match="16-byte"):
        flat = torch.zeros(t[0].numel() + 8, dtype=torch.bfloat16, device="cuda")
        ext.gla_bidir_fwd(flat[1:1 + t[0].numel()].view_as(t[0]), *t[1:], -1.0, 1.0, 0)
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        ext.swiglu_fwd(torch.zeros(4, 64, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError, match="not built"):  # status codes of the C ABI come back as exceptions
        ext.gla_bidir_locgate_fwd(*[x.float() for x in t], torch.zeros(2 * 64 * 9, device="cuda"), 8, 8, -1.0, 1.0)


def test_model_through_the_operators_matches_the_ctypes_model(monkeypatch):
    """ViG-S eval logits with the block's mixer, the norms and the MLP on torch.ops.vig_amd against the same model on
    the ctypes binding: the same kernels in the same order, so the logits agree bit for bit."""
    _ops()
    announce("ViG-S eval forward: operator library against ctypes binding")
    torch.manual_seed(0)
    model = layers.vig_small().eval().to("cuda", torch.bfloat16)
    x = torch.randn(4, 3, 224, 224, device="cuda").to(torch.bfloat16)
    with torch.no_grad():
        a = model(x)
        monkeypatch.setattr(_ext, "_ops", None)  # what VIG_AMD_NO_EXT=1 gives
        b = model(x)
    _same(a, b)
