"""GPU parity of the backward of the bidirectional GLA op (through the C ABI and through autograd) against the
fp64 oracle's adjoint recurrences (themselves pinned by finite differences and autograd in tests/test_oracle.py)."""
import numpy as np
import pytest
import torch

import vig_amd
from oracle import gla_oracle as O
from vig_amd.synthetic import make_gla_inputs

from .util import announce, f64

pytestmark = pytest.mark.gpu


def _do(shape, seed, dtype):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _rel(got, want, floor=0.0):
    """max|got - want| over the larger of max|want| and `floor`.  The gate gradient is a difference of two terms
    (q*dq - k*dk) that can cancel exactly (L = 1), so it is measured against the size of those terms."""
    return float(np.abs(got - want).max() / max(np.abs(want).max(), floor, 1e-30))


def _check_all(got, want, q, tol=1e-4):
    floor = float(np.abs(f64(q) * want[0]).max())
    for name, g_, w_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, want):
        if w_ is None:
            assert g_ is None
            continue
        assert _rel(f64(g_), w_, floor if name.startswith("dg") else 0.0) <= tol, name


@pytest.mark.parametrize("L", [1, 2, 15, 16, 17, 64, 196, 300])
def test_backward_fp32_ragged_lengths(L):
    announce(f"backward fp32 L={L}")
    q, k, v, gf, gb = make_gla_inputs(2, 2, L, 64, 64, seed=300 + L)
    do = _do(v.shape, 7, torch.float32)
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    got = vig_amd.gla_bidir_backward(*(t.cuda() for t in (q, k, v, gf, gb, do)), out_scale=0.5)
    _check_all(got, want, q)


@pytest.mark.parametrize("Dk,Dv", [(16, 32), (32, 32), (32, 64), (64, 32)])
def test_backward_fp32_head_dims_and_causal(Dk, Dv):
    announce(f"backward fp32 Dk={Dk} Dv={Dv}, causal only")
    q, k, v, gf, _ = make_gla_inputs(1, 3, 50, Dk, Dv, seed=9, gate_scale=0.5)
    do = _do(v.shape, 8, torch.float32)
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), None, f64(do))
    got = vig_amd.gla_bidir_backward(q.cuda(), k.cuda(), v.cuda(), gf.cuda(), None, do.cuda())
    _check_all(got, want, q)


def test_backward_bf16_io():
    """bf16 tensors and gates through the exact path, fp32 arithmetic inside: every gradient within half an output ulp (2^-8 relative,
    elementwise, plus a small absolute floor) of the oracle on the same bf16-rounded inputs."""
    announce("backward bf16 io, ViG-S head shape")
    q, k, v, gf, gb = make_gla_inputs(2, 3, 196, 32, 64, seed=12, dtype=torch.bfloat16)
    do = _do(v.shape, 9, torch.bfloat16)
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.25)
    got = vig_amd.gla_bidir_backward(*(t.cuda() for t in (q, k, v, gf, gb, do)), out_scale=0.25, exact=True)
    for name, g_, w_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, want):
        err = np.abs(f64(g_) - w_)
        assert np.all(err <= 2.0 ** -8 * np.abs(w_) + 1e-3 * np.abs(w_).max()), name


def test_autograd_through_the_wrappers():
    """loss.backward() through batch_bid_fused_chunk_gla (gates as one [2B,...] tensor) and fused_chunk_gla."""
    announce("autograd through the op wrappers")
    q, k, v, gf, gb = make_gla_inputs(2, 2, 70, 32, 64, seed=21)
    do = _do(v.shape, 10, torch.float32)
    tq, tk, tv = (t.cuda().requires_grad_(True) for t in (q, k, v))
    tg = torch.cat([gf, gb], 0).cuda().requires_grad_(True)
    o, _ = vig_amd.batch_bid_fused_chunk_gla(tq, tk, tv, tg)
    assert o.requires_grad
    (o * do.cuda()).sum().backward()
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    assert _rel(f64(tq.grad), want[0]) <= 1e-4 and _rel(f64(tk.grad), want[1]) <= 1e-4
    assert _rel(f64(tv.grad), want[2]) <= 1e-4
    assert _rel(f64(tg.grad[:2]), want[3]) <= 1e-4 and _rel(f64(tg.grad[2:]), want[4]) <= 1e-4
    # forward value of the recorded call equals the plain call
    with torch.no_grad():
        o2, _ = vig_amd.batch_bid_fused_chunk_gla(tq, tk, tv, tg)
    assert torch.equal(o.detach(), o2)
    # causal wrapper
    tq2 = q.cuda().requires_grad_(True)
    o3, _ = vig_amd.fused_chunk_gla(tq2, k.cuda(), v.cuda(), gf.cuda())
    (o3 * do.cuda()).sum().backward()
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), None, f64(do))
    assert _rel(f64(tq2.grad), want[0]) <= 1e-4


# ---- the matrix-core backward (bf16 tensors and gates, Dk in {32, 64}, Dv = 64, L <= 256) ----
MFMA_BWD_TOL = 2e-2  # max |error| over the gradient's largest magnitude (bf16 operands, fp32 accumulation)


def _check_mfma(got, want, q, tol=MFMA_BWD_TOL):
    floor = float(np.abs(f64(q) * want[0]).max())
    worst = {}
    for name, g_, w_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, want):
        assert np.isfinite(f64(g_)).all(), name
        worst[name] = _rel(f64(g_), w_, floor if name.startswith("dg") else 0.0)
    print("  " + " ".join(f"{k}:{v:.2e}" for k, v in worst.items()), flush=True)
    for name, e in worst.items():
        assert e <= tol, (name, e)


@pytest.mark.parametrize("B,H,L,Dk", [(2, 2, 1, 64), (1, 3, 17, 64), (2, 1, 32, 64), (1, 2, 33, 64), (2, 2, 64, 64),
                                      (2, 3, 196, 64), (1, 2, 255, 64), (1, 3, 256, 64), (2, 2, 1, 32), (1, 3, 33, 32),
                                      (2, 6, 196, 32), (1, 2, 256, 32)])
def test_backward_mfma_lengths(B, H, L, Dk):
    announce(f"backward on the matrix cores B{B} H{H} L={L} Dk={Dk}")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, Dk, 64, seed=500 + L, dtype=torch.bfloat16)
    do = _do(v.shape, 10, torch.bfloat16)
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    got = vig_amd.gla_bidir_backward(*(t.cuda() for t in (q, k, v, gf, gb, do)), out_scale=0.5)
    _check_mfma(got, want, q)


@pytest.mark.parametrize("Dk", [64, 32])
def test_backward_mfma_many_slabs_against_exact_path(Dk):
    """More slabs than workgroups (persistent loop), against the fp32-arithmetic kernel on the same inputs."""
    announce(f"backward on the matrix cores, 600 slabs, Dk={Dk}, against the recurrent kernel")
    q, k, v, gf, gb = (t.cuda() for t in make_gla_inputs(100, 6, 196, Dk, 64, seed=77, dtype=torch.bfloat16))
    do = _do(v.shape, 11, torch.bfloat16).cuda()
    want = [f64(t) for t in vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, out_scale=0.5, exact=True)]
    got = vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, out_scale=0.5)
    _check_mfma(got, want, q.cpu())


def test_backward_mfma_strong_gates_fall_back_per_slab():
    """Every third slab has gates beyond the quadratic form's range: those come from the recurrent kernel, bit for
    bit, the others from the matrix cores."""
    announce("backward, strong gates in every third slab")
    B, H, L = 4, 3, 196
    q, k, v, gf, gb = make_gla_inputs(B, H, L, 64, 64, seed=81, dtype=torch.bfloat16)
    _, _, _, sf, sb = make_gla_inputs(B, H, L, 64, 64, seed=82, dtype=torch.bfloat16, gate_scale=2.0)
    strong = (torch.arange(B * H).reshape(B, H) % 3 == 1)[:, :, None, None]
    gf, gb = torch.where(strong, sf, gf), torch.where(strong, sb, gb)
    do = _do(v.shape, 12, torch.bfloat16)
    dev = [t.cuda() for t in (q, k, v, gf, gb, do)]
    exact = vig_amd.gla_bidir_backward(*dev, out_scale=0.5, exact=True)
    got = vig_amd.gla_bidir_backward(*dev, out_scale=0.5)
    sel = strong[:, :, 0, 0].cuda()
    for name, g_, e_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, exact):
        assert torch.isfinite(g_.float()).all(), name
        assert torch.equal(g_[sel], e_[sel]), name
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    keep = ~strong[:, :, 0, 0].numpy()
    _check_mfma([g_.cpu()[keep] for g_ in got], [w_[keep] for w_ in want], q[keep])


def test_random_shapes_matrix_core_paths_against_exact_paths():
    """Forty random (B, H, L <= 256, Dk) shapes with gate strengths from ViG's /16 up to the reference tests'
    clamp_min(-3): forward and backward on the matrix cores (out-of-range slabs included, which go to the recurrent
    kernel slab by slab) against the fp32-arithmetic kernels on the same inputs."""
    announce("random shapes, forward and backward, matrix-core paths against the exact paths")
    rng = np.random.default_rng(7)
    for it in range(40):
        B, H, L = int(rng.integers(1, 9)), int(rng.integers(1, 7)), int(rng.integers(1, 257))
        Dk = int(rng.choice([32, 64]))
        gate_scale = float(rng.choice([1 / 16, 1 / 16, 0.25, 1.0]))
        q, k, v, gf, gb = (t.cuda() for t in make_gla_inputs(B, H, L, Dk, 64, seed=1000 + it, dtype=torch.bfloat16,
                                                             gate_scale=gate_scale))
        gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
        do = _do(v.shape, 2000 + it, torch.bfloat16).cuda()
        case = f"B{B} H{H} L{L} Dk{Dk} gates x{gate_scale}"
        o = vig_amd.gla_bidir_forward(q, k, v, gf, gb).float()
        oe = vig_amd.gla_bidir_forward(q, k, v, gf, gb, exact=True).float()
        assert bool(((o - oe).abs() <= 2e-2 + 2.0 ** -7 * oe.abs()).all()), case
        got = vig_amd.gla_bidir_backward(q, k, v, gf, gb, do)
        want = vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, exact=True)
        floor = float((q.float() * want[0].float()).abs().max())
        for name, g_, w_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, want):
            assert torch.isfinite(g_.float()).all(), (case, name)
            den = max(float(w_.float().abs().max()), floor if name.startswith("dg") else 0.0, 1e-30)
            assert float((g_.float() - w_.float()).abs().max()) / den <= MFMA_BWD_TOL, (case, name)


@pytest.mark.parametrize("B,H,L,Dk", [(2, 2, 1, 64), (1, 3, 33, 64), (2, 6, 196, 64), (1, 2, 256, 64), (2, 3, 70, 32),
                                      (3, 6, 196, 32), (80, 6, 196, 32)])
def test_backward_mfma_causal(B, H, L, Dk):
    """The one-direction (causal) op's backward on the matrix cores: the forward direction alone, against the adjoint
    recurrence for small cases and against the fp32-arithmetic kernel for the many-slab case."""
    announce(f"causal backward on the matrix cores B{B} H{H} L={L} Dk={Dk}")
    q, k, v, gf, _ = make_gla_inputs(B, H, L, Dk, 64, seed=900 + L + B, dtype=torch.bfloat16)
    do = _do(v.shape, 13, torch.bfloat16)
    dev = [t.cuda() for t in (q, k, v, gf)]
    got = vig_amd.gla_bidir_backward(*dev, None, do.cuda(), out_scale=1.0)
    assert got[4] is None
    if B * H <= 64:
        want = O.gla_recurrent_backward(f64(q), f64(k), f64(v), f64(gf), f64(do))
    else:
        want = [f64(t) for t in vig_amd.gla_bidir_backward(*dev, None, do.cuda(), out_scale=1.0, exact=True)[:4]]
    _check_mfma(got[:4], want, q)


@pytest.mark.parametrize("B,H,L,Dk,bidir", [(2, 2, 257, 64, True), (1, 3, 300, 64, True), (2, 2, 512, 64, True),
                                            (1, 2, 700, 64, True), (2, 3, 1030, 32, True), (1, 2, 300, 32, True),
                                            (2, 2, 300, 64, False), (1, 3, 1000, 32, False)])
def test_backward_mfma_long_sequences(B, H, L, Dk, bidir):
    """L > 256: the sequence as chained segments on the matrix cores (state passes, segment scan, one quadratic form
    per segment plus the products with the linking states), against the adjoint recurrences of the oracle."""
    announce(f"segmented backward on the matrix cores B{B} H{H} L={L} Dk={Dk} bidirectional={bidir}")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, Dk, 64, seed=600 + L, dtype=torch.bfloat16)
    do = _do(v.shape, 14, torch.bfloat16)
    if bidir:
        want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
        got = vig_amd.gla_bidir_backward(*(t.cuda() for t in (q, k, v, gf, gb, do)), out_scale=0.5)
        _check_mfma(got, want, q)
    else:
        want = O.gla_recurrent_backward(f64(q), f64(k), f64(v), f64(gf), f64(do))
        got = vig_amd.gla_bidir_backward(q.cuda(), k.cuda(), v.cuda(), gf.cuda(), None, do.cuda(), out_scale=1.0)
        assert got[4] is None
        _check_mfma(got[:4], want, q)


def test_backward_mfma_long_sequences_many_segments_against_exact_path():
    """More segments than workgroups and stronger gates (a state decays to nothing within a few segments), against the
    fp32-arithmetic kernel on the same inputs; and a second call on the same workspace-sized problem gives the same bits."""
    announce("segmented backward, 24 x 16 segments, against the recurrent kernel")
    q, k, v, gf, gb = (t.cuda() for t in make_gla_inputs(8, 3, 4096, 64, 64, seed=78, dtype=torch.bfloat16))
    do = _do(v.shape, 15, torch.bfloat16).cuda()
    want = [f64(t) for t in vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, out_scale=0.5, exact=True)]
    got = vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, out_scale=0.5)
    _check_mfma(got, want, q.cpu())
    again = vig_amd.gla_bidir_backward(q, k, v, gf, gb, do, out_scale=0.5)
    for a, b in zip(got, again):
        assert torch.equal(a, b)


def test_backward_mfma_long_sequences_strong_gates_fall_back_per_sequence():
    """One sequence of three has gates beyond the quadratic form's range in one of its segments: that whole sequence
    comes from the recurrent kernel, bit for bit, the others from the matrix cores."""
    announce("segmented backward, strong gates in one segment of one sequence")
    B, H, L = 1, 3, 600
    q, k, v, gf, gb = make_gla_inputs(B, H, L, 64, 64, seed=83, dtype=torch.bfloat16)
    _, _, _, sf, sb = make_gla_inputs(B, H, L, 64, 64, seed=84, dtype=torch.bfloat16, gate_scale=2.0)
    gf[:, 1, 400:], gb[:, 1, 400:] = sf[:, 1, 400:], sb[:, 1, 400:]
    do = _do(v.shape, 16, torch.bfloat16)
    dev = [t.cuda() for t in (q, k, v, gf, gb, do)]
    exact = vig_amd.gla_bidir_backward(*dev, out_scale=0.5, exact=True)
    got = vig_amd.gla_bidir_backward(*dev, out_scale=0.5)
    for name, g_, e_ in zip(("dq", "dk", "dv", "dg_fwd", "dg_bwd"), got, exact):
        assert torch.isfinite(g_.float()).all(), name
        assert torch.equal(g_[:, 1], e_[:, 1]), name
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    keep = [0, 2]
    _check_mfma([g_.cpu()[:, keep] for g_ in got], [w_[:, keep] for w_ in want], q[:, keep])


@pytest.mark.parametrize("B,H,L", [(2, 3, 128), (2, 3, 196), (1, 6, 784), (1, 3, 3136)])
def test_backward_hiervig_head_shape_on_the_matrix_cores(B, H, L):
    """HierViG's head shape (Dk 16, Dv 32, vig_h.py:521-527): the backward zero-padded to 32 / 64 channels on the
    matrix-core kernels (one slab for L <= 256, linked segments beyond), against the adjoint recurrences; a caller
    that sizes the workspace for the recurrent kernel only still gets that kernel (the exact path, bit for bit)."""
    announce(f"backward of the Dk16/Dv32 head shape B{B} H{H} L={L}")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, 16, 32, seed=700 + L, dtype=torch.bfloat16)
    do = _do(v.shape, 17, torch.bfloat16)
    dev = [t.cuda() for t in (q, k, v, gf, gb, do)]
    want = O.bidir_gla_backward(f64(q), f64(k), f64(v), f64(gf), f64(gb), f64(do), out_scale=0.5)
    got = vig_amd.gla_bidir_backward(*dev, out_scale=0.5)
    _check_mfma(got, want, q)
    exact = vig_amd.gla_bidir_backward(*dev, out_scale=0.5, exact=True)
    assert any(not torch.equal(a, b) for a, b in zip(got, exact))  # (it did take the other path)
    # through the C ABI with the smaller workspace: the recurrent kernel
    from vig_amd import _lib
    lib = _lib.load()
    small = lib.vig_gla_bidir_bwd_workspace(B, H, L, 16, 32, 1)
    assert small < lib.vig_gla_bidir_bwd_workspace_for(B, H, L, 16, 32, _lib.VIG_BF16, _lib.VIG_BF16, 1)
    ws = torch.empty(small, dtype=torch.uint8, device="cuda")
    outs = [torch.empty_like(t) for t in (dev[0], dev[1], dev[2], dev[3], dev[4])]
    rc = lib.vig_gla_bidir_bwd(*(t.data_ptr() for t in dev), *(t.data_ptr() for t in outs), ws.data_ptr(), small,
                               B, H, L, 16, 32, 16 ** -0.5, 0.5, _lib.VIG_BF16, _lib.VIG_BF16, None)
    assert rc == 0
    torch.cuda.synchronize()
    for a, b in zip(outs, exact):
        assert torch.equal(a, b)


def test_long_sequence_forward_and_backward_replay_as_a_graph():
    """The multi-launch paths of a long sequence (forward: state pass, segment scan, output pass; backward: dual
    state pass, segment scan, quadratic forms, flag pass) are plain kernel sequences on the caller's stream: captured
    as one HIP graph they reproduce the eager results bit for bit on every replay, with eager work and
    synchronisations between the replays and after the inputs change in place."""
    announce("L = 700 forward + backward captured as a HIP graph, 4 replays")
    q, k, v, gf, gb = (t.cuda() for t in make_gla_inputs(2, 3, 700, 64, 64, seed=91, dtype=torch.bfloat16))
    do = _do(v.shape, 18, torch.bfloat16).cuda()
    q2, k2, v2, gf2, gb2 = (t.cuda() for t in make_gla_inputs(2, 3, 700, 64, 64, seed=92, dtype=torch.bfloat16))
    static = [t.clone() for t in (q, k, v, gf, gb, do)]

    def run(ts):
        o = vig_amd.gla_bidir_forward(*ts[:5])
        return (o,) + tuple(vig_amd.gla_bidir_backward(*ts))

    want_a = [t.clone() for t in run([q, k, v, gf, gb, do])]
    want_b = [t.clone() for t in run([q2, k2, v2, gf2, gb2, do])]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(static)
    for i in range(4):
        src, want = (([q, k, v, gf, gb], want_a), ([q2, k2, v2, gf2, gb2], want_b))[i % 2]
        for dst, s_ in zip(static[:5], src):
            dst.copy_(s_)
        graph.replay()
        torch.cuda.synchronize()
        for name, g_, w_ in zip(("o", "dq", "dk", "dv", "dg_fwd", "dg_bwd"), outs, want):
            assert torch.equal(g_, w_), (i, name)
        run([q2, k2, v2, gf2, gb2, do])  # eager work between the replays
        torch.cuda.synchronize()


def test_autograd_keeps_the_exact_path():
    """gla_bidir_forward(exact=True) under autograd: the backward runs the fp32-arithmetic kernel too, bit-equal to
    gla_bidir_backward(exact=True) (and different from the matrix-core gradients of the default path)."""
    announce("autograd with exact=True, bf16")
    t = [x.cuda() for x in make_gla_inputs(2, 2, 196, 64, 64, seed=77, dtype=torch.bfloat16)]
    leaves = [x.clone().requires_grad_() for x in t]
    o = vig_amd.gla_bidir_forward(*leaves, exact=True)
    d_o = torch.randn_like(o)
    o.backward(d_o)
    want = vig_amd.gla_bidir_backward(*t, d_o, exact=True)
    other = vig_amd.gla_bidir_backward(*t, d_o, exact=False)
    for leaf, w in zip(leaves, want):
        assert torch.equal(leaf.grad, w)
    assert any(not torch.equal(a, b) for a, b in zip(want, other))


@pytest.mark.parametrize("dtype,L,Dk", [(torch.float32, 70, 32), (torch.float32, 150, 64), (torch.bfloat16, 196, 64),
                                        (torch.bfloat16, 300, 32)])
def test_causal_op_gradients_with_initial_state(dtype, L, Dk):
    """fused_chunk_gla(initial_state=S0, output_final_state=True) while autograd records: outputs, final state and the
    gradients of q, k, v, g (S0 a constant, as chunk_fuse.py:565-566 detaches it) against torch autograd through a
    float64 recurrence started from S0 on the same rounded inputs."""
    announce(f"causal op gradients with an initial state {dtype} L={L} Dk={Dk}")
    B, H, Dv = 2, 2, 64
    q, k, v, g, _ = make_gla_inputs(B, H, L, Dk, Dv, seed=71, dtype=dtype)
    gen = torch.Generator().manual_seed(72)
    s0 = torch.randn(B, H, Dk, Dv, generator=gen)
    do = torch.randn(B, H, L, Dv, generator=gen).to(dtype)
    # float64 reference: S_t = exp(g_t) * S_{t-1} + k_t v_t^T, o_t = scale q_t S_t (naive.py:13-44 with a start state)
    rq, rk, rv, rg = (t.double().requires_grad_(True) for t in (q, k, v, g))
    S = s0.double()
    outs = []
    for t in range(L):
        S = torch.exp(rg[:, :, t, :, None]) * S + rk[:, :, t, :, None] * rv[:, :, t, None, :]
        outs.append(torch.einsum("bhk,bhkv->bhv", rq[:, :, t] * Dk ** -0.5, S))
    ro = torch.stack(outs, 2)
    ro.backward(do.double())
    tq, tk, tv, tg = (t.cuda().requires_grad_(True) for t in (q, k, v, g))
    o, final = vig_amd.fused_chunk_gla(tq, tk, tv, tg, initial_state=s0.cuda(), output_final_state=True)
    assert final is not None and not final.requires_grad
    o.backward(do.cuda())
    fp32 = dtype == torch.float32
    scale_of = lambda w: max(1.0, float(w.abs().max()))
    assert (o.detach().double().cpu() - ro.detach()).abs().max() <= (1e-4 if fp32 else 2e-2) * scale_of(ro.detach())
    assert (final.double().cpu() - S.detach()).abs().max() <= (1e-4 if fp32 else 1e-2) * scale_of(S.detach())
    for name, got, want in (("dq", tq.grad, rq.grad), ("dk", tk.grad, rk.grad), ("dv", tv.grad, rv.grad), ("dg", tg.grad, rg.grad)):
        err = (got.double().cpu() - want).abs().max().item()
        assert err <= (1e-4 if fp32 else 2e-2) * scale_of(want), f"{name}: {err:.3e} against {scale_of(want):.3e}"
