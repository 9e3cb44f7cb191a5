"""GPU parity: the HIP path (through the C ABI) against the fp64 CPU oracle.

Tolerances (stated by the task): fp32 mode max|a-b|/max|b| <= 1e-4; bf16 mode
max|a-b| <= 2e-2 against the oracle run on the same bf16-rounded inputs.
"""
import numpy as np
import pytest
import torch

import vig_amd
from vig_amd.synthetic import CONFIGS, make_config_inputs, make_gla_inputs

from .util import bf16_grid_stats, announce, f64, max_abs, max_rel, oracle_bidir

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-4
BF16_TOL = 2e-2


def dev(*ts):
    return tuple(t.cuda() if t is not None else None for t in ts)


def test_cfg0_fp32_bidirectional():
    announce("cfg0 fp32 B2 H3 L197 D64 via vig_gla_bidir_fwd")
    q, k, v, gf, gb = make_config_inputs(0)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert max_rel(got, want) <= FP32_TOL


@pytest.mark.parametrize("L", [1, 2, 15, 16, 17, 63, 64, 65, 196, 197, 300])
def test_fp32_ragged_lengths(L):
    announce(f"fp32 ragged L={L}")
    q, k, v, gf, gb = make_gla_inputs(2, 2, L, 64, 64, seed=L)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert max_rel(got, want) <= FP32_TOL


@pytest.mark.parametrize("Dk,Dv", [(16, 32), (32, 64), (64, 32), (128, 64)])
def test_fp32_head_dims(Dk, Dv):
    announce(f"fp32 Dk={Dk} Dv={Dv}")
    q, k, v, gf, gb = make_gla_inputs(1, 3, 50, Dk, Dv, seed=7)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert max_rel(got, want) <= FP32_TOL


def test_fp32_strong_gates():
    """Gates as in the reference's op tests: logsigmoid(randn).clamp_min(-3), no /16 (tests/ops/test_gla.py)."""
    announce("fp32 strong gates L=300")
    q, k, v, gf, gb = make_gla_inputs(2, 2, 300, 64, 64, seed=3, gate_scale=1.0)
    gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert max_rel(got, want) <= FP32_TOL


def test_fp32_causal_only_and_wrappers():
    announce("fp32 causal-only + wrapper conventions")
    q, k, v, gf, gb = make_gla_inputs(2, 2, 70, 32, 64, seed=11)
    dq, dk_, dv_, dgf, dgb = dev(q, k, v, gf, gb)
    o, st = vig_amd.fused_chunk_gla(dq, dk_, dv_, dgf)
    assert st is None
    assert max_rel(f64(o), oracle_bidir(q, k, v, gf, None)) <= FP32_TOL
    g2 = torch.cat([dgf, dgb], dim=0)
    want_half = oracle_bidir(q, k, v, gf, gb, out_scale=0.5)
    o1, _ = vig_amd.batch_bid_fused_chunk_gla(dq, dk_, dv_, g2)
    o2, _ = vig_amd.bid_fused_recurrent_gla(dq, dk_, dv_, g2, None)
    assert max_rel(f64(o1), want_half) <= FP32_TOL
    assert max_rel(f64(o2), want_half) <= FP32_TOL
    of, orv = vig_amd.fused_recurrent_gla(dq, dk_, dv_, dgf, causal=False)
    # causal=False: the reverse sweep shares the forward gates (naive.py:46-58)
    from oracle import gla_oracle as O
    assert max_rel(f64(orv), O.gla_recurrent(f64(q), f64(k), f64(v), f64(gf), reverse=True)) <= FP32_TOL
    assert max_rel(f64(of), O.gla_recurrent(f64(q), f64(k), f64(v), f64(gf))) <= FP32_TOL


def test_fp32_zero_gate_closed_form():
    """g = 0: o = scale * (tril(QK^T) + triu(QK^T)) V -- library matmul, no oracle involved."""
    announce("fp32 g=0 closed form")
    q, k, v, _, _ = make_gla_inputs(1, 2, 100, 64, 64, seed=5)
    z = torch.zeros_like(q)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, z, z)))
    A = (q.double() @ k.double().transpose(-1, -2)) * (64 ** -0.5)
    want = ((torch.tril(A) + torch.triu(A)) @ v.double()).numpy()
    assert max_rel(got, want) <= FP32_TOL


@pytest.mark.parametrize("L", [1, 17, 196, 197])
def test_bf16_exact_path_small(L):
    announce(f"bf16 io through the fp32-arithmetic kernel L={L}")
    q, k, v, gf, gb = make_gla_inputs(2, 3, L, 64, 64, seed=100 + L, dtype=torch.bfloat16)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb), exact=True))
    assert max_abs(got, want) <= BF16_TOL


@pytest.mark.parametrize("L,Dk", [(1, 64), (5, 64), (16, 64), (49, 64), (64, 64), (65, 64), (196, 64), (197, 64),
                                   (256, 64), (257, 64), (300, 64), (196, 32), (197, 32), (700, 32)])
def test_bf16_default_path(L, Dk):
    announce(f"bf16 default (MFMA) path L={L} Dk={Dk}")
    q, k, v, gf, gb = make_gla_inputs(3, 2, L, Dk, 64, seed=200 + L, dtype=torch.bfloat16)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert max_abs(got, want) <= BF16_TOL


def test_bf16_causal_only():
    announce("bf16 default path, forward direction only")
    q, k, v, gf, _ = make_gla_inputs(2, 2, 196, 64, 64, seed=31, dtype=torch.bfloat16)
    want = oracle_bidir(q, k, v, gf, None)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, None)))
    assert max_abs(got, want) <= BF16_TOL


def test_bf16_zero_gate_closed_form():
    announce("bf16 g=0 closed form")
    q, k, v, _, _ = make_gla_inputs(1, 2, 196, 64, 64, seed=6, dtype=torch.bfloat16)
    z = torch.zeros_like(q)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, z, z)))
    A = (q.double() @ k.double().transpose(-1, -2)) * (64 ** -0.5)
    want = ((torch.tril(A) + torch.triu(A)) @ v.double()).numpy()
    # without decay |o| reaches ~10, where the bf16 output grid itself is coarser than 2e-2:
    # allow half an output ulp (2^-8 relative) on top of the absolute tolerance
    assert np.all(np.abs(got - want) <= BF16_TOL + 2.0 ** -8 * np.abs(want))


@pytest.mark.parametrize("gate_scale,L", [(0.25, 196), (1.0, 196), (1.0, 700)])
def test_bf16_strong_gates_default_path(gate_scale, L):
    """Gates far stronger than ViG's /16: chunk totals beyond what the fp16 score operands take, so the kernel has
    to fall back to its split-bf16 scores (per workgroup, from the first such segment on)."""
    announce(f"bf16 default path, strong gates x{gate_scale} L={L}")
    q, k, v, gf, gb = make_gla_inputs(3, 2, L, 64, 64, seed=41, dtype=torch.bfloat16, gate_scale=gate_scale)
    gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    assert max_abs(got, want) <= BF16_TOL


def test_bf16_mixed_gate_strength_many_items():
    """More (batch, head) slabs than workgroups, a few of them with strong gates: workgroups switch score variants
    at different items, and every slab still has to match."""
    announce("bf16 default path, 600 slabs, every 7th with strong gates")
    q, k, v, gf, gb = make_gla_inputs(100, 6, 196, 64, 64, seed=43, dtype=torch.bfloat16)
    _, _, _, sf, sb = make_gla_inputs(100, 6, 196, 64, 64, seed=44, dtype=torch.bfloat16, gate_scale=1.0)
    strong = (torch.arange(600).reshape(100, 6) % 7 == 3)[:, :, None, None]
    gf = torch.where(strong, sf.clamp_min(-3), gf)
    gb = torch.where(strong, sb.clamp_min(-3), gb)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    assert max_abs(got, want) <= BF16_TOL


@pytest.mark.parametrize("qs,ks,L,Dk,everywhere", [(2000.0, 1.0, 196, 64, True), (1.0, 3000.0, 196, 64, True),
                                                  (600.0, 600.0, 700, 64, True), (2000.0, 2000.0, 196, 32, True),
                                                  (30000.0, 1.0, 196, 64, False), (1.0, 30000.0, 300, 64, False)])
def test_bf16_large_magnitude_inputs(qs, ks, L, Dk, everywhere):
    """|q| or |k| beyond what the fp16 score operands hold (raw value x 2^6 must stay below 65504): ordinary bf16
    values, mild gates.  The kernel has to notice and take its split-bf16 scores; results finite and within the bf16
    bar relative to the output scale.  `everywhere` False: a single large element in one slab of many."""
    announce(f"bf16 default path, large inputs q x{qs} k x{ks} L={L} Dk={Dk} everywhere={everywhere}")
    q, k, v, gf, gb = make_gla_inputs(5, 2, L, Dk, 64, seed=51, dtype=torch.bfloat16)
    if everywhere:
        q, k = (q.float() * qs).bfloat16(), (k.float() * ks).bfloat16()
    else:
        q, k = q.clone(), k.clone()
        (q if qs > 1 else k)[3, 1, L // 2 + 7, 5] = max(qs, ks)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    # the absolute bar of unit-scale inputs, scaled with the outputs (their bf16 grid alone is 2^-8 relative)
    assert max_abs(got, want) <= BF16_TOL * max(1.0, np.abs(want).max() / 4.0)
    if not everywhere:  # the slabs without the large element keep the plain absolute bar
        ok = np.ones(5 * 2, dtype=bool)
        ok[3 * 2 + 1] = False
        d = np.abs(got - want).reshape(10, -1).max(axis=1)
        assert (d[ok] <= BF16_TOL).all()


@pytest.mark.parametrize("gate_scale,L,both", [(1.0, 196, True), (1.0 / 16, 196, True), (1.0, 700, True), (0.5, 130, False)])
def test_bf16_wide_entry_point(gate_scale, L, both):
    """vig_gla_bidir_fwd_wide (starts with the split-bf16 score variant): same accuracy bar on strong and on mild
    gates, slab and long-sequence modes, one or two directions."""
    announce(f"bf16 wide-range entry point, gates x{gate_scale} L={L} both={both}")
    q, k, v, gf, gb = make_gla_inputs(40, 2, L, 64, 64, seed=46, dtype=torch.bfloat16, gate_scale=gate_scale)
    gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
    if not both:
        gb = None
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb), strong_gates=True))
    assert np.isfinite(got).all()
    assert max_abs(got, want) <= BF16_TOL


@pytest.mark.parametrize("B,L", [(2, 300), (200, 196), (3, 64)])
def test_bf16_strong_gates_one_direction(B, L):
    """One direction only: half of the waves idle along and must keep the barrier count of the working half, also
    through the segment that refuses the fp16 variant and is walked again (several slabs per workgroup at B = 200)."""
    announce(f"bf16 default path, forward direction only, strong gates, B{B} L{L}")
    q, k, v, gf, _ = make_gla_inputs(B, 3, L, 64, 64, seed=45, dtype=torch.bfloat16, gate_scale=1.0)
    gf = gf.clamp_min(-3)
    want = oracle_bidir(q, k, v, gf, None)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, None)))
    assert np.isfinite(got).all()
    assert max_abs(got, want) <= BF16_TOL


def test_bf16_long_sequences_many_slabs_mixed_gate_strength():
    """More (sequence, segment) workgroups than the chip holds at once, every 7th sequence with gates too strong for
    the fp16 form: segments of one launch take different forms, and the states of a strongly gated sequence stay its own."""
    announce("bf16 long sequences, 240 sequences x 3 segments, mixed gate strength")
    B, H, L = 40, 6, 500
    q, k, v, gf, gb = make_gla_inputs(B, H, L, 32, 64, seed=91, dtype=torch.bfloat16)
    _, _, _, sf, sb = make_gla_inputs(B, H, L, 32, 64, seed=92, dtype=torch.bfloat16, gate_scale=1.0)
    strong = (torch.arange(B * H).reshape(B, H) % 7 == 3)[:, :, None, None]
    gf, gb = torch.where(strong, sf.clamp_min(-3), gf), torch.where(strong, sb.clamp_min(-3), gb)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    assert np.all(np.abs(got - want) <= BF16_TOL + 2.0 ** -8 * np.abs(want))


@pytest.mark.parametrize("L,Dk,both", [(257, 64, True), (449, 64, True), (1569, 64, True), (1000, 32, True),
                                       (480, 64, False), (2049, 32, False)])
def test_bf16_long_sequences_segment_edges(L, Dk, both):
    """Sequences cut into state-chained segments of whole 32-token tiles: lengths that leave the last segment with
    one token, with empty trailing tiles, with eight segments of seven tiles and one token more; one or two
    directions.  Mild gates, so that what crosses the segment edges carries weight."""
    announce(f"bf16 long sequence L={L} Dk={Dk} both={both}")
    q, k, v, gf, gb = make_gla_inputs(2, 3, L, Dk, 64, seed=700 + L, dtype=torch.bfloat16, gate_scale=1.0 / 32)
    if not both:
        gb = None
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    st = bf16_grid_stats(got, want)
    print(f"  max-abs err {max_abs(got, want):.3e} max|o| {np.abs(want).max():.2f} internal rms {st['internal_rms']:.2e}", flush=True)
    assert np.all(np.abs(got - want) <= BF16_TOL + 2.0 ** -8 * np.abs(want))


def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        L = int(rng.choice([rng.integers(1, 33), rng.integers(33, 257), rng.integers(257, 900)]))
        out.append((int(rng.integers(1, 4)), int(rng.integers(1, 4)), L, int(rng.choice([32, 64])),
                    float(rng.choice([1 / 64, 1 / 16, 1 / 4, 1.0])), bool(rng.integers(0, 2)), 9000 + i))
    return out


@pytest.mark.parametrize("B,H,L,Dk,gate_scale,both,seed", _random_shapes(36, 2024))
def test_bf16_random_shapes(B, H, L, Dk, gate_scale, both, seed):
    """Seeded random shapes across the slab / long-sequence boundary, both head widths, one or two directions, gates
    from mild to strong (the fp16 form, the general form and mixtures of them within one launch)."""
    announce(f"bf16 random shape B{B} H{H} L{L} Dk{Dk} gates x{gate_scale} both={both} seed={seed}")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, Dk, 64, seed=seed, dtype=torch.bfloat16, gate_scale=gate_scale)
    gf, gb = gf.clamp_min(-3), (gb.clamp_min(-3) if both else None)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    assert np.all(np.abs(got - want) <= BF16_TOL + 2.0 ** -8 * np.abs(want))


@pytest.mark.parametrize("vscale,gate_scale", [(1000.0, 1.0 / 64), (1e-4, 1.0 / 64), (1000.0, 1.0)])
def test_bf16_long_sequence_state_magnitudes(vscale, gate_scale):
    """States entering the segments far above and far below 1 (they reach the matrix cores as fp16, scaled by a power of
    two when the scan saw anything above 2^14 or nothing above 2^-4), with weak gates and with gates strong enough for
    the general form: same-signed keys and values make every state element grow with the history."""
    announce(f"bf16 long sequence, states scaled: v x{vscale}, gates x{gate_scale}")
    q, k, v, gf, gb = make_gla_inputs(2, 2, 900, 64, 64, seed=77, dtype=torch.bfloat16, gate_scale=gate_scale)
    k, v = k.abs(), (v.float().abs() * vscale).bfloat16()
    if gate_scale >= 1.0:
        gf, gb = gf.clamp_min(-3), gb.clamp_min(-3)
    want = oracle_bidir(q, k, v, gf, gb)
    got = f64(vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb)))
    assert np.isfinite(got).all()
    top = np.abs(want).max()
    print(f"  max|o| {top:.3e} max-abs err {max_abs(got, want):.3e}", flush=True)
    # the bf16 output grid (2^-8 relative) and the operands' roundings, relative to the output scale
    assert np.all(np.abs(got - want) <= BF16_TOL * top / 4.0 + 2.0 ** -8 * np.abs(want))


# (internal rms error, fraction of large outputs off the correctly rounded oracle value, grid steps such an output may
# be off) allowed per named workload: about 2.5 times what the shipped arithmetic measures (2.7e-4 / 5.2 % on the three
# 196-token workloads bar the Dk = 32 one, 3.7e-4 / 6.3 %; the same 2.7e-4 / 5.2 % on the state-chained 4096-token
# workload).  An internal error of 1e-3 (e.g. score operands or state fragments rounded to bf16: that workload measured
# 5.4e-4 / 9.4 % with bf16 state fragments) passes the 2e-2 max-abs bar and fails these.
INTERNAL_BOUNDS = {1: (7e-4, 0.13, 1), 2: (7e-4, 0.13, 1), 3: (7e-4, 0.13, 1), 4: (9.5e-4, 0.16, 1)}


@pytest.mark.parametrize("idx,batch", [(1, None), (2, None), (3, None), (4, None)])
def test_bf16_named_configs_full_size(idx, batch):
    """Full-size named workloads against the oracle (the oracle finishes these in seconds)."""
    s = CONFIGS[idx]
    announce(f"bf16 {s.name} batch={batch or s.B}")
    q, k, v, gf, gb = make_config_inputs(idx, batch=batch)
    want = oracle_bidir(q, k, v, gf, gb)
    o = vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb))
    got = f64(o)
    err = max_abs(got, want)
    st = bf16_grid_stats(got, want)
    print(f"  {s.name}: max-abs err {err:.3e}  max|o| {np.abs(want).max():.3f}  internal error (outputs below 2^-5) rms "
          f"{st['internal_rms']:.2e} max {st['internal_max']:.2e}; outputs >= 0.5: {100 * st['frac_off']:.2f} % off the "
          f"rounded oracle, worst {st['max_steps_large']:.2f} grid steps", flush=True)
    assert err <= BF16_TOL
    # resolution below the output grid: the kernel's own error, read off the small outputs (where the bf16 grid is
    # fine) and off the share of large outputs that miss the correctly rounded oracle value (never by more than one
    # grid step); bounds about three times the measured figures
    rms_bound, frac_bound, steps_bound = INTERNAL_BOUNDS[idx]
    assert st["internal_rms"] <= rms_bound, f"internal rms error {st['internal_rms']:.2e} (bound {rms_bound:.1e})"
    assert st["frac_off"] <= frac_bound, f"{100 * st['frac_off']:.2f} % of large outputs off the rounded oracle"
    assert st["max_steps_large"] <= steps_bound + 1e-9
    # size-independent properties at full size: linearity in v and determinism
    o2 = vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb))
    assert torch.equal(o, o2), "kernel is not deterministic"
    # odd symmetry in v (linearity); matrix-core accumulation is not guaranteed sign-symmetric to the last
    # bit, so allow one output ulp
    o_neg = vig_amd.gla_bidir_forward(*dev(q, k, -v, gf, gb))
    asym = (o_neg.float() + o.float()).abs().max().item()
    assert asym <= 2.0 ** -7 * float(np.abs(want).max()), f"odd symmetry in v violated: {asym}"


def test_bf16_flip_symmetry_full_size():
    """bwd(x, g) == flip(fwd(flip x, flip g)) at the ViG-S shape, bit-exact is not required (<= 2 bf16 roundings)."""
    announce("bf16 flip symmetry cfg1 quarter batch")
    q, k, v, gf, gb = make_config_inputs(1, batch=32)
    dq, dk_, dv_, dgf, dgb = dev(q, k, v, gf, gb)
    a = vig_amd.gla_bidir_forward(dq, dk_, dv_, dgf, dgb)
    fl = lambda x: x.flip(dims=[2]).contiguous()
    b = fl(vig_amd.gla_bidir_forward(fl(dq), fl(dk_), fl(dv_), fl(dgb), fl(dgf)))
    assert (a.float() - b.float()).abs().max().item() <= BF16_TOL


@pytest.mark.parametrize("B,H,L", [(2, 3, 128), (2, 3, 196), (1, 6, 784), (1, 3, 3136)])
def test_bf16_hiervig_head_shape_on_the_matrix_cores(B, H, L):
    """Dk 16 / Dv 32 (HierViG) from L = 128 on: zero-padded to Dk 32 / Dv 64 inside the library; against the oracle,
    and against the fp32-arithmetic kernel on the same inputs."""
    announce(f"bf16 Dk=16 Dv=32 B{B} H{H} L={L} (padded onto the matrix-core kernel)")
    q, k, v, gf, gb = make_gla_inputs(B, H, L, 16, 32, seed=600 + L, dtype=torch.bfloat16)
    want = oracle_bidir(q, k, v, gf, gb)
    got = vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb))
    assert got.shape == (B, H, L, 32)
    # |o| reaches ~5 here (k is scaled by 16^-0.5 only), where the bf16 output grid alone is coarser than 2e-2:
    # allow half an output ulp (2^-8 relative) on top of the absolute tolerance
    assert np.all(np.abs(f64(got) - want) <= BF16_TOL + 2.0 ** -8 * np.abs(want))
    exact = vig_amd.gla_bidir_forward(*dev(q, k, v, gf, gb), exact=True)
    assert np.all(np.abs(f64(got) - f64(exact)) <= BF16_TOL + 2.0 ** -7 * np.abs(want))
    assert not torch.equal(got, exact)  # (the two kernels round differently: proves the padded path ran)


@pytest.mark.parametrize("B,H,L,Dk,both", [(3, 6, 196, 32, True), (2, 3, 196, 64, True), (2, 2, 37, 64, True),
                                           (1, 4, 256, 32, False), (130, 2, 100, 64, True)])
def test_q_k_v_read_in_place_from_projection_rows(B, H, L, Dk, both):
    """vig_gla_bidir_fwd_strided: q, k, v as head-split views of one [B, L, H*(2*Dk + Dv) + extra] matrix (the stacked
    input projection's output, classification/models/vig.py:436-438) give bit for bit the result of the op on
    contiguous copies, and the op is checked against the oracle on the same inputs; views the kernel cannot read in
    place (rows off a 16-byte boundary, long sequences) are copied by the Python op."""
    announce(f"strided q/k/v B={B} H={H} L={L} Dk={Dk} both={both}")
    from vig_amd import _lib, ops
    Dv = 64
    q, k, v, gf, gb = (t.bfloat16() for t in dev(*make_gla_inputs(B, H, L, Dk, Dv, seed=31 + L)))
    if not both:
        gb = None
    row = H * (2 * Dk + Dv) + 24  # (other column blocks follow in the same rows)
    z = torch.randn(B, L, row, device="cuda").bfloat16()
    z[..., :H * Dk] = q.transpose(1, 2).reshape(B, L, H * Dk)
    z[..., H * Dk:2 * H * Dk] = k.transpose(1, 2).reshape(B, L, H * Dk)
    z[..., 2 * H * Dk:2 * H * Dk + H * Dv] = v.transpose(1, 2).reshape(B, L, H * Dv)
    qs, ks, vs = (t.unflatten(-1, (H, d)).transpose(1, 2)
                  for t, d in zip(z[..., :H * (2 * Dk + Dv)].split((H * Dk, H * Dk, H * Dv), -1), (Dk, Dk, Dv)))
    assert not qs.is_contiguous() and torch.equal(qs, q) and torch.equal(vs, v)
    want = vig_amd.gla_bidir_forward(q, k, v, gf, gb)
    assert ops._head_view_strides(ks) == (L * row, Dk, row)
    got = vig_amd.gla_bidir_forward(qs, ks, vs, gf, gb)
    assert torch.equal(got, want)
    # one strided operand among contiguous ones
    assert torch.equal(vig_amd.gla_bidir_forward(q, ks, v, gf, gb), want)
    if B * H * L <= 4000:
        ref = oracle_bidir(q, k, v, gf, gb)
        assert max_abs(f64(got), ref) <= BF16_TOL
    # the C ABI refuses what the slab kernel does not take
    lib = _lib.load()
    import ctypes
    st = (ctypes.c_longlong * 3)(L * row, Dk, row)
    sv = (ctypes.c_longlong * 3)(L * row, Dv, row)
    bad = (ctypes.c_longlong * 3)(L * row, Dk, row + 4)
    out = torch.empty_like(v)

    def call(sq, L_arg=L):
        return lib.vig_gla_bidir_fwd_strided(qs.data_ptr(), ks.data_ptr(), vs.data_ptr(), gf.data_ptr(),
                                             gb.data_ptr() if both else None, out.data_ptr(), B, H, L_arg, Dk, Dv,
                                             ctypes.addressof(sq), ctypes.addressof(st), ctypes.addressof(sv), Dk ** -0.5,
                                             1.0, _lib.VIG_BF16, _lib.VIG_BF16, ops._stream_ptr(q))
    assert call(st) == _lib.VIG_OK
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert call(bad) == _lib.VIG_EINVAL
    assert call(st, 300) == _lib.VIG_ENOTSUP


def test_strided_views_refuse_bad_out_and_gates():
    """Head-split views take the in-place path, which must refuse what the dense path refuses: an `out` of the wrong
    shape or dtype and a reverse gate tensor that does not match the forward one raise before any kernel sees them."""
    announce("in-place path: bad out / g_bwd raise")
    B, H, L, Dk = 2, 3, 40, 64
    qkv = torch.randn(B, L, H * (2 * Dk + 64)).bfloat16().cuda()
    q, k, v = (qkv[..., i * H * 64:(i + 1) * H * 64].unflatten(-1, (H, 64)).transpose(1, 2) for i in range(3))
    gf = (-torch.rand(B, H, L, Dk) / 16).bfloat16().cuda()
    ok = vig_amd.gla_bidir_forward(q, k, v, gf, gf.clone())
    assert ok.shape == (B, H, L, 64)
    with pytest.raises(ValueError):
        vig_amd.gla_bidir_forward(q, k, v, gf, gf.clone(), out=torch.empty(B, H, L - 8, 64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        vig_amd.gla_bidir_forward(q, k, v, gf, gf.clone(), out=torch.empty(B, H, L, 64, dtype=torch.float32, device="cuda"))
    with pytest.raises(ValueError):
        vig_amd.gla_bidir_forward(q, k, v, gf, gf[:, :, :L - 8].contiguous())
    with pytest.raises(ValueError):
        vig_amd.gla_bidir_forward(q, k, v, gf, gf.float())


def test_pointers_off_a_16_byte_boundary():
    """The library refuses a tensor that does not start on a 16-byte boundary (nothing is enqueued); the Python op
    copies such a view first and gives the result of the aligned call."""
    announce("misaligned views: C ABI refuses, Python op copies")
    from vig_amd import _lib, ops
    lib = _lib.load()
    B, H, L, D = 2, 2, 70, 64
    q, k, v, gf, gb = (t.bfloat16() for t in dev(*make_gla_inputs(B, H, L, D, D, seed=5)))
    want = vig_amd.gla_bidir_forward(q, k, v, gf, gb)

    def shifted(t):  # the same values in a view that starts one element into its storage
        flat = torch.empty(t.numel() + 8, dtype=t.dtype, device=t.device)
        flat[1:1 + t.numel()] = t.reshape(-1)
        view = flat[1:1 + t.numel()].view(t.shape)
        assert view.is_contiguous() and view.data_ptr() % 16 == 2
        return view

    got = vig_amd.gla_bidir_forward(shifted(q), k, shifted(v), gf, shifted(gb))
    assert torch.equal(got, want)
    out = torch.empty_like(v)
    ws_bytes = lib.vig_gla_bidir_fwd_workspace(B, H, L, D, D, _lib.VIG_BF16)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    args = dict(q=q, k=k, v=v, gf=gf, gb=gb, out=out)
    for name in args:
        a = dict(args)
        a[name] = shifted(args[name])
        rc = lib.vig_gla_bidir_fwd(a["q"].data_ptr(), a["k"].data_ptr(), a["v"].data_ptr(), a["gf"].data_ptr(),
                                   a["gb"].data_ptr(), a["out"].data_ptr(), ws.data_ptr(), ws_bytes, B, H, L, D, D,
                                   D ** -0.5, 1.0, _lib.VIG_BF16, _lib.VIG_BF16, ops._stream_ptr(q))
        assert rc == _lib.VIG_EINVAL, name
    with pytest.raises(ValueError):
        vig_amd.gla_bidir_forward(q, k, v, gf, gb, out=shifted(out))
    x = shifted(torch.randn(40, 384, device="cuda").bfloat16())
    w = torch.ones(384, device="cuda")
    assert torch.equal(ops.rmsnorm(x, w), ops.rmsnorm(x.clone(), w))
    assert lib.vig_rmsnorm_fwd(x.data_ptr(), None, w.data_ptr(), torch.empty_like(x).data_ptr(), None, 40, 384,
                               1e-6, 0, _lib.VIG_BF16, ops._stream_ptr(x)) == _lib.VIG_EINVAL


@pytest.mark.parametrize("dtype,L,Dk,Dv", [(torch.float32, 70, 32, 64), (torch.float32, 300, 64, 64), (torch.bfloat16, 196, 64, 64),
                                           (torch.bfloat16, 64, 32, 64), (torch.bfloat16, 700, 64, 64), (torch.bfloat16, 1000, 32, 64),
                                           (torch.bfloat16, 50, 16, 32)])
def test_causal_op_with_initial_and_final_state(dtype, L, Dk, Dv):
    """fused_chunk_gla(initial_state=, output_final_state=True) against the oracle's recurrence started from the same
    state (chunk_fuse.py:70-72,99-101); also state passing: the second half of a sequence started from the first
    half's final state reproduces the whole sequence (outputs and final state)."""
    announce(f"causal op with states {dtype} L={L} Dk={Dk} Dv={Dv}")
    from oracle import gla_oracle as O
    B, H = 3, 2
    q, k, v, gf, _ = make_gla_inputs(B, H, L, Dk, Dv, seed=61, dtype=dtype)
    gen = torch.Generator().manual_seed(62)
    s0 = torch.randn(B, H, Dk, Dv, generator=gen)
    want_o, want_s = O.gla_recurrent(f64(q), f64(k), f64(v), f64(gf), initial_state=f64(s0), return_state=True)
    o, s = vig_amd.fused_chunk_gla(*dev(q, k, v, gf), initial_state=s0.cuda(), output_final_state=True)
    assert s.dtype == torch.float32 and tuple(s.shape) == (B, H, Dk, Dv)
    if dtype == torch.float32:
        assert max_rel(f64(o), want_o) <= FP32_TOL and max_rel(f64(s), want_s) <= FP32_TOL
    else:
        assert max_abs(f64(o), want_o) <= BF16_TOL * max(1.0, np.abs(want_o).max() / 4.0)
        assert max_rel(f64(s), want_s) <= 1e-2  # the state accumulates bf16-rounded operands in fp32
    # no state in: the plain causal op; final state only
    o1, s1 = vig_amd.fused_chunk_gla(*dev(q, k, v, gf), output_final_state=True)
    o_plain, none = vig_amd.fused_chunk_gla(*dev(q, k, v, gf))
    assert none is None
    tol = FP32_TOL if dtype == torch.float32 else 1e-2
    assert max_rel(f64(o1), f64(o_plain)) <= tol
    # state passing across a split of the sequence
    cut = L // 2
    a = [t[:, :, :cut].contiguous() for t in (q, k, v, gf)]
    b = [t[:, :, cut:].contiguous() for t in (q, k, v, gf)]
    oa, sa = vig_amd.fused_chunk_gla(*dev(*a), output_final_state=True)
    ob, sb = vig_amd.fused_chunk_gla(*dev(*b), initial_state=sa, output_final_state=True)
    whole = f64(o1)
    assert max_rel(np.concatenate([f64(oa), f64(ob)], axis=2), whole) <= (FP32_TOL if dtype == torch.float32 else 2e-2)
    assert max_rel(f64(sb), f64(s1)) <= (FP32_TOL if dtype == torch.float32 else 1e-2)
    # the recurrent wrapper carries states too, in fp32 arithmetic
    o2, s2 = vig_amd.fused_recurrent_gla(*dev(q, k, v, gf), initial_state=s0.cuda(), output_final_state=True)
    if dtype == torch.float32:
        assert max_rel(f64(o2), want_o) <= FP32_TOL and max_rel(f64(s2), want_s) <= FP32_TOL
    else:
        assert max_rel(f64(s2), want_s) <= 1e-5
