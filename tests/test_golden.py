"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the oracle on the CPU and the
HIP path on the GPU against the same frozen vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import gla_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return dict(np.load(os.path.join(GOLDEN, name), allow_pickle=False))


def _f64(d, *names):
    return [d[n].astype(np.float64) for n in names]


@pytest.mark.parametrize("name", ["gla_f32_L37_D16_32.npz", "gla_f32_L70_D64_64.npz"])
def test_oracle_reproduces_gla_fixtures(name):
    d = _load(name)
    q, k, v, gf, gb = _f64(d, "q", "k", "v", "gf", "gb")
    np.testing.assert_allclose(O.bidir_gla_recurrent(q, k, v, gf, gb, out_scale=0.5), d["o_bidir_half"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.gla_recurrent(q, k, v, gf), d["o_causal"], rtol=1e-12, atol=1e-13)
    # the independently derived quadratic form agrees with the frozen recurrence output
    np.testing.assert_allclose(O.gla_parallel(q, k, v, gf), d["o_causal"], rtol=1e-9, atol=1e-10)


def test_oracle_reproduces_neighbour_fixtures():
    d = _load("neighbours_grid5x4.npz")
    hw, H = (5, 4), 2
    np.testing.assert_allclose(O.dirgate_reference(d["gk_lin"], H, 16.0), d["dirgate"], rtol=1e-12)
    np.testing.assert_allclose(O.dwconv3x3_reference(d["x"], d["conv_w"], hw, bias=d["conv_b"], silu=True), d["dwconv_silu"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.locality_blend_reference(d["o"], d["x"], d["glin"], d["w_g"], d["w_l"], eps=1e-6), d["blend"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.rmsnorm_residual_reference(d["x"], d["w_norm"], 1e-6, residual=d["residual"])[0], d["rmsnorm_y"], rtol=1e-12)
    np.testing.assert_allclose(O.swiglu_reference(d["gate_up"]), d["swiglu"], rtol=1e-12, atol=1e-13)


def _cuda(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["gla_f32_L37_D16_32.npz", "gla_f32_L70_D64_64.npz"])
def test_hip_gla_fp32_against_fixtures(name):
    import vig_amd
    print(f"[case] golden {name}", flush=True)
    d = _load(name)
    q, k, v, gf, gb = (_cuda(d[n]) for n in ("q", "k", "v", "gf", "gb"))
    got = vig_amd.gla_bidir_forward(q, k, v, gf, gb, out_scale=0.5).double().cpu().numpy()
    assert np.abs(got - d["o_bidir_half"]).max() / np.abs(d["o_bidir_half"]).max() <= 1e-4
    got, _ = vig_amd.fused_chunk_gla(q, k, v, gf)
    assert np.abs(got.double().cpu().numpy() - d["o_causal"]).max() / np.abs(d["o_causal"]).max() <= 1e-4


@pytest.mark.gpu
def test_hip_gla_bf16_against_fixture():
    import vig_amd
    print("[case] golden gla_bf16_L196_D32_64", flush=True)
    d = _load("gla_bf16_L196_D32_64.npz")
    q, k, v, gf, gb = (_cuda(d[n], torch.bfloat16) for n in ("q", "k", "v", "gf", "gb"))
    for n, t in zip(("q", "k", "v", "gf", "gb"), (q, k, v, gf, gb)):  # the fixture inputs are bf16-representable
        assert np.array_equal(t.float().cpu().numpy(), d[n])
    got = vig_amd.gla_bidir_forward(q, k, v, gf, gb, out_scale=0.25).double().cpu().numpy()
    assert np.abs(got - d["o_bidir_quarter"]).max() <= 2e-2


@pytest.mark.gpu
def test_hip_neighbours_against_fixtures():
    import vig_amd
    print("[case] golden neighbours_grid5x4", flush=True)
    d = _load("neighbours_grid5x4.npz")
    hw, H = (5, 4), 2
    close = lambda got, want, tol=2e-6: np.all(np.abs(got.double().cpu().numpy() - want) <= tol * np.maximum(1.0, np.abs(want)))
    assert close(vig_amd.dirgate(_cuda(d["gk_lin"]), H, 16.0), d["dirgate"])
    assert close(vig_amd.dirgate(_cuda(d["gk_lin"]), H, 16.0, clamp_min=-0.03), d["dirgate_clamped"])
    w = _cuda(d["conv_w"])
    assert close(vig_amd.dwconv3x3(_cuda(d["x"]), w, hw, bias=_cuda(d["conv_b"]), silu=True), d["dwconv_silu"])
    assert close(vig_amd.locality_gate(_cuda(d["o"]), w, hw), d["locality_gate"])
    assert close(vig_amd.locality_blend(_cuda(d["o"]), _cuda(d["x"]), _cuda(d["glin"]), _cuda(d["w_g"]), _cuda(d["w_l"]), eps=1e-6), d["blend"], 5e-6)
    assert close(vig_amd.rmsnorm(_cuda(d["x"]), _cuda(d["w_norm"]), 1e-6, residual=_cuda(d["residual"])), d["rmsnorm_y"])
    assert close(vig_amd.swiglu(_cuda(d["gate_up"])), d["swiglu"])
