"""Host-side behaviour that needs no GPU: the bench driver's contract, the op wrappers' argument checks, the
workspace arithmetic of the C ABI and the dispatch rules of the fused-gate wrapper."""
import json
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)


def test_workspace_sizes():
    from vig_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built here")
    lib = _lib.load()
    ws = lib.vig_gla_bidir_fwd_workspace
    state = (64 * 64 + 64) * 4 * 2  # one fp32 state + decays per (sequence, segment, direction)
    assert ws(128, 6, 196, 64, 64, 1) == 128 * 6 * 196 * 64 * 4          # bf16: the exact path's fp32 accumulator
    assert ws(2, 3, 197, 64, 64, 0) == 0                                  # fp32 tensors accumulate in the output
    assert ws(8, 3, 4096, 64, 64, 1) >= 8 * 3 * 16 * state               # long sequences: segment states
    # Dk 16 / Dv 32 from L = 128 on: padded copies of q, k, two gates (32 channels) and v, o (64 channels), bf16
    pad = (4 * 32 + 2 * 64) * 2
    assert ws(4, 3, 196, 16, 32, 1) == max(4 * 3 * 196 * pad, 4 * 3 * 196 * 32 * 4)
    assert ws(4, 3, 64, 16, 32, 1) == 4 * 3 * 64 * 32 * 4                 # short: recurrent kernel only
    wb = lib.vig_gla_bidir_bwd_workspace
    n_qk, n_v = 2 * 3 * 50 * 64, 2 * 3 * 50 * 64
    assert wb(2, 3, 50, 64, 64, 1) == (3 * n_qk + n_v) * 4 + 2 * 3 * 4   # recurrent scratch + one flag per slab
    assert wb(2, 3, 50, 128, 64, 1) == 0                                  # no backward for Dk = 128
    # L > 256 on the matrix cores: behind the 256-byte aligned scratch + flags, per (sequence, segment, direction) two
    # state-pass slots, the S_in Q terms and carries (fp32) and three bf16 64 x 64 matrices
    n_qk = n_v = 2 * 3 * 600 * 64
    base = ((3 * n_qk + n_v) * 4 + 2 * 3 * 4 + 255) // 256 * 256
    slots = 2 * 3 * 3 * 2
    assert wb(2, 3, 600, 64, 64, 1) == base + slots * ((2 * (4096 + 64) + 4096 + 128) * 4 + 3 * 4096 * 2)
    assert wb(2, 3, 600, 64, 32, 1) == (3 * n_qk + n_v // 2) * 4 + 2 * 3 * 4  # Dv = 32: recurrent kernel only


def test_wrappers_reject_what_is_not_built():
    import vig_amd

    q = torch.zeros(1, 1, 4, 64)
    with pytest.raises(NotImplementedError):
        vig_amd.fused_recurrent_gla(q, q, q, q, gv=q)
    with pytest.raises(NotImplementedError):  # a state in or out belongs to the causal op (recurrent_fuse.py:650-652)
        vig_amd.fused_recurrent_gla(q, q, q, q, output_final_state=True, causal=False)
    with pytest.raises(NotImplementedError):
        vig_amd.batch_bid_fused_chunk_gla(q, q, q, torch.cat([q, q]), initial_state=torch.zeros(1, 1, 64, 64))
    from vig_amd._lib import VigGlaError
    with pytest.raises(VigGlaError):  # CPU tensors: there is no CPU path, and the wrappers say so
        vig_amd.gla_bidir_locality_gate(q, q, q, q, q, torch.zeros(64, 1, 3, 3), (2, 2))


def test_layers_mirror_the_reference_constructors():
    from vig_amd import layers

    with pytest.raises(AssertionError):
        layers.GatedLinearAttention(d_model=64, num_heads=2, mode="no_such_mode")
    with pytest.raises(NotImplementedError):
        layers.GatedLinearAttention(d_model=64, num_heads=2, rope_mode="2dv1")
    m = layers.GLA2D(d_model=96, expand_k=0.5, expand_v=1.0, num_heads=3, channel_first=True)
    assert (m.head_qk_dim, m.head_v_dim, m.channel_first, m.d_group) == (16, 32, True, 2)
    mlp = layers.GLAMLP(384)
    assert mlp.intermediate_size == 1024  # 4 * 384 * 2 / 3 rounded up to a multiple of 256 (vig.py:480-483)


def test_checkpoint_variants_and_cache_invalidation(tmp_path):
    """'model' / 'model_ema' / bare state dicts / a 'module.' prefix (classification/utils/utils.py:17-103), and the
    derived weight copies of the layers do not survive a load or a train()/eval() switch."""
    from vig_amd import evaluate, layers

    torch.manual_seed(0)
    kw = dict(img_size=32, depth=1, num_heads=2, embed_dim=64, num_classes=5)
    a, b = layers.ViG(**kw), layers.ViG(**kw)
    with torch.no_grad():
        for p in b.parameters():
            p.add_(1.0)
    path = str(tmp_path / "c.pth")
    torch.save({"model": a.state_dict(), "model_ema": {"module." + k: v for k, v in b.state_dict().items()},
                "max_accuracy": 1.0, "epoch": 2}, path)
    m = layers.ViG(**kw)
    evaluate.load_checkpoint(m, path)
    assert all(torch.equal(x, y) for x, y in zip(m.state_dict().values(), a.state_dict().values()))
    evaluate.load_checkpoint(m, path, use_ema=True)
    assert all(torch.equal(x, y) for x, y in zip(m.state_dict().values(), b.state_dict().values()))
    torch.save({"model": a.state_dict()}, path)          # no EMA copy in the file: 'model' serves (utils.py:73)
    evaluate.load_checkpoint(m, path, use_ema=True)
    assert all(torch.equal(x, y) for x, y in zip(m.state_dict().values(), a.state_dict().values()))
    torch.save(b.state_dict(), path)                       # bare state dict
    evaluate.load_checkpoint(m, path)
    assert all(torch.equal(x, y) for x, y in zip(m.state_dict().values(), b.state_dict().values()))
    # caches: filled by hand here (no GPU), gone after a load, after train()/eval() and after invalidate_caches
    # (bf16 parameters, so that the fp32 copy is a tensor of its own)
    m, a = m.to(torch.bfloat16), a.to(torch.bfloat16)
    norm = m.blocks[0].attn_norm
    norm._w32()
    assert "_w32_cache" in norm.__dict__
    m.load_state_dict(a.state_dict())
    assert "_w32_cache" not in norm.__dict__
    norm._w32()
    m.train()
    assert "_w32_cache" not in norm.__dict__
    norm._w32()
    norm.weight.data.mul_(2.0)  # behind the version counter: the stale copy would survive ...
    assert torch.equal(norm._w32(), norm.weight.detach().float() / 2)
    layers.invalidate_caches(m)  # ... until the caller says so
    assert torch.equal(norm._w32(), norm.weight.detach().float())
