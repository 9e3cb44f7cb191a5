"""Seeded synthetic inputs for the bidirectional GLA workloads.

The distributions mirror what ViG's block feeds the op
(classification/models/vig.py:432-441): q, k, v ~ N(0,1) with k pre-scaled by
Dk^-0.5, and per-direction log-gates logsigmoid(N(0,1))/16.  Everything is drawn
on the CPU from one torch.Generator so the GPU box and the CPU checker see the
same numbers; draw order is q, k, v, g_fwd, g_bwd.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F


@dataclass(frozen=True)
class GLAShape:
    name: str
    B: int
    H: int
    L: int
    Dk: int
    Dv: int
    dtype: str  # "f32" | "bf16"
    grid: tuple | None = None  # (h, w) token grid when L == h*w

    @property
    def tokens(self) -> int:
        return self.B * self.H * self.L

    def alg_flops(self) -> int:
        """8*Dk*Dv per token: k v^T accumulate + q S read-out, both directions."""
        return self.tokens * 8 * self.Dk * self.Dv

    def alg_bytes(self, gate_bytes: int | None = None) -> int:
        """q,k,v,o once + the two gate tensors once."""
        io = 4 if self.dtype == "f32" else 2
        gb = io if gate_bytes is None else gate_bytes
        return self.tokens * (io * (2 * self.Dk + 2 * self.Dv) + gb * 2 * self.Dk)


# The named workloads (index = seed offset).
CONFIGS = {
    0: GLAShape("cfg0_cpu_plumbing_B2_H3_L197_D64_f32", 2, 3, 197, 64, 64, "f32", None),
    1: GLAShape("cfg1_vig_s_B128_H6_L196_D64_bf16", 128, 6, 196, 64, 64, "bf16", (14, 14)),
    2: GLAShape("cfg2_vig_b_B64_H12_L196_D64_bf16", 64, 12, 196, 64, 64, "bf16", (14, 14)),
    3: GLAShape("cfg3_vig_t_hires_B8_H3_L4096_D64_bf16", 8, 3, 4096, 64, 64, "bf16", (64, 64)),
    4: GLAShape("cfg4_vig_s_layer_B256_H6_L196_Dk32_Dv64_bf16", 256, 6, 196, 32, 64, "bf16", (14, 14)),
}


def torch_dtype(name: str) -> torch.dtype:
    return {"f32": torch.float32, "bf16": torch.bfloat16}[name]


def make_gla_inputs(B, H, L, Dk, Dv, seed, dtype=torch.float32, gate_scale=1.0 / 16.0):
    """Returns (q, k, v, g_fwd, g_bwd) as CPU tensors of `dtype`.

    Generated in float32 and rounded once to `dtype`; a checker must consume the
    rounded tensors (input rounding alone moves bf16 outputs by ~1e-2).
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, H, L, Dk, generator=gen)
    k = torch.randn(B, H, L, Dk, generator=gen) * (Dk ** -0.5)
    v = torch.randn(B, H, L, Dv, generator=gen)
    gf = F.logsigmoid(torch.randn(B, H, L, Dk, generator=gen)) * gate_scale
    gb = F.logsigmoid(torch.randn(B, H, L, Dk, generator=gen)) * gate_scale
    return tuple(t.to(dtype).contiguous() for t in (q, k, v, gf, gb))


def make_config_inputs(idx: int, batch: int | None = None, seed_offset: int = 0):
    """Inputs of named workload `idx` (seed 1000+idx); `batch` overrides B."""
    s = CONFIGS[idx]
    B = s.B if batch is None else batch
    return make_gla_inputs(B, s.H, s.L, s.Dk, s.Dv, 1000 + idx + seed_offset, torch_dtype(s.dtype))


def make_locality_weight(C: int, seed: int, dtype=torch.float32):
    """3x3 depthwise weights ~ N(0, 1/9), shape [C, 1, 3, 3]."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(C, 1, 3, 3, generator=gen) / 3.0).to(dtype).contiguous()
