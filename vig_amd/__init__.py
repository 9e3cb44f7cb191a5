"""vig_amd: MI355X (gfx950) bidirectional gated-linear-attention forward for ViG.

The compute lives in vig_amd/lib/libvig_gla.so (HIP, C ABI in include/vig_gla.h);
this package is the Python host side that mirrors the reference's op and block
interfaces over it.
"""
from . import ops  # noqa: F401
from .ops import (  # noqa: F401
    batch_bid_fused_chunk_gla,
    bid_fused_recurrent_gla,
    dirgate,
    dwconv3x3,
    fused_chunk_gla,
    fused_recurrent_gla,
    gla_bidir_backward,
    gla_bidir_forward,
    gla_causal_state_forward,
    gla_bidir_locality_gate,
    locality_blend,
    locality_gate,
    rmsnorm,
    split_heads,
    swiglu,
)

__all__ = [
    "batch_bid_fused_chunk_gla", "bid_fused_recurrent_gla", "dirgate", "dwconv3x3", "fused_chunk_gla",
    "fused_recurrent_gla", "gla_bidir_backward", "gla_bidir_forward", "gla_causal_state_forward", "gla_bidir_locality_gate", "locality_blend", "locality_gate", "rmsnorm", "split_heads", "swiglu",
]
