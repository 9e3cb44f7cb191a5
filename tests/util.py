"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import gla_oracle as O


def f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().double().numpy()


def oracle_bidir(q, k, v, gf, gb, scale=None, out_scale=1.0):
    if gb is None:
        return out_scale * O.gla_recurrent(f64(q), f64(k), f64(v), f64(gf), scale=scale)
    return O.bidir_gla_recurrent(f64(q), f64(k), f64(v), f64(gf), f64(gb), scale=scale, out_scale=out_scale)


def max_rel(got, want) -> float:
    return float(np.abs(got - want).max() / np.abs(want).max())


def max_abs(got, want) -> float:
    return float(np.abs(got - want).max())


def announce(msg: str):
    print(f"[case] {msg}", flush=True)
