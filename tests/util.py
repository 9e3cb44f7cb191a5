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


def bf16_grid_stats(got, want, small=2.0 ** -5, large=0.5):
    """Separates a kernel's internal error from the bf16 grid of its output.

    `got` holds bf16 values (as float64), `want` the float64 oracle.  Returns a dict:
      internal_rms, internal_max: got - want over the outputs of magnitude below `small`, where the bf16 grid (step
                 <= 2^-13) is finer than any internal error of interest: what the kernel's arithmetic adds before the
                 output rounding, seen directly;
      frac_off:  among outputs of magnitude >= `large`, the fraction that is not the correctly rounded oracle value: an
                 internal error e moves such an output to the neighbouring grid point with probability ~ |e| / step,
                 so this measures the same error where the grid (step 2^-9 and up) hides it from a max-abs figure;
      max_steps_large: the worst distance from the rounded oracle value there, in grid steps (1 = a neighbour).
    A kernel whose pre-rounding result is exact gives zeros throughout.
    """
    w = torch.from_numpy(np.ascontiguousarray(want))
    rounded = w.to(torch.bfloat16).double().numpy()
    sm = np.abs(want) < small
    big = np.abs(want) >= large
    d = (got - want)[sm]
    mag = np.maximum(np.abs(rounded[big]), np.abs(got[big]))
    step = 2.0 ** (np.floor(np.log2(mag)) - 7)
    return {"internal_rms": float(np.sqrt(np.mean(d * d))) if d.size else 0.0,
            "internal_max": float(np.abs(d).max()) if d.size else 0.0,
            "frac_off": float((got[big] != rounded[big]).mean()) if big.any() else 0.0,
            "max_steps_large": float((np.abs(got[big] - rounded[big]) / step).max()) if big.any() else 0.0}
