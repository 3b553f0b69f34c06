"""Shared helpers of the GPU parity tests: input builders and the parity metrics."""
from __future__ import annotations


import numpy as np

from oracle import oracle as orc
from refgen import normal_f32

TOL = 1e-3  # north star: GEMV outputs within max relative error 1e-3 of the CPU path


FLOOR = 1e-2  # outputs below 1 % of their row's rms are compared absolutely (1e-5 rms), see rel_err


def rel_err(y: np.ndarray, ref: np.ndarray) -> float:
    """max_i |y_i - ref_i| / max(|ref_i|, FLOOR * rms(ref)) per output row, worst row.

    A dot product of K ~ 5000 terms summed in f32 carries an absolute error of about 1e-6 of the
    row's rms whatever the order (the CPU path against f64 shows the same); an output that happens
    to cancel to almost nothing therefore has no meaningful RELATIVE error, and is held to
    TOL * FLOOR * rms instead.  Every GEMV test additionally holds the reference's own acceptance
    bound gamma(K/16 + 10) * sum|w x| against an f64 evaluation (gamma_ratio), which has no floor."""
    y = np.asarray(y, np.float64).reshape(ref.shape)
    r = np.asarray(ref, np.float64)
    if r.ndim == 1:
        r, y = r[None], y[None]
    rms = np.sqrt((r * r).mean(axis=1, keepdims=True))
    den = np.maximum(np.abs(r), FLOOR * np.maximum(rms, 1e-30))
    return float(np.max(np.abs(y - r) / den))


def gamma_ratio(y, w, rows, cols, gs, x) -> float:
    """max |y - y_f64| / (gamma(K/16 + 10) * sum|w x|): <= 1 means inside the reference's own fp32 bound."""
    yr, ab = orc.gemv_f64(w, rows, cols, gs, x)
    y = np.asarray(y, np.float64).reshape(yr.shape)
    return float(np.max(np.abs(y - yr) / np.maximum(orc.gamma(cols) * ab, np.finfo(np.float64).tiny)))


def quantized_normal(seed: int, stream: int, rows: int, cols: int, sigma: float = 0.02):
    """The benchmark's weights: N(0, sigma^2) through the ceil encoder -> (container bytes, global scale)."""
    v = normal_f32(seed, stream, rows * cols, sigma)
    return orc.quantize_ceil(v)


