"""Shared helpers for the parity tests: dfdx-style views and the tolerance rule."""
from __future__ import annotations

import math

import numpy as np


def row_major_strides(shape):
    """Shape::strides (reference: dfdx-core/src/shapes/shape.rs:188-197)."""
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    return strides


def permute(shape, strides, axes):
    """Zero-copy permute (reference: dfdx-core/src/shapes/permutes.rs:29-36)."""
    return [shape[a] for a in axes], [strides[a] for a in axes]


def logical(storage_f64: np.ndarray, shape, strides, offset=0) -> np.ndarray:
    """Materialise the logical tensor a (storage, shape, strides) view denotes."""
    idx = np.full(tuple(shape), offset, dtype=np.int64)
    for ax, (n, s) in enumerate(zip(shape, strides)):
        sh = [1] * len(shape)
        sh[ax] = n
        idx = idx + (np.arange(n, dtype=np.int64) * s).reshape(sh)
    return storage_f64.reshape(-1)[idx]


def rng(seed: int) -> np.random.Generator:
    """Counter-based generator; every tensor in the tests names its seed."""
    return np.random.Generator(np.random.Philox(seed))


# Tolerance stated by the task for parity with dfdx's Cpu matmul:
#   f32:        max|err| <= 1e-5 * sqrt(K) * max|a| * max|b|
#   f16 / bf16: max|err| <= 2e-3 * sqrt(K) * max|a| * max|b|   (f32 accumulate)
# f64 is not named; 1e-12 is used for it.
TOL_COEF = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3, "f64": 1e-12}


def tolerance(dtype: str, k: int, amax: float, bmax: float) -> float:
    return TOL_COEF[dtype] * math.sqrt(max(k, 1)) * amax * bmax


def assert_within(dtype, k, got_f64, want_f64, a_f64, b_f64, extra=0.0, what=""):
    amax = float(np.max(np.abs(a_f64))) if a_f64.size else 0.0
    bmax = float(np.max(np.abs(b_f64))) if b_f64.size else 0.0
    tol = tolerance(dtype, k, amax, bmax) + extra
    err = float(np.max(np.abs(got_f64 - want_f64))) if got_f64.size else 0.0
    assert np.all(np.isfinite(got_f64)), f"{what}: non-finite output"
    assert err <= tol, f"{what}: max|err| {err:.3e} > tol {tol:.3e} (dtype {dtype}, K {k})"
    return err, tol
