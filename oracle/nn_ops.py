"""CPU restatement of the module-level ops around dfdx's matmul -- test infrastructure, never the product path.

Plain numpy / Python loops following the reference's ``Cpu`` kernels line by line where the order of floating-point
operations matters.  Values travel as float64 arrays that hold exactly representable storage-type values; every
function that rounds does so through ``round_to(dtype)``, i.e. with the storage type's round-to-nearest-even, at
the points where the reference's code produces a value of the element type ``E``.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this module.
"""
from __future__ import annotations

import numpy as np

from . import f32_to_bf16, bf16_to_f32


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    """Round float64 values to the storage type and widen back (RNE, as `half`/f32 arithmetic does)."""
    x = np.asarray(x, dtype=np.float64)
    if dtype == "f64":
        return x
    if dtype == "f32":
        return x.astype(np.float32).astype(np.float64)
    if dtype == "f16":
        return x.astype(np.float16).astype(np.float64)
    if dtype == "bf16":
        # float64 -> float32 -> bf16 double rounding differs from a direct rounding only on exact ties of the
        # float32 step, which the tolerances used with this helper absorb.
        return bf16_to_f32(f32_to_bf16(x.astype(np.float32))).astype(np.float64)
    raise ValueError(dtype)


# ---------------------------------------------------------------------------------------------- Bias1D --

def bias_forward(x: np.ndarray, bias: np.ndarray, dtype: str) -> np.ndarray:
    """``Bias1D::try_forward`` (dfdx/src/nn/layers/bias1d.rs:62-78): bias broadcast over the leading axes, one add
    in the element type per output (binary add kernel, tensor_ops/utilities/cpu_kernels.rs:120-160)."""
    return round_to(np.asarray(x, np.float64) + np.asarray(bias, np.float64), dtype)


def bias_backward(grad_out: np.ndarray, grad_bias: np.ndarray, dtype: str, faithful: bool = True) -> np.ndarray:
    """The broadcast operand's gradient of that add (tensor_ops/utilities/cpu_kernels.rs:164-203): the loop visits
    grad_out in row-major order and does ``grad_rhs[rhs_i] += dy * go`` with dy = 1 in the element type, i.e. each
    column is summed row after row with a rounding to ``dtype`` after every add (``faithful=True``).
    ``faithful=False`` sums each column exactly (float64) and rounds once: the value a wide accumulator targets."""
    go = np.asarray(grad_out, np.float64).reshape(-1, grad_bias.shape[-1])
    acc = np.asarray(grad_bias, np.float64).copy()
    if not faithful:
        return round_to(acc + go.sum(axis=0), dtype)
    for r in range(go.shape[0]):
        acc = round_to(acc + go[r], dtype)
    return acc
