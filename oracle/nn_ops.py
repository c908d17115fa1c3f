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


# ------------------------------------------------------------------------------------------ scalar mul --

def scalar_mul_forward(x: np.ndarray, scalar: float, dtype: str) -> np.ndarray:
    """``t * scalar`` (ScalarMulKernelOp::f, tensor_ops/mul/cpu_kernel.rs:5-11, applied to every element of the
    storage by the unary kernel, utilities/cpu_kernels.rs:73-78); the scalar is held in the element type."""
    s = round_to(np.float64(scalar), dtype)
    return round_to(np.asarray(x, np.float64) * s, dtype)


def scalar_mul_backward(scalar: float, grad_inp: np.ndarray, grad_out: np.ndarray, dtype: str) -> np.ndarray:
    """``*x += df * grad_out[i]`` with the constant df = scalar (utilities/cpu_kernels.rs:89-93): the product and
    the add each round to the element type."""
    s = round_to(np.float64(scalar), dtype)
    return round_to(np.asarray(grad_inp, np.float64) + round_to(s * np.asarray(grad_out, np.float64), dtype), dtype)


# --------------------------------------------------------------------------------------------- softmax --

def _seq_sum_last(x: np.ndarray, dtype: str) -> np.ndarray:
    """Sum over the last axis the way the Cpu reduction does it for f32 / plain f16: one accumulator of the
    element type per output, elements added in index order (tensor_ops/sum_to/cpu_kernel.rs:72-103).  (The
    AMP<f16> impl, :8-41, keeps that accumulator in f32 instead.)"""
    acc = np.zeros(x.shape[:-1], np.float64)
    for j in range(x.shape[-1]):
        acc = round_to(acc + x[..., j], dtype)
    return acc


def softmax_forward(x: np.ndarray, dtype: str, faithful: bool = True) -> np.ndarray:
    """``try_softmax`` over the last axis (tensor_ops/softmax.rs:70-83): m = max, tm = t - m, e = exp(tm),
    s = sum(e), out = e / s, every step a kernel that rounds to the element type.  ``faithful=False`` evaluates the
    same formula in float64 and rounds once."""
    x = np.asarray(x, np.float64)
    m = x.max(axis=-1, keepdims=True)
    if not faithful:
        e = np.exp(x - m)
        return round_to(e / e.sum(axis=-1, keepdims=True), dtype)
    tm = round_to(x - m, dtype)
    e = round_to(np.exp(tm), dtype)
    s = _seq_sum_last(e, dtype)[..., None]
    return round_to(e / s, dtype)


def softmax_backward(x: np.ndarray, grad_out: np.ndarray, dtype: str, faithful: bool = True) -> np.ndarray:
    """Gradient of that composition w.r.t. t, as the tape replays it (softmax.rs:70-83 with the binary div, the
    broadcast sum and exp backward ops): with e, s as above,
        g_e  = g / s                       (div backward, lhs; utilities/cpu_kernels.rs:164-187)
        g_s  = sum_j( -e_j / s^2 * g_j )   (div backward, broadcast rhs: accumulated element by element)
        g_e += g_s                         (sum backward: broadcast add)
        g_t  = g_e * e                     (exp backward, df = f(x))
    ``faithful=False`` returns out * (g - sum_j g_j out_j) evaluated in float64, rounded once."""
    x = np.asarray(x, np.float64)
    g = np.asarray(grad_out, np.float64)
    m = x.max(axis=-1, keepdims=True)
    if not faithful:
        e = np.exp(x - m)
        p = e / e.sum(axis=-1, keepdims=True)
        return round_to(p * (g - (g * p).sum(axis=-1, keepdims=True)), dtype)
    tm = round_to(x - m, dtype)
    e = round_to(np.exp(tm), dtype)
    s = _seq_sum_last(e, dtype)[..., None]
    g_e = round_to(round_to(1.0 / s, dtype) * g, dtype)
    contrib = round_to(round_to(-e / round_to(s * s, dtype), dtype) * g, dtype)
    g_s = _seq_sum_last(contrib, dtype)[..., None]
    g_e = round_to(g_e + g_s, dtype)
    return round_to(e * g_e, dtype)


# --------------------------------------------------------------------------------------------- reshape --

def _view_indices(shape, strides) -> np.ndarray:
    idx = np.zeros(tuple(shape), dtype=np.int64)
    for ax, (n, s) in enumerate(zip(shape, strides)):
        sh = [1] * len(shape)
        sh[ax] = n
        idx = idx + (np.arange(n, dtype=np.int64) * s).reshape(sh)
    return idx.reshape(-1)


def reshape_forward(storage: np.ndarray, shape, strides) -> np.ndarray:
    """``ReshapeKernel::forward`` (tensor_ops/reshape_to/cpu_kernel.rs:8-21): the view's elements in logical
    row-major order, copied into a fresh contiguous buffer."""
    return np.asarray(storage).reshape(-1)[_view_indices(shape, strides)].copy()


def reshape_backward(shape, strides, grad_inp: np.ndarray, grad_out: np.ndarray, dtype: str) -> np.ndarray:
    """``ReshapeKernel::backward`` (cpu_kernel.rs:22-34): ``grad_inp[i] += grad_out[o]`` walking both index
    sequences together; a repeated i (broadcast view) accumulates in visiting order."""
    out = np.asarray(grad_inp, np.float64).copy().reshape(-1)
    go = np.asarray(grad_out, np.float64).reshape(-1)
    idx = _view_indices(shape, strides)
    if len(np.unique(idx)) == len(idx):
        out[idx] = round_to(out[idx] + go, dtype)
        return out
    for o, i in enumerate(idx):
        out[i] = np.reshape(round_to(out[i] + go[o], dtype), -1)[0]
    return out


# ------------------------------------------------------------------------------- LayerNorm1D, ReLU, add --

def normalize_forward(x: np.ndarray, epsilon: float, dtype: str, faithful: bool = True) -> np.ndarray:
    """``try_normalize`` over the last axis (tensor_ops/normalize.rs:35-49): mean = sum * (1/n) (mean_to.rs:38-44),
    centered = t - mean, std = sqrt(mean(centered^2) + epsilon), out = centered / std -- every step a kernel that
    rounds to the element type, the sums running in index order.  ``faithful=False`` evaluates the same formula in
    float64 and rounds once."""
    x = np.asarray(x, np.float64)
    n = x.shape[-1]
    if not faithful:
        c = x - x.mean(axis=-1, keepdims=True)
        return round_to(c / np.sqrt((c * c).mean(axis=-1, keepdims=True) + epsilon), dtype)
    inv_n = round_to(np.float64(1.0 / n), dtype)
    mean = round_to(_seq_sum_last(x, dtype) * inv_n, dtype)[..., None]
    centered = round_to(x - mean, dtype)
    var = round_to(_seq_sum_last(round_to(centered * centered, dtype), dtype) * inv_n, dtype)[..., None]
    std = round_to(np.sqrt(round_to(var + round_to(np.float64(epsilon), dtype), dtype)), dtype)
    return round_to(centered / std, dtype)


def layer_norm_forward(x, gamma, beta, epsilon: float, dtype: str, faithful: bool = True) -> np.ndarray:
    """``LayerNorm1D::try_forward`` (dfdx/src/nn/layers/layer_norm1d.rs:87-91): normalize over the last axis, times
    gamma, plus beta (one rounding per op when ``faithful``)."""
    gamma, beta = np.asarray(gamma, np.float64), np.asarray(beta, np.float64)
    if not faithful:
        x = np.asarray(x, np.float64)
        c = x - x.mean(axis=-1, keepdims=True)
        return round_to(c / np.sqrt((c * c).mean(axis=-1, keepdims=True) + epsilon) * gamma + beta, dtype)
    xhat = normalize_forward(x, epsilon, dtype, True)
    return round_to(round_to(gamma * xhat, dtype) + beta, dtype)


def layer_norm_backward(x, gamma, grad_out, epsilon: float, dtype: str, grad_x, grad_gamma, grad_beta):
    """Gradients of that composition, accumulated into the given buffers and rounded once (the closed form of what the
    tape replays through div / sqrt / mean / square / sub / mul / add backward ops; its rounding at every op is not
    restated).  With xhat the normalized rows, rstd = 1 / sqrt(var + epsilon) and gh = grad_out * gamma:
        grad_x += rstd * (gh - mean(gh) - xhat * mean(gh * xhat)),
        grad_gamma += sum_rows grad_out * xhat,   grad_beta += sum_rows grad_out."""
    x, g = np.asarray(x, np.float64), np.asarray(grad_out, np.float64)
    gamma = np.asarray(gamma, np.float64)
    c = x - x.mean(axis=-1, keepdims=True)
    rstd = 1.0 / np.sqrt((c * c).mean(axis=-1, keepdims=True) + epsilon)
    xhat = c * rstd
    gh = g * gamma
    gx = rstd * (gh - gh.mean(axis=-1, keepdims=True) - xhat * (gh * xhat).mean(axis=-1, keepdims=True))
    cols = x.shape[-1]
    return (round_to(np.asarray(grad_x, np.float64) + gx, dtype),
            round_to(np.asarray(grad_gamma, np.float64) + (g * xhat).reshape(-1, cols).sum(axis=0), dtype),
            round_to(np.asarray(grad_beta, np.float64) + g.reshape(-1, cols).sum(axis=0), dtype))


def relu_forward(x: np.ndarray, dtype: str) -> np.ndarray:
    """``ReLUKernelOp::f`` (tensor_ops/relu/cpu_kernel.rs:7-9): max(x, 0) on every element of the storage."""
    return round_to(np.maximum(np.asarray(x, np.float64), 0.0), dtype)


def relu_backward(x: np.ndarray, grad_x: np.ndarray, grad_out: np.ndarray, dtype: str) -> np.ndarray:
    """``*g += df(x) * grad_out`` with df = 1 for x > 0, else 0 (relu/cpu_kernel.rs:11-17, utilities/cpu_kernels.rs:
    95-104)."""
    x = np.asarray(x, np.float64)
    return round_to(np.asarray(grad_x, np.float64) + np.where(x > 0.0, np.asarray(grad_out, np.float64), 0.0), dtype)


def add_forward(lhs: np.ndarray, rhs: np.ndarray, dtype: str) -> np.ndarray:
    """``BinaryAddKernelOp::f`` (tensor_ops/add/cpu_kernel.rs:7-9) on two tensors of one layout."""
    return round_to(np.asarray(lhs, np.float64) + np.asarray(rhs, np.float64), dtype)


def add_backward(grad_lhs: np.ndarray, grad_rhs: np.ndarray, grad_out: np.ndarray, dtype: str):
    """Both operands receive grad_out (const derivatives 1, add/cpu_kernel.rs:11-26)."""
    go = np.asarray(grad_out, np.float64)
    return round_to(np.asarray(grad_lhs, np.float64) + go, dtype), round_to(np.asarray(grad_rhs, np.float64) + go, dtype)
