"""CPU restatement of dfdx's conv2d (unfold + GEMM) -- test infrastructure, never the product path.

Follows dfdx-core/src/tensor_ops/conv2d/cpu_kernel.rs step by step: the patch buffers are filled exactly as
``fwd_conv2d`` / ``bwd_conv2d`` fill them (same index arithmetic, zeros where the window leaves the image) and every
product goes through the C oracle's strided GEMM with the dims, strides and accumulate flags of the reference's
``Self::matmul`` calls, so rounding happens where the reference rounds.  Buffers are flat numpy arrays of the
storage type (bf16 as uint16 bit patterns), as in ``oracle/__init__.py``.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from . import NP_DTYPES, gemm, to_f64, to_storage


@dataclass(frozen=True)
class Conv2DOp:
    """``Conv2DOp`` (conv2d/mod.rs:14-29), fields in the reference's order."""
    kernel: int
    stride: int
    padding: int
    dilation: int
    groups: int
    batch: int
    chan_in: int
    chan_out: int
    h_in: int
    h_out: int
    w_in: int
    w_out: int

    @staticmethod
    def make(batch, chan_in, chan_out, h_in, w_in, kernel, stride=1, padding=0, dilation=1, groups=1) -> "Conv2DOp":
        """Output size rule of ``TryConv2D for (usize, Kernel)`` (conv2d/mod.rs:143-160)."""
        size = lambda d: (d + 2 * padding - 1 - dilation * (kernel - 1)) // stride + 1
        assert d_ok(h_in, padding, dilation, kernel) and d_ok(w_in, padding, dilation, kernel), "kernel larger than padded image"
        return Conv2DOp(kernel, stride, padding, dilation, groups, batch, chan_in, chan_out, h_in, size(h_in), w_in, size(w_in))


def d_ok(d, padding, dilation, kernel):
    return d + 2 * padding - 1 >= dilation * (kernel - 1)


def _unfold_input_index(op: Conv2DOp):
    """For every slot of the forward patch buffer (C, K, K, OH, OW) the image element it takes, or -1
    (fwd_conv2d, cpu_kernel.rs:53-72: y = oh*stride + dilation*k1 - padding, likewise x)."""
    c, k1, k2, oh, ow = np.meshgrid(np.arange(op.chan_in), np.arange(op.kernel), np.arange(op.kernel),
                                    np.arange(op.h_out), np.arange(op.w_out), indexing="ij")
    y = oh * op.stride + op.dilation * k1 - op.padding
    x = ow * op.stride + op.dilation * k2 - op.padding
    ok = (y >= 0) & (y < op.h_in) & (x >= 0) & (x < op.w_in)
    idx = c * (op.h_in * op.w_in) + y * op.w_in + x
    return np.where(ok, idx, -1).reshape(-1)


def _unfold_output_index(op: Conv2DOp):
    """For every slot of the backward patch buffer (O, K, K, H, W) the grad_out element it takes, or -1
    (``unfold_idx``, cpu_kernel.rs:10-38, used by bwd_conv2d :112-128)."""
    o, k1, k2, y, x = np.meshgrid(np.arange(op.chan_out), np.arange(op.kernel), np.arange(op.kernel),
                                  np.arange(op.h_in), np.arange(op.w_in), indexing="ij")
    oh = y + op.padding - op.dilation * k1
    ow = x + op.padding - op.dilation * k2
    ok = (oh >= 0) & (oh % op.stride == 0) & (ow >= 0) & (ow % op.stride == 0)
    oh, ow = oh // op.stride, ow // op.stride
    ok &= (oh < op.h_out) & (ow < op.w_out)
    idx = o * (op.h_out * op.w_out) + oh * op.w_out + ow
    return np.where(ok, idx, -1).reshape(-1)


def _gather(src: np.ndarray, idx: np.ndarray) -> np.ndarray:
    out = np.zeros(idx.shape, dtype=src.dtype)
    ok = idx >= 0
    out[ok] = src[idx[ok]]
    return out


def conv2d_forward(dtype: str, op: Conv2DOp, img: np.ndarray, filters: np.ndarray, acc64: bool = False) -> np.ndarray:
    """``Conv2DKernel::forward`` for Cpu (cpu_kernel.rs:175-202) on contiguous (B, C, H, W) / (O, C/G, K, K)
    buffers; returns the (B, O, OH, OW) buffer."""
    m = op.chan_out // op.groups
    k = (op.chan_in // op.groups) * op.kernel * op.kernel
    n = op.h_out * op.w_out
    out = np.zeros(op.batch * op.chan_out * n, dtype=NP_DTYPES[dtype])
    idx = _unfold_input_index(op)
    lstride, ostride = op.chan_in * op.h_in * op.w_in, op.chan_out * n
    for b in range(op.batch):
        buf = _gather(img[b * lstride:(b + 1) * lstride], idx)
        for g in range(op.groups):  # cpu_kernel.rs:80-91
            gemm(dtype, m, k, n, False, filters[g * m * k:], (k, 1), buf[g * k * n:], (n, 1),
                 out[b * ostride + g * m * n:], (n, 1), acc64=acc64)
    return out


def conv2d_backward(dtype: str, op: Conv2DOp, img: np.ndarray, grad_img: np.ndarray, filters: np.ndarray,
                    grad_filters: np.ndarray, grad_out: np.ndarray, acc64: bool = False) -> None:
    """``Conv2DKernel::backward`` for Cpu (cpu_kernel.rs:204-278): grads accumulated in place."""
    G, cg, og, K = op.groups, op.chan_in // op.groups, op.chan_out // op.groups, op.kernel
    # filters (O, C/G, K, K) -> f1023 (G, C/G, O/G, K, K)   (cpu_kernel.rs:225-236)
    f5 = filters.reshape(G, og, cg, K, K)
    f1023 = np.ascontiguousarray(f5.transpose(0, 2, 1, 3, 4)).reshape(-1)
    grad_f1023 = np.zeros_like(f1023)
    idx = _unfold_output_index(op)
    hw, ohw = op.h_in * op.w_in, op.h_out * op.w_out
    lstride, ostride = op.chan_in * hw, op.chan_out * ohw
    for b in range(op.batch):
        buf = _gather(grad_out[b * ostride:(b + 1) * ostride], idx)
        m, k, n = cg, og * K * K, hw  # img_g += filters^T * unfold(grad_out)   (cpu_kernel.rs:131-149)
        for g in range(G):
            gemm(dtype, m, k, n, True, f1023[g * m * k:], (k, 1), buf[g * k * n:], (n, 1),
                 grad_img[b * lstride + g * m * n:], (n, 1), acc64=acc64)
        m, k, n = cg, hw, og * K * K  # weight_g^T += img * unfold(patches)^T   (cpu_kernel.rs:151-169)
        for g in range(G):
            gemm(dtype, m, k, n, True, img[b * lstride + g * m * k:], (k, 1), buf[g * k * n:], (1, k),
                 grad_f1023[g * m * n:], (n, 1), acc64=acc64)
    # untranspose: grad_rhs[idx] += grad_f1023[i]   (cpu_kernel.rs:264-275); one add in the element type
    back = grad_f1023.reshape(G, cg, og, K, K).transpose(0, 2, 1, 3, 4).reshape(-1)
    total = to_f64(grad_filters, dtype) + to_f64(np.ascontiguousarray(back), dtype)
    grad_filters[:] = to_storage(total, dtype)
