"""CPU oracle for dfdx's matmul path -- test infrastructure, never the product path.

Thin ctypes/numpy front-end over ``libdfdx_matmul_oracle.so`` (built from
``dfdx_matmul_oracle.c`` by ``oracle/Makefile``).  Only the tests, the smoke
check and the benchmark's CPU-baseline leg import this package.

Arrays are numpy arrays of dtype float32 / float16 / float64; bf16 is carried
as ``uint16`` bit patterns together with ``dtype="bf16"``.  A *view* is a
``(storage, shape, strides)`` triple with strides in elements, which is what a
dfdx ``Tensor`` exposes to its kernels (reference:
dfdx-core/src/tensor/tensor_impls.rs:32-39).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdfdx_matmul_oracle.so")

DT_F32, DT_F16, DT_BF16, DT_F64 = 0, 1, 2, 3
DTYPE_CODES = {"f32": DT_F32, "f16": DT_F16, "bf16": DT_BF16, "f64": DT_F64}
NP_DTYPES = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16, "f64": np.float64}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds)."""
    src = os.path.join(_HERE, "dfdx_matmul_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdfdx_matmul_oracle.so"])
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_gemm.restype = ctypes.c_int
    return _lib


def _ptr(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(x):
    return ctypes.c_int64(int(x))


def _strides(s):
    return (ctypes.c_int64 * len(s))(*[int(v) for v in s])


def check_dtype(dtype: str, *arrays: np.ndarray):
    want = NP_DTYPES[dtype]
    for a in arrays:
        if a.dtype != want:
            raise TypeError(f"dtype {dtype} needs numpy {want}, got {a.dtype}")
        if not a.flags["C_CONTIGUOUS"]:
            raise ValueError("storage arrays must be C-contiguous")


# ------------------------------------------------------------- conversions --
def f32_to_f16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_f16(_ptr(x), _ptr(out), _i64(x.size))
    return out.view(np.float16)


def f16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x).view(np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().oracle_f16_to_f32(_ptr(x), _ptr(out), _i64(x.size))
    return out


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns (uint16), round-to-nearest-even."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16(_ptr(x), _ptr(out), _i64(x.size))
    return out


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().oracle_bf16_to_f32(_ptr(x), _ptr(out), _i64(x.size))
    return out


def to_storage(x: np.ndarray, dtype: str) -> np.ndarray:
    """Round float values into the storage dtype (bf16 -> uint16 bit patterns)."""
    if dtype == "bf16":
        return f32_to_bf16(np.asarray(x, dtype=np.float32))
    return np.ascontiguousarray(x, dtype=NP_DTYPES[dtype])


def to_f64(x: np.ndarray, dtype: str) -> np.ndarray:
    """Storage array -> float64 values."""
    if dtype == "bf16":
        return bf16_to_f32(x).astype(np.float64)
    return x.astype(np.float64)


# -------------------------------------------------------------------- gemm --
def gemm(dtype, m, k, n, accum, a, a_strides, b, b_strides, c, c_strides, acc64=False,
         a_off=0, b_off=0, c_off=0):
    """MatMulImpl::matmul (cpu_kernel.rs:38-50): strided C = (accum ? C : 0) + A.B, in place on ``c``."""
    check_dtype(dtype, a, b, c)
    isz = a.itemsize
    rc = lib().oracle_gemm(
        DTYPE_CODES[dtype], _i64(m), _i64(k), _i64(n), int(bool(accum)), int(bool(acc64)),
        ctypes.c_void_p(a.ctypes.data + a_off * isz), _i64(a_strides[0]), _i64(a_strides[1]),
        ctypes.c_void_p(b.ctypes.data + b_off * isz), _i64(b_strides[0]), _i64(b_strides[1]),
        ctypes.c_void_p(c.ctypes.data + c_off * isz), _i64(c_strides[0]), _i64(c_strides[1]))
    if rc:
        raise MemoryError("oracle_gemm failed")
    return c


def _fwd(name, dtype, dims, lhs, ls, rhs, rs, acc64):
    check_dtype(dtype, lhs, rhs)
    n_out = int(np.prod(dims[:-3], dtype=np.int64)) * dims[-3] * dims[-1]
    out = np.zeros(n_out, dtype=NP_DTYPES[dtype])
    rc = getattr(lib(), name)(DTYPE_CODES[dtype], int(bool(acc64)), *[_i64(d) for d in dims],
                              _ptr(lhs), _strides(ls), _ptr(rhs), _strides(rs), _ptr(out))
    if rc:
        raise MemoryError(name)
    return out


def _bwd(name, dtype, dims, lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64):
    check_dtype(dtype, lhs, rhs, grad_lhs, grad_rhs, grad_out)
    rc = getattr(lib(), name)(DTYPE_CODES[dtype], int(bool(acc64)), *[_i64(d) for d in dims],
                              _ptr(lhs), _strides(ls), _ptr(grad_lhs), _ptr(rhs), _strides(rs),
                              _ptr(grad_rhs), _ptr(grad_out))
    if rc:
        raise MemoryError(name)


def matmat_forward(dtype, m, k, n, lhs, ls, rhs, rs, acc64=False):
    """MatMatKernel::forward (cpu_kernel.rs:235-254) -> flat (m*n) row-major out."""
    return _fwd("oracle_matmat_forward", dtype, (m, k, n), lhs, ls, rhs, rs, acc64)


def matmat_backward(dtype, m, k, n, lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64=False):
    """MatMatKernel::backward (cpu_kernel.rs:255-287); grads accumulated in place."""
    _bwd("oracle_matmat_backward", dtype, (m, k, n), lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64)


def matmat_br_forward(dtype, b, m, k, n, lhs, ls, rhs, rs, acc64=False):
    """MatMatBrKernel::forward (cpu_kernel.rs:294-316)."""
    return _fwd("oracle_matmat_br_forward", dtype, (b, m, k, n), lhs, ls, rhs, rs, acc64)


def matmat_br_backward(dtype, b, m, k, n, lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64=False):
    """MatMatBrKernel::backward (cpu_kernel.rs:317-351)."""
    _bwd("oracle_matmat_br_backward", dtype, (b, m, k, n), lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64)


def matmat_batch3_forward(dtype, b, m, k, n, lhs, ls, rhs, rs, acc64=False):
    """MatMatBatch3Kernel::forward (cpu_kernel.rs:358-382)."""
    return _fwd("oracle_matmat_batch3_forward", dtype, (b, m, k, n), lhs, ls, rhs, rs, acc64)


def matmat_batch3_backward(dtype, b, m, k, n, lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64=False):
    """MatMatBatch3Kernel::backward (cpu_kernel.rs:383-417)."""
    _bwd("oracle_matmat_batch3_backward", dtype, (b, m, k, n), lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64)


def matmat_batch4_forward(dtype, b, s, m, k, n, lhs, ls, rhs, rs, acc64=False):
    """MatMatBatch4Kernel::forward (cpu_kernel.rs:424-448)."""
    return _fwd("oracle_matmat_batch4_forward", dtype, (b, s, m, k, n), lhs, ls, rhs, rs, acc64)


def matmat_batch4_backward(dtype, b, s, m, k, n, lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64=False):
    """MatMatBatch4Kernel::backward (cpu_kernel.rs:449-485)."""
    _bwd("oracle_matmat_batch4_backward", dtype, (b, s, m, k, n), lhs, ls, grad_lhs, rhs, rs, grad_rhs, grad_out, acc64)
