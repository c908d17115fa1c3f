"""``Rocm``: the host-side mirror of a dfdx device for the matmul path.

Method names and argument meaning follow the reference's kernel traits
(dfdx-core/src/tensor_ops/matmul/mod.rs:116-131,197-212,234-249,273-288):
``forward(lhs, rhs) -> out`` allocates a fresh contiguous output, and
``backward(lhs, grad_lhs, rhs, grad_rhs, grad_out)`` accumulates into gradient
buffers that are laid out like the operands' physical storage.  A tensor is a
:class:`View`: device storage + shape + strides in elements, which is what a
dfdx ``Tensor`` hands its kernels (tensor_impls.rs:32-39).  Shape mismatches
raise ``AssertionError`` before any kernel runs, like the reference's
``assert_eq!`` (mod.rs:192,229,267-268,306-308).

PyTorch is used for device memory only (allocation, host<->device copies).
"""
from __future__ import annotations

import ctypes
import os
import weakref
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

DTYPES = {"f32": 0, "f16": 1, "bf16": 2, "f64": 3}
ITEMSIZE = {"f32": 4, "f16": 2, "bf16": 2, "f64": 8}
NP_DTYPES = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16, "f64": np.float64}

KERNEL_AUTO, KERNEL_GENERIC, KERNEL_MFMA, KERNEL_GEMV = 0, 1, 2, 3
ZERO_DEFERRED = 2   # dfdx_rocm_alloc: zero as far as the library can tell, fill only if needed
NOALLOC_SCRATCH_BYTES = 32 << 20   # DFDX_ROCM_NOALLOC_SCRATCH_BYTES
ERR_SCRATCH_TOO_SMALL = -5


class RocmError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"dfdx_rocm error {code}: {msg}")
        self.code = code


class GemmDesc(ctypes.Structure):
    """``dfdx_rocm_gemm_desc`` (include/dfdx_rocm.h)."""
    _fields_ = [
        ("dtype", ctypes.c_int32), ("accumulate", ctypes.c_int32),
        ("m", ctypes.c_int64), ("n", ctypes.c_int64), ("k", ctypes.c_int64),
        ("batch1", ctypes.c_int64), ("batch2", ctypes.c_int64),
        ("a", ctypes.c_void_p), ("a_rs", ctypes.c_int64), ("a_cs", ctypes.c_int64),
        ("a_b1", ctypes.c_int64), ("a_b2", ctypes.c_int64),
        ("b", ctypes.c_void_p), ("b_rs", ctypes.c_int64), ("b_cs", ctypes.c_int64),
        ("b_b1", ctypes.c_int64), ("b_b2", ctypes.c_int64),
        ("c", ctypes.c_void_p), ("c_rs", ctypes.c_int64), ("c_cs", ctypes.c_int64),
        ("c_b1", ctypes.c_int64), ("c_b2", ctypes.c_int64),
        ("bias", ctypes.c_void_p),
        ("reduce_batch", ctypes.c_int32), ("kernel", ctypes.c_int32),
        ("variant", ctypes.c_int32), ("flags", ctypes.c_int32),
    ]


class Conv2DOp(ctypes.Structure):
    """Mirrors ``dfdx_rocm_conv2d_op`` == the reference's ``Conv2DOp`` (conv2d/mod.rs:14-29)."""
    _fields_ = [(n, ctypes.c_size_t) for n in ("kernel", "stride", "padding", "dilation", "groups", "batch",
                                               "chan_in", "chan_out", "h_in", "h_out", "w_in", "w_out")]


def lib_path() -> str:
    return os.path.join(_HERE, "lib", "libdfdx_rocm.so")


_lib = None

# every symbol include/dfdx_rocm.h declares
EXPORTS = [
    "dfdx_rocm_create", "dfdx_rocm_destroy", "dfdx_rocm_strerror", "dfdx_rocm_device_info",
    "dfdx_rocm_alloc", "dfdx_rocm_free", "dfdx_rocm_memset_zero", "dfdx_rocm_copy_h2d", "dfdx_rocm_copy_d2h",
    "dfdx_rocm_copy_d2d", "dfdx_rocm_synchronize", "dfdx_rocm_zero_deferred", "dfdx_rocm_settle_zeros", "dfdx_rocm_forget_zeros",
    "dfdx_rocm_enable_cache", "dfdx_rocm_disable_cache",
    "dfdx_rocm_empty_cache", "dfdx_rocm_cache_stats", "dfdx_rocm_gemm", "dfdx_rocm_gemm_noalloc", "dfdx_rocm_gemm_plan",
    "dfdx_rocm_mfma_variant_count", "dfdx_rocm_gemm_time", "dfdx_rocm_gemm_time_rotating",
    "dfdx_rocm_matmat_forward", "dfdx_rocm_matmat_backward",
    "dfdx_rocm_matmat_br_forward", "dfdx_rocm_matmat_br_backward",
    "dfdx_rocm_matmat_batch3_forward", "dfdx_rocm_matmat_batch3_backward",
    "dfdx_rocm_matmat_batch4_forward", "dfdx_rocm_matmat_batch4_backward",
    "dfdx_rocm_linear_forward", "dfdx_rocm_linear_backward",
    "dfdx_rocm_bias_forward", "dfdx_rocm_bias_backward",
    "dfdx_rocm_scalar_mul_forward", "dfdx_rocm_scalar_mul_backward",
    "dfdx_rocm_softmax_forward", "dfdx_rocm_softmax_backward",
    "dfdx_rocm_reshape_forward", "dfdx_rocm_reshape_backward",
    "dfdx_rocm_layer_norm_forward", "dfdx_rocm_layer_norm_backward",
    "dfdx_rocm_relu_forward", "dfdx_rocm_relu_backward",
    "dfdx_rocm_add_forward", "dfdx_rocm_add_backward",
    "dfdx_rocm_conv2d_forward", "dfdx_rocm_conv2d_backward",
]


def load_library() -> ctypes.CDLL:
    """Load the built HIP library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is missing: build it with `make -C dfdx_amd/csrc` (or __graft_entry__.build())")
        lib = ctypes.CDLL(path)
        lib.dfdx_rocm_strerror.restype = ctypes.c_char_p
        lib.dfdx_rocm_strerror.argtypes = [ctypes.c_int]
        for name in EXPORTS:
            fn = getattr(lib, name)
            if name != "dfdx_rocm_strerror":
                fn.restype = ctypes.c_int
        _lib = lib
    return _lib


@dataclass
class View:
    """Device storage seen through a shape and element strides (a dfdx tensor's kernel-side face)."""
    storage: "object"           # torch.uint8 CUDA tensor owning the bytes
    dtype: str
    shape: tuple
    strides: tuple
    offset: int = 0             # in elements
    owner: "object" = None      # keeps an arena's declarations alive exactly as long as views of it exist (zeros_many)

    @property
    def ptr(self) -> int:
        return self.storage.data_ptr() + self.offset * ITEMSIZE[self.dtype]

    def permute(self, *axes) -> "View":
        """Zero-copy permute (reference: tensor_ops/permute_to.rs:38-52)."""
        return View(self.storage, self.dtype, tuple(self.shape[a] for a in axes),
                    tuple(self.strides[a] for a in axes), self.offset, self.owner)

    def numel_storage(self) -> int:
        return self.storage.numel() // ITEMSIZE[self.dtype]


class _Arena:
    """One allocation that several Views are carved from.  When the last View of it goes, whatever zero declarations
    its pieces still carry are withdrawn (``dfdx_rocm_forget_zeros``) BEFORE torch gets the memory back, so that a later
    settle cannot write zeros into memory that has a new owner by then."""

    def __init__(self, dev: "Rocm", raw):
        self.raw = raw
        self._fin = weakref.finalize(self, _forget_range, weakref.ref(dev), raw, raw.data_ptr(), raw.numel())
        self._fin.atexit = False   # at interpreter exit the context goes first and takes its declarations with it

    def forget(self):
        self._fin()


def _forget_range(dev_ref, raw, ptr, nbytes):
    # `raw` is held by this callback's arguments: the memory is still allocated while the declarations are dropped
    dev = dev_ref()
    if dev is not None and getattr(dev, "ctx", None):
        dev.lib.dfdx_rocm_forget_zeros(dev.ctx, ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes))
    del raw


def _row_major(shape):
    s = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        s[i] = s[i + 1] * shape[i + 1]
    return tuple(s)


def _i64arr(v: Sequence[int]):
    return (ctypes.c_int64 * len(v))(*[int(x) for x in v])


class Rocm:
    """One GPU context.  ``Rocm(ordinal)`` ~ ``Cuda::try_build(ordinal, seed)`` (tensor/cuda/device.rs:72-90)."""

    def __init__(self, ordinal: int = 0):
        import torch

        self._torch = torch
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the Rocm device needs an MI355X (there is no CPU fallback)")
        self.lib = load_library()
        self.ordinal = ordinal
        self.device = torch.device("cuda", ordinal)
        torch.cuda.set_device(ordinal)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        ctx = ctypes.c_void_p()
        self._check(self.lib.dfdx_rocm_create(ordinal, ctypes.c_void_p(stream), ctypes.byref(ctx)))
        self.ctx = ctx

    def close(self):
        if getattr(self, "ctx", None):
            self.lib.dfdx_rocm_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ------------------------------------------------------------------ misc --
    def _check(self, code: int):
        if code != 0:
            raise RocmError(code, self.lib.dfdx_rocm_strerror(code).decode())

    def synchronize(self):
        self._check(self.lib.dfdx_rocm_synchronize(self.ctx))

    def device_info(self):
        name = ctypes.create_string_buffer(128)
        cus, mhz = ctypes.c_int(), ctypes.c_int()
        self._check(self.lib.dfdx_rocm_device_info(self.ctx, name, 128, ctypes.byref(cus), ctypes.byref(mhz)))
        return {"name": name.value.decode(), "compute_units": cus.value, "clock_mhz": mhz.value}

    # ----------------------------------------------------------------- cache --
    def enable_cache(self):
        """``Cache::enable_cache`` (tensor/storage_traits.rs:41-77): freed buffers are kept for the next allocation of their size."""
        self._check(self.lib.dfdx_rocm_enable_cache(self.ctx))

    def disable_cache(self):
        self._check(self.lib.dfdx_rocm_disable_cache(self.ctx))

    def empty_cache(self):
        self._check(self.lib.dfdx_rocm_empty_cache(self.ctx))

    def cache_stats(self):
        n, b = ctypes.c_size_t(), ctypes.c_size_t()
        self._check(self.lib.dfdx_rocm_cache_stats(self.ctx, ctypes.byref(n), ctypes.byref(b)))
        return n.value, b.value

    def alloc(self, nbytes: int, zeroed=True) -> int:
        """``Storage::try_alloc_len`` / ``alloc_empty`` through the library's own allocator; returns the device address.
        ``zeroed`` = ``ZERO_DEFERRED``: zero as far as the library's calls can tell, the fill only runs if a call needs it."""
        p = ctypes.c_void_p()
        self._check(self.lib.dfdx_rocm_alloc(self.ctx, ctypes.c_size_t(nbytes), int(zeroed), ctypes.byref(p)))
        return p.value

    def free(self, ptr: int):
        self._check(self.lib.dfdx_rocm_free(self.ctx, ctypes.c_void_p(ptr)))

    def zero_deferred(self, ptr: int, nbytes: int):
        """Declares ``nbytes`` at ``ptr`` zero without filling them (``dfdx_rocm_zero_deferred``): the first call that
        accumulates into the whole buffer stores 0 + value, any other first use runs the fill."""
        self._check(self.lib.dfdx_rocm_zero_deferred(self.ctx, ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes)))

    def forget_zeros(self, ptr: int, nbytes: int):
        """Withdraws the zero declarations inside ``[ptr, ptr + nbytes)`` without filling (``dfdx_rocm_forget_zeros``):
        what the owner of declared storage calls before it releases that storage unsettled."""
        self._check(self.lib.dfdx_rocm_forget_zeros(self.ctx, ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes)))

    def settle_zeros(self):
        """Runs every deferred fill still pending: needed before code outside the library reads such a buffer."""
        self._check(self.lib.dfdx_rocm_settle_zeros(self.ctx))

    # --------------------------------------------------------------- storage --
    def tensor(self, host: np.ndarray, dtype: str, shape=None, strides=None) -> View:
        """Upload ``host`` (storage order) and view it; bf16 storage is given as uint16 bit patterns."""
        torch = self._torch
        host = np.ascontiguousarray(host)
        if host.dtype != NP_DTYPES[dtype]:
            raise TypeError(f"{dtype} storage must be numpy {NP_DTYPES[dtype]}, got {host.dtype}")
        shape = tuple(host.shape) if shape is None else tuple(shape)
        strides = _row_major(shape) if strides is None else tuple(strides)
        raw = torch.from_numpy(host.reshape(-1).view(np.uint8).copy()).to(self.device)
        if raw.numel() == 0:
            raw = torch.zeros(16, dtype=torch.uint8, device=self.device)
        return View(raw, dtype, shape, strides)

    def zeros(self, dtype: str, shape, numel_storage: Optional[int] = None, strides=None) -> View:
        """Zero-filled storage (``Storage::try_alloc_len``, tensor/cuda/device.rs:259-266)."""
        torch = self._torch
        shape = tuple(shape)
        n = int(np.prod(shape, dtype=np.int64)) if numel_storage is None else numel_storage
        raw = self._zeroed_bytes(max(n * ITEMSIZE[dtype], 16))
        return View(raw, dtype, shape, _row_major(shape) if strides is None else tuple(strides))

    def zeros_many(self, likes, deferred: bool = False) -> list:
        """Zero-filled storages for several tensors at once: one allocation, ONE fill launch, each view on its own
        256 B-aligned piece.  ``likes`` are Views whose dtype / shape give the sizes (contiguous row-major results).
        What a pooling allocator behind ``try_alloc_grad`` would do for the gradient buffers of one backward pass:
        small fills are launch-bound (3.5 us for 2 MiB), one large fill runs at the HBM write rate.
        ``deferred``: no fill at all; every piece is declared zero (``zero_deferred``) and the first backward op that
        accumulates into the whole of it stores instead -- read the results through this object (``to_host``) or
        call ``settle_zeros`` first.  The declarations are withdrawn when the last of the returned Views (and of the
        Views derived from them) is dropped, so the arena never goes back to the allocator with a fill still promised."""
        sizes = [max(int(np.prod(v.shape, dtype=np.int64)) * ITEMSIZE[v.dtype], 16) for v in likes]
        offs, total = [], 0
        for n in sizes:
            offs.append(total)
            total += (n + 255) // 256 * 256
        owner = None
        if deferred:
            arena = self._torch.empty(max(total, 16), dtype=self._torch.uint8, device=self.device)
            owner = _Arena(self, arena)
            try:
                for o, n in zip(offs, sizes):
                    self.zero_deferred(arena.data_ptr() + o, n)
            except Exception:
                owner.forget()
                raise
        else:
            arena = self._zeroed_bytes(max(total, 16))
        return [View(arena[o:o + n], v.dtype, tuple(v.shape), _row_major(tuple(v.shape)), 0, owner)
                for v, o, n in zip(likes, offs, sizes)]

    def _zeroed_bytes(self, nbytes: int):
        """Device memory from torch's allocator, cleared by the library's own fill kernel (``dfdx_rocm_memset_zero``)."""
        raw = self._torch.empty(nbytes, dtype=self._torch.uint8, device=self.device)
        self._check(self.lib.dfdx_rocm_memset_zero(self.ctx, ctypes.c_void_p(raw.data_ptr()), ctypes.c_size_t(nbytes)))
        return raw

    def empty(self, dtype: str, shape) -> View:
        """Uninitialised storage for an output that a forward kernel overwrites (``alloc_empty``,
        tensor_ops/matmul/cuda_kernel.rs:253)."""
        shape = tuple(shape)
        n = int(np.prod(shape, dtype=np.int64))
        raw = self._torch.empty(max(n * ITEMSIZE[dtype], 16), dtype=self._torch.uint8, device=self.device)
        return View(raw, dtype, shape, _row_major(shape))

    def zeros_like_storage(self, v: View) -> View:
        """A gradient buffer for ``v``: zero-filled, same physical length, same strides (gradients.rs:53-58)."""
        raw = self._zeroed_bytes(v.storage.numel())
        return View(raw, v.dtype, v.shape, v.strides, v.offset)

    def to_host(self, v: View) -> np.ndarray:
        """The storage bytes as a flat numpy array of the storage dtype."""
        n = v.numel_storage()
        self.settle_zeros()   # the storage may still wait for a deferred zero fill
        return v.storage.cpu().numpy().view(NP_DTYPES[v.dtype])[:n].copy()

    # ------------------------------------------------------------------ gemm --
    def gemm_desc(self, dtype, m, k, n, a, a_strides, b, b_strides, c, c_strides, accumulate=False,
                  batch=(1, 1), a_batch=(0, 0), b_batch=(0, 0), c_batch=(0, 0), bias=None, reduce_batch=False,
                  kernel=KERNEL_AUTO, variant=0, no_split_k=False, split_k=0) -> GemmDesc:
        d = GemmDesc()
        d.dtype, d.accumulate = DTYPES[dtype], int(bool(accumulate))
        d.m, d.n, d.k = m, n, k
        d.batch1, d.batch2 = batch
        d.a, d.a_rs, d.a_cs, d.a_b1, d.a_b2 = a, a_strides[0], a_strides[1], a_batch[0], a_batch[1]
        d.b, d.b_rs, d.b_cs, d.b_b1, d.b_b2 = b, b_strides[0], b_strides[1], b_batch[0], b_batch[1]
        d.c, d.c_rs, d.c_cs, d.c_b1, d.c_b2 = c, c_strides[0], c_strides[1], c_batch[0], c_batch[1]
        d.bias = bias
        d.reduce_batch, d.kernel, d.variant = int(bool(reduce_batch)), kernel, variant
        d.flags = (1 if no_split_k else 0) | ((split_k & 0xff) << 8)
        return d

    def gemm(self, desc: GemmDesc):
        """``MatMulImpl::matmul`` / ``Cuda::gemm[_batch]`` (cpu_kernel.rs:38-50, cuda_kernel.rs:153-237)."""
        self._check(self.lib.dfdx_rocm_gemm(self.ctx, ctypes.byref(desc)))

    def gemm_noalloc(self, desc: GemmDesc):
        """The same product with the partial sums of a split reduction in the library's fixed scratch array: allocates
        nothing; ``RocmError`` (code -5) when the plan needs more than ``NOALLOC_SCRATCH_BYTES``."""
        self._check(self.lib.dfdx_rocm_gemm_noalloc(self.ctx, ctypes.byref(desc)))

    def gemm_plan(self, desc: GemmDesc):
        kernel, variant = ctypes.c_int(), ctypes.c_int()
        name = ctypes.create_string_buffer(96)
        self._check(self.lib.dfdx_rocm_gemm_plan(self.ctx, ctypes.byref(desc), ctypes.byref(kernel),
                                                 ctypes.byref(variant), name, 96))
        return kernel.value, variant.value, name.value.decode()

    def gemm_time(self, desc: GemmDesc, warmup: int, iters: int) -> float:
        ms = ctypes.c_float()
        self._check(self.lib.dfdx_rocm_gemm_time(self.ctx, ctypes.byref(desc), warmup, iters, ctypes.byref(ms)))
        return ms.value

    def gemm_time_rotating(self, descs, warmup: int, iters: int) -> float:
        """Average ms per launch with launch i running ``descs[i % len(descs)]`` (each on its own buffers)."""
        arr = (GemmDesc * len(descs))(*descs)
        ms = ctypes.c_float()
        self._check(self.lib.dfdx_rocm_gemm_time_rotating(self.ctx, arr, len(descs), warmup, iters, ctypes.byref(ms)))
        return ms.value

    def mfma_variant_count(self, dtype: str) -> int:
        return self.lib.dfdx_rocm_mfma_variant_count(DTYPES[dtype])

    # --------------------------------------------------------- kernel traits --
    def forward(self, lhs: View, rhs: View) -> View:
        """Dispatch on rank like ``TryMatMul`` (mod.rs:133-311); rank-1 operands are reshapes (mod.rs:139-174)."""
        dt = lhs.dtype
        assert lhs.dtype == rhs.dtype
        L, R = len(lhs.shape), len(rhs.shape)
        vp = ctypes.c_void_p
        if L == 1 and R == 1:      # outer product: (M,1) x (1,N)
            m, n = lhs.shape[0], rhs.shape[0]
            out = self.empty(dt, (m, n))
            self._check(self.lib.dfdx_rocm_matmat_forward(
                self.ctx, DTYPES[dt], _c(m), _c(1), _c(n), vp(lhs.ptr), _i64arr((lhs.strides[0], 1)),
                vp(rhs.ptr), _i64arr((n * rhs.strides[0], rhs.strides[0])), vp(out.ptr)))
            return out
        if L == 1 and R == 2:      # (1,K) x (K,N) -> (N,)
            assert lhs.shape[0] == rhs.shape[0], f"left: {lhs.shape[0]}\n right: {rhs.shape[0]}"
            k, n = rhs.shape
            out = self.empty(dt, (n,))
            self._check(self.lib.dfdx_rocm_matmat_forward(
                self.ctx, DTYPES[dt], _c(1), _c(k), _c(n), vp(lhs.ptr), _i64arr((k * lhs.strides[0], lhs.strides[0])),
                vp(rhs.ptr), _i64arr(rhs.strides), vp(out.ptr)))
            return out
        if L == 2 and R == 1:      # (M,K) x (K,1) -> (M,)
            assert lhs.shape[1] == rhs.shape[0], f"left: {lhs.shape[1]}\n right: {rhs.shape[0]}"
            m, k = lhs.shape
            out = self.empty(dt, (m,))
            self._check(self.lib.dfdx_rocm_matmat_forward(
                self.ctx, DTYPES[dt], _c(m), _c(k), _c(1), vp(lhs.ptr), _i64arr(lhs.strides),
                vp(rhs.ptr), _i64arr((rhs.strides[0], 1)), vp(out.ptr)))
            return out
        if L == 2 and R == 2:
            assert lhs.shape[1] == rhs.shape[0], f"left: {lhs.shape[1]}\n right: {rhs.shape[0]}"
            (m, k), n = lhs.shape, rhs.shape[1]
            out = self.empty(dt, (m, n))
            self._check(self.lib.dfdx_rocm_matmat_forward(
                self.ctx, DTYPES[dt], _c(m), _c(k), _c(n), vp(lhs.ptr), _i64arr(lhs.strides),
                vp(rhs.ptr), _i64arr(rhs.strides), vp(out.ptr)))
            return out
        if L == 3 and R == 2:
            assert lhs.shape[2] == rhs.shape[0], f"left: {lhs.shape[2]}\n right: {rhs.shape[0]}"
            (b, m, k), n = lhs.shape, rhs.shape[1]
            out = self.empty(dt, (b, m, n))
            self._check(self.lib.dfdx_rocm_matmat_br_forward(
                self.ctx, DTYPES[dt], _c(b), _c(m), _c(k), _c(n), vp(lhs.ptr), _i64arr(lhs.strides),
                vp(rhs.ptr), _i64arr(rhs.strides), vp(out.ptr)))
            return out
        if L == 3 and R == 3:
            assert lhs.shape[0] == rhs.shape[0], f"left: {lhs.shape[0]}\n right: {rhs.shape[0]}"
            assert lhs.shape[2] == rhs.shape[1], f"left: {lhs.shape[2]}\n right: {rhs.shape[1]}"
            (b, m, k), n = lhs.shape, rhs.shape[2]
            out = self.empty(dt, (b, m, n))
            self._check(self.lib.dfdx_rocm_matmat_batch3_forward(
                self.ctx, DTYPES[dt], _c(b), _c(m), _c(k), _c(n), vp(lhs.ptr), _i64arr(lhs.strides),
                vp(rhs.ptr), _i64arr(rhs.strides), vp(out.ptr)))
            return out
        if L == 4 and R == 4:
            assert lhs.shape[0] == rhs.shape[0], f"left: {lhs.shape[0]}\n right: {rhs.shape[0]}"
            assert lhs.shape[1] == rhs.shape[1], f"left: {lhs.shape[1]}\n right: {rhs.shape[1]}"
            assert lhs.shape[3] == rhs.shape[2], f"left: {lhs.shape[3]}\n right: {rhs.shape[2]}"
            (b, s, m, k), n = lhs.shape, rhs.shape[3]
            out = self.empty(dt, (b, s, m, n))
            self._check(self.lib.dfdx_rocm_matmat_batch4_forward(
                self.ctx, DTYPES[dt], _c(b), _c(s), _c(m), _c(k), _c(n), vp(lhs.ptr), _i64arr(lhs.strides),
                vp(rhs.ptr), _i64arr(rhs.strides), vp(out.ptr)))
            return out
        raise TypeError(f"matmul of rank {L} by rank {R} is not defined (mod.rs:133-311)")

    def backward(self, lhs: View, grad_lhs: View, rhs: View, grad_rhs: View, grad_out: View):
        """``D::backward(lhs, grad_lhs, rhs, grad_rhs, grad_out)``; grad_out contiguous; grads accumulate."""
        dt = lhs.dtype
        L, R = len(lhs.shape), len(rhs.shape)
        vp = ctypes.c_void_p
        if L <= 2 and R <= 2:
            if L == 1 and R == 1:
                m, k, n = lhs.shape[0], 1, rhs.shape[0]
                ls, rs = (lhs.strides[0], 1), (n * rhs.strides[0], rhs.strides[0])
            elif L == 1:
                (k, n), m = rhs.shape, 1
                ls, rs = (k * lhs.strides[0], lhs.strides[0]), rhs.strides
            elif R == 1:
                (m, k), n = lhs.shape, 1
                ls, rs = lhs.strides, (rhs.strides[0], 1)
            else:
                (m, k), n = lhs.shape, rhs.shape[1]
                ls, rs = lhs.strides, rhs.strides
            self._check(self.lib.dfdx_rocm_matmat_backward(
                self.ctx, DTYPES[dt], _c(m), _c(k), _c(n), vp(lhs.ptr), _i64arr(ls), vp(grad_lhs.ptr),
                vp(rhs.ptr), _i64arr(rs), vp(grad_rhs.ptr), vp(grad_out.ptr)))
            return
        if L == 3 and R == 2:
            (b, m, k), n = lhs.shape, rhs.shape[1]
            fn, dims = self.lib.dfdx_rocm_matmat_br_backward, (b, m, k, n)
        elif L == 3 and R == 3:
            (b, m, k), n = lhs.shape, rhs.shape[2]
            fn, dims = self.lib.dfdx_rocm_matmat_batch3_backward, (b, m, k, n)
        elif L == 4 and R == 4:
            (b, s, m, k), n = lhs.shape, rhs.shape[3]
            fn, dims = self.lib.dfdx_rocm_matmat_batch4_backward, (b, s, m, k, n)
        else:
            raise TypeError(f"matmul of rank {L} by rank {R} is not defined")
        self._check(fn(self.ctx, DTYPES[dt], *[_c(d) for d in dims], vp(lhs.ptr), _i64arr(lhs.strides),
                       vp(grad_lhs.ptr), vp(rhs.ptr), _i64arr(rhs.strides), vp(grad_rhs.ptr), vp(grad_out.ptr)))

    def linear_forward(self, x: View, weight: View, bias: Optional[View]) -> View:
        """``Linear::try_forward`` (dfdx/src/nn/layers/linear.rs:82-89); weight is the (O, I) storage."""
        o, i = weight.shape
        assert weight.strides == (i, 1), "Linear weight storage is (O, I) row-major"
        assert x.shape[-1] == i, f"left: {x.shape[-1]}\n right: {i}"
        if len(x.shape) == 1:
            rows, xs = 1, (i * x.strides[0], x.strides[0])
        elif len(x.shape) == 2:
            rows, xs = x.shape[0], x.strides
        else:
            assert x.strides == _row_major(x.shape), "batched Linear input must be contiguous to fold its rows"
            rows, xs = int(np.prod(x.shape[:-1])), (i, 1)
        out = self.empty(x.dtype, tuple(x.shape[:-1]) + (o,))
        self._check(self.lib.dfdx_rocm_linear_forward(
            self.ctx, DTYPES[x.dtype], _c(rows), _c(i), _c(o), ctypes.c_void_p(x.ptr), _i64arr(xs),
            ctypes.c_void_p(weight.ptr), ctypes.c_void_p(bias.ptr if bias is not None else None),
            ctypes.c_void_p(out.ptr)))
        return out

    def _linear_rows(self, x: View, i: int):
        if len(x.shape) == 1:
            return 1, (i * x.strides[0], x.strides[0])
        if len(x.shape) == 2:
            return x.shape[0], x.strides
        assert x.strides == _row_major(x.shape), "batched Linear input must be contiguous to fold its rows"
        return int(np.prod(x.shape[:-1])), (i, 1)

    def linear_backward(self, x: View, grad_x: View, weight: View, grad_weight: View, grad_bias: Optional[View],
                        grad_out: View):
        """Backward of ``Linear``: grad_x += go.W, grad_weight += go^T.x, grad_bias += column sums of go."""
        o, i = weight.shape
        assert weight.strides == (i, 1), "Linear weight storage is (O, I) row-major"
        assert x.shape[-1] == i, f"left: {x.shape[-1]}\n right: {i}"
        assert grad_out.shape == tuple(x.shape[:-1]) + (o,) and grad_out.strides == _row_major(grad_out.shape)
        rows, xs = self._linear_rows(x, i)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_linear_backward(
            self.ctx, DTYPES[x.dtype], _c(rows), _c(i), _c(o), vp(x.ptr), _i64arr(xs), vp(grad_x.ptr),
            vp(weight.ptr), vp(grad_weight.ptr), vp(grad_bias.ptr if grad_bias is not None else None),
            vp(grad_out.ptr)))

    def bias_forward(self, x: View, bias: View) -> View:
        """``Bias1D::try_forward`` (dfdx/src/nn/layers/bias1d.rs:62-78) on a contiguous input."""
        cols = bias.shape[0]
        assert x.shape[-1] == cols, f"left: {x.shape[-1]}\n right: {cols}"
        assert x.strides == _row_major(x.shape) and bias.strides == (1,)
        rows = int(np.prod(x.shape[:-1], dtype=np.int64))
        out = self.empty(x.dtype, x.shape)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_bias_forward(self.ctx, DTYPES[x.dtype], _c(rows), _c(cols), vp(x.ptr),
                                                    vp(bias.ptr), vp(out.ptr)))
        return out

    def bias_backward(self, grad_out: View, grad_bias: View):
        """grad_bias += column sums of grad_out (the broadcast operand's share of the add's backward)."""
        cols = grad_bias.shape[0]
        assert grad_out.shape[-1] == cols and grad_out.strides == _row_major(grad_out.shape)
        rows = int(np.prod(grad_out.shape[:-1], dtype=np.int64))
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_bias_backward(self.ctx, DTYPES[grad_out.dtype], _c(rows), _c(cols),
                                                     vp(grad_out.ptr), vp(grad_bias.ptr)))

    # ------------------------------------------------- ops between attention's GEMMs --
    def scalar_mul_forward(self, x: View, scalar: float) -> View:
        """``x * scalar`` over the physical storage (unary kernel, utilities/cpu_kernels.rs:46-79); same strides."""
        out = View(self._torch.empty_like(x.storage), x.dtype, x.shape, x.strides, x.offset)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_scalar_mul_forward(self.ctx, DTYPES[x.dtype], _c(x.numel_storage()),
                                                          vp(x.storage.data_ptr()), ctypes.c_double(scalar),
                                                          vp(out.storage.data_ptr())))
        return out

    def scalar_mul_backward(self, scalar: float, grad_inp: View, grad_out: View):
        assert grad_inp.numel_storage() == grad_out.numel_storage()
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_scalar_mul_backward(self.ctx, DTYPES[grad_inp.dtype], _c(grad_inp.numel_storage()),
                                                           ctypes.c_double(scalar), vp(grad_inp.storage.data_ptr()),
                                                           vp(grad_out.storage.data_ptr())))

    def softmax_forward(self, x: View, scale: float = 1.0) -> View:
        """softmax(scale * x) over the last axis of a contiguous tensor (softmax.rs:70-83)."""
        assert x.strides == _row_major(x.shape), "softmax input must be contiguous"
        cols = x.shape[-1]
        rows = int(np.prod(x.shape[:-1], dtype=np.int64))
        out = View(self._torch.empty_like(x.storage), x.dtype, x.shape, x.strides)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_softmax_forward(self.ctx, DTYPES[x.dtype], _c(rows), _c(cols), vp(x.ptr),
                                                       ctypes.c_float(scale), vp(out.ptr)))
        return out

    def softmax_backward(self, out: View, grad_x: View, grad_out: View, scale: float = 1.0):
        assert out.strides == _row_major(out.shape) and grad_out.shape == out.shape and grad_x.shape == out.shape
        cols = out.shape[-1]
        rows = int(np.prod(out.shape[:-1], dtype=np.int64))
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_softmax_backward(self.ctx, DTYPES[out.dtype], _c(rows), _c(cols), vp(out.ptr),
                                                        ctypes.c_float(scale), vp(grad_x.ptr), vp(grad_out.ptr)))

    def reshape_forward(self, x: View, new_shape) -> View:
        """``try_reshape_like`` (reshape_to/mod.rs:90-115): free for a contiguous tensor, a copy otherwise."""
        new_shape = tuple(int(d) for d in new_shape)
        assert int(np.prod(x.shape, dtype=np.int64)) == int(np.prod(new_shape, dtype=np.int64)), \
            f"left: {int(np.prod(x.shape))}\n right: {int(np.prod(new_shape))}"
        if x.strides == _row_major(x.shape):
            return View(x.storage, x.dtype, new_shape, _row_major(new_shape), x.offset, x.owner)
        out = self.empty(x.dtype, new_shape)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_reshape_forward(self.ctx, DTYPES[x.dtype], len(x.shape), _i64arr(x.shape),
                                                       _i64arr(x.strides), vp(x.ptr), vp(out.ptr)))
        return out

    def reshape_backward(self, x: View, grad_inp: View, grad_out: View):
        """Backward of a copying reshape: grad_inp (laid out like x's storage) += grad_out through x's strides."""
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_reshape_backward(self.ctx, DTYPES[x.dtype], len(x.shape), _i64arr(x.shape),
                                                        _i64arr(x.strides), vp(grad_inp.ptr), vp(grad_out.ptr)))

    # ------------------------------------------- ops between an encoder block's GEMMs --
    def layer_norm_forward(self, x: View, gamma: View, beta: View, epsilon: float = 1e-5) -> View:
        """``LayerNorm1D::try_forward`` over the last axis of a contiguous tensor (layer_norm1d.rs:87-91)."""
        assert x.strides == _row_major(x.shape), "layer norm input must be contiguous"
        cols = x.shape[-1]
        assert gamma.shape == (cols,) and beta.shape == (cols,), f"left: {gamma.shape}\n right: {(cols,)}"
        rows = int(np.prod(x.shape[:-1], dtype=np.int64))
        out = View(self._torch.empty_like(x.storage), x.dtype, x.shape, x.strides)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_layer_norm_forward(self.ctx, DTYPES[x.dtype], _c(rows), _c(cols), vp(x.ptr), vp(gamma.ptr),
                                                          vp(beta.ptr), ctypes.c_double(epsilon), vp(out.ptr)))
        return out

    def layer_norm_backward(self, x: View, gamma: View, grad_x: View, grad_gamma: View, grad_beta: View, grad_out: View,
                            epsilon: float = 1e-5):
        assert x.strides == _row_major(x.shape) and grad_out.shape == x.shape and grad_x.shape == x.shape
        cols = x.shape[-1]
        rows = int(np.prod(x.shape[:-1], dtype=np.int64))
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_layer_norm_backward(self.ctx, DTYPES[x.dtype], _c(rows), _c(cols), vp(x.ptr), vp(gamma.ptr),
                                                           ctypes.c_double(epsilon), vp(grad_x.ptr), vp(grad_gamma.ptr),
                                                           vp(grad_beta.ptr), vp(grad_out.ptr)))

    def relu_forward(self, x: View) -> View:
        """``t.relu()`` over the physical storage (relu/cpu_kernel.rs:3-18); same strides."""
        out = View(self._torch.empty_like(x.storage), x.dtype, x.shape, x.strides, x.offset)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_relu_forward(self.ctx, DTYPES[x.dtype], _c(x.numel_storage()), vp(x.storage.data_ptr()),
                                                    vp(out.storage.data_ptr())))
        return out

    def relu_backward(self, x: View, grad_x: View, grad_out: View):
        assert grad_x.numel_storage() == grad_out.numel_storage() == x.numel_storage()
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_relu_backward(self.ctx, DTYPES[x.dtype], _c(x.numel_storage()), vp(x.storage.data_ptr()),
                                                     vp(grad_x.storage.data_ptr()), vp(grad_out.storage.data_ptr())))

    def add_forward(self, lhs: View, rhs: View) -> View:
        """``lhs + rhs`` for two tensors of one shape and layout (add/cpu_kernel.rs:4-26)."""
        assert lhs.shape == rhs.shape, f"left: {lhs.shape}\n right: {rhs.shape}"
        assert lhs.strides == rhs.strides and lhs.numel_storage() == rhs.numel_storage()
        out = View(self._torch.empty_like(lhs.storage), lhs.dtype, lhs.shape, lhs.strides, lhs.offset)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_add_forward(self.ctx, DTYPES[lhs.dtype], _c(lhs.numel_storage()), vp(lhs.storage.data_ptr()),
                                                   vp(rhs.storage.data_ptr()), vp(out.storage.data_ptr())))
        return out

    def add_backward(self, grad_lhs: View, grad_rhs: View, grad_out: View):
        assert grad_lhs.numel_storage() == grad_rhs.numel_storage() == grad_out.numel_storage()
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_add_backward(self.ctx, DTYPES[grad_out.dtype], _c(grad_out.numel_storage()),
                                                    vp(grad_lhs.storage.data_ptr()), vp(grad_rhs.storage.data_ptr()),
                                                    vp(grad_out.storage.data_ptr())))

    # ---------------------------------------------------------------- conv2d --
    def _conv2d_op(self, img: View, filters: View, stride, padding, dilation, groups) -> Conv2DOp:
        """Shape checks and output size of ``try_conv2d`` (conv2d/mod.rs:143-160, 279-308)."""
        shape = img.shape if len(img.shape) == 4 else (1,) + tuple(img.shape)
        batch, chan_in, h, w = shape
        chan_out, cg, kernel, k2 = filters.shape
        assert chan_in == cg * groups, f"left: {chan_in}\n right: {cg * groups}"
        assert kernel == k2, f"left: {kernel}\n right: {k2}"
        assert chan_out % groups == 0
        if img.strides != _row_major(img.shape) or filters.strides != _row_major(filters.shape):
            raise ValueError("Image & filter inputs to conv2d must be contiguous")
        size = lambda d: (d + 2 * padding - 1 - dilation * (kernel - 1)) // stride + 1
        assert h + 2 * padding - 1 >= dilation * (kernel - 1) and w + 2 * padding - 1 >= dilation * (kernel - 1)
        return Conv2DOp(kernel, stride, padding, dilation, groups, batch, chan_in, chan_out, h, size(h), w, size(w))

    def conv2d_forward(self, img: View, filters: View, stride=1, padding=0, dilation=1, groups=1) -> View:
        """``(img, filters).conv2d(stride, padding, dilation, groups)``; img (B, C, H, W) or (C, H, W)."""
        op = self._conv2d_op(img, filters, stride, padding, dilation, groups)
        lead = (op.batch,) if len(img.shape) == 4 else ()
        out = self.empty(img.dtype, lead + (op.chan_out, op.h_out, op.w_out))
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_conv2d_forward(self.ctx, DTYPES[img.dtype], ctypes.byref(op), vp(img.ptr),
                                                      vp(filters.ptr), vp(out.ptr)))
        return out

    def conv2d_backward(self, img: View, grad_img: View, filters: View, grad_filters: View, grad_out: View,
                        stride=1, padding=0, dilation=1, groups=1):
        op = self._conv2d_op(img, filters, stride, padding, dilation, groups)
        vp = ctypes.c_void_p
        self._check(self.lib.dfdx_rocm_conv2d_backward(self.ctx, DTYPES[img.dtype], ctypes.byref(op), vp(img.ptr),
                                                       vp(grad_img.ptr), vp(filters.ptr), vp(grad_filters.ptr),
                                                       vp(grad_out.ptr)))


def _c(v: int):
    return ctypes.c_int64(int(v))
