"""GPU: the storage helpers of the C ABI.  `dfdx_rocm_memset_zero` / `dfdx_rocm_alloc(zeroed)` stand in for
``Storage::try_alloc_len`` (tensor/cuda/device.rs:259-266: a fresh buffer is all zeros, which every gradient buffer
relies on, tensor/gradients.rs:53-58).  The fill is a kernel of this library: every byte of the range is cleared and
no byte outside it is touched, at any alignment and size."""
import ctypes

import numpy as np
import pytest

from gpu_util import announce, device

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("offset", [0, 1, 7, 15, 16, 33])
def test_memset_zero_clears_exactly_the_range(offset):
    import torch

    dev = device()
    sizes = [0, 1, 5, 15, 16, 17, 31, 255, 4096, 16384, 16385, 65536 + 3, (1 << 20) + 17, 5 * (1 << 20) + 1]
    for nbytes in sizes:
        total = offset + nbytes + 64
        buf = torch.full((total,), 0xA5, dtype=torch.uint8, device="cuda")
        announce("memset_zero", "offset", offset, "bytes", nbytes)
        dev._check(dev.lib.dfdx_rocm_memset_zero(dev.ctx, ctypes.c_void_p(buf.data_ptr() + offset), ctypes.c_size_t(nbytes)))
        dev.synchronize()
        got = buf.cpu().numpy()
        assert np.all(got[:offset] == 0xA5), (offset, nbytes)
        assert np.all(got[offset:offset + nbytes] == 0), (offset, nbytes)
        assert np.all(got[offset + nbytes:] == 0xA5), (offset, nbytes)


def test_alloc_zeroed_and_free():
    dev = device()
    for nbytes in (1, 100, 1 << 20, (64 << 20) + 24):
        ptr = ctypes.c_void_p()
        announce("alloc zeroed", nbytes)
        dev._check(dev.lib.dfdx_rocm_alloc(dev.ctx, ctypes.c_size_t(nbytes), 1, ctypes.byref(ptr)))
        host = np.full(nbytes, 0x5A, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_d2h(dev.ctx, host.ctypes.data_as(ctypes.c_void_p), ptr, ctypes.c_size_t(nbytes)))
        dev._check(dev.lib.dfdx_rocm_free(dev.ctx, ptr))
        assert not host.any()


def test_zeros_views_are_zero():
    dev = device()
    v = dev.zeros("f16", (3, 5, 7))
    assert not dev.to_host(v).any()
    w = dev.zeros_like_storage(dev.tensor(np.ones(1000, np.float32), "f32"))
    assert not dev.to_host(w).any()


def test_allocation_cache_reuses_and_releases():
    """`Cache` (tensor/storage_traits.rs:41-77) over `TensorCache` semantics (tensor/cache.rs:105-149, and its own unit
    tests :192-260): off at first; while on, a freed buffer is handed to the next allocation of exactly its size (and to
    no other size), zero-filled again when asked; `empty` and `disable` give everything back."""
    dev = device()
    announce("allocation cache")
    assert dev.cache_stats() == (0, 0)
    a = dev.alloc(1 << 20)
    dev.free(a)
    assert dev.cache_stats() == (0, 0)                 # disabled: freed for real
    dev.enable_cache()
    try:
        a = dev.alloc(1 << 20, zeroed=False)
        b = dev.alloc(1 << 20, zeroed=False)
        c = dev.alloc(4096, zeroed=False)
        ones = np.full(1 << 20, 0x77, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_h2d(dev.ctx, ctypes.c_void_p(a), ones.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(ones.nbytes)))
        dev.free(a)
        dev.free(c)
        assert dev.cache_stats() == (2, (1 << 20) + 4096)
        d = dev.alloc(2 << 20, zeroed=False)           # another size: a fresh buffer, the cache keeps its two
        assert d not in (a, c) and dev.cache_stats() == (2, (1 << 20) + 4096)
        e = dev.alloc(1 << 20, zeroed=True)            # same size: the cached buffer, cleared again
        assert e == a and dev.cache_stats() == (1, 4096)
        host = np.full(1 << 20, 0x5A, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_d2h(dev.ctx, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(e), ctypes.c_size_t(host.nbytes)))
        assert not host.any()
        f = dev.alloc(4096, zeroed=False)
        assert f == c and dev.cache_stats() == (0, 0)
        for p in (b, d, e, f):
            dev.free(p)
        assert dev.cache_stats() == (4, (1 << 20) * 2 + (2 << 20) + 4096)
        dev.empty_cache()
        assert dev.cache_stats() == (0, 0)
        g = dev.alloc(1 << 20)
        dev.free(g)
        assert dev.cache_stats()[0] == 1
    finally:
        dev.disable_cache()                            # also empties
    assert dev.cache_stats() == (0, 0)
    h = dev.alloc(64)
    dev.free(h)
    assert dev.cache_stats() == (0, 0)


def test_workspace_growth_does_not_disturb_queued_work():
    """A split product that needs a larger workspace than the context holds gets a new one while the launches queued
    before it keep the old one (retired, freed at the next synchronize): both results are right, in either order."""
    import oracle
    from gpu_util import make_operand, values
    from helpers import assert_within, rng
    from dfdx_amd import Rocm

    dev = Rocm(0)   # a context of its own: its workspace starts empty
    g = rng(91)
    outs = []
    for (m, k, n, split) in ((64, 2048, 64, 4), (256, 4096, 512, 8), (128, 2048, 128, 4), (512, 4096, 1024, 8)):
        a, astr = make_operand(g, m, k, True, "f32")
        b, bstr = make_operand(g, k, n, False, "f32")
        c = np.zeros(m * n, np.float32)
        da, db, dc = dev.tensor(a, "f32"), dev.tensor(b, "f32"), dev.tensor(c, "f32")
        desc = dev.gemm_desc("f32", m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, (n, 1), split_k=split, kernel=2, variant=4)
        announce("workspace growth", (m, k, n), dev.gemm_plan(desc)[2])
        assert "splitk" in dev.gemm_plan(desc)[2]
        dev.gemm(desc)   # no synchronize in between: the next, larger product is planned while this one may still run
        outs.append((dc, values(a, "f32", (m, k), astr), values(b, "f32", (k, n), bstr), (m, k, n), (da, db)))
    dev.synchronize()
    for dc, A, B, (m, k, n), _keep in outs:
        assert_within("f32", k, dev.to_host(dc).astype(np.float64).reshape(m, n), A @ B, A, B, extra=1e-5)
