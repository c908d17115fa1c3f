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
