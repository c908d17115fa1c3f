"""One context shared by several host threads (the reference's devices are Clone + Send + Sync,
dfdx-core/src/tensor/storage_traits.rs:15-17): call sequences that use the context's shared scratch memory --
split-k GEMMs, bias backward, conv2d -- must give the single-threaded bits when issued concurrently."""
import threading

import numpy as np
import pytest

import oracle
from helpers import rng
from gpu_util import announce, device

pytestmark = pytest.mark.gpu


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


def test_concurrent_split_k_bias_and_conv2d_calls():
    dev, g = device(), rng(901)
    announce("threads sharing one context")
    dtype = "f16"
    jobs = []
    for t in range(4):
        m, k, n = 256, 4096 + 1024 * t, 256                       # weight-gradient shaped: planned with split-k
        a, b = upload(dev, g.standard_normal((k, m)), dtype), upload(dev, g.standard_normal((k, n)), dtype)
        go = upload(dev, g.standard_normal((2048, 512 + 64 * t)), dtype)
        img = upload(dev, g.standard_normal((2, 16, 20 + t, 24)), dtype)
        flt = upload(dev, g.standard_normal((32, 16, 3, 3)) / 12.0, dtype)
        jobs.append((m, k, n, a, b, go, img, flt))

    def run(job):
        m, k, n, a, b, go, img, flt = job
        c = dev.zeros(dtype, (m, n))
        desc = dev.gemm_desc(dtype, m, k, n, a.ptr, (1, m), b.ptr, (n, 1), c.ptr, (n, 1), accumulate=True)
        assert "splitk" in dev.gemm_plan(desc)[2]
        dev.gemm(desc)
        gb = dev.zeros(dtype, (go.shape[1],))
        dev.bias_backward(go, gb)
        y = dev.conv2d_forward(img, flt, padding=1)
        gi, gf = dev.zeros_like_storage(img), dev.zeros_like_storage(flt)
        dev.conv2d_backward(img, gi, flt, gf, y, padding=1)
        return [dev.to_host(t).copy() for t in (c, gb, y, gi, gf)]

    want = [run(j) for j in jobs]
    got = [[None] * 6 for _ in jobs]
    errors = []

    def worker(i):
        try:
            for r in range(6):
                got[i][r] = run(jobs[i])
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(len(jobs)):
        for r in range(6):
            for w, x in zip(want[i], got[i][r]):
                np.testing.assert_array_equal(x, w)
