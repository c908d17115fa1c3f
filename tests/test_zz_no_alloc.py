"""GPU: the entry point that allocates nothing (`dfdx_rocm_gemm_noalloc`) against `dfdx_rocm_gemm`.

Both plan the same kernels; the only difference is where the f32 partial sums of a split reduction live (the
library's fixed per-GPU scratch array instead of a context-owned buffer that grows on demand), so the two results
must be identical bit for bit -- and both within the stated tolerance of the oracle
(max|err| <= 2e-3*sqrt(K)*max|a|*max|b| for f16 / bf16, 1e-5*sqrt(K)*... for f32).  Every case makes two calls in a
row, the second on a smaller product, because all calls on a GPU share the one array and it keeps the last call's
contents.  Runs last (file name) so that a failure here cannot hide another test.
"""
import numpy as np
import pytest

import oracle
from helpers import assert_within, rng
from gpu_util import announce, device, make_operand, values

pytestmark = pytest.mark.gpu

from dfdx_amd import RocmError  # noqa: E402
from dfdx_amd.rocm import ERR_SCRATCH_TOO_SMALL, KERNEL_AUTO, NOALLOC_SCRATCH_BYTES  # noqa: E402


def both_entries(dtype, m, k, n, layout, accumulate, seed, split_k=0, expect_split=True, check_oracle=True):
    """One product through both entry points on identical inputs; returns nothing, asserts everything."""
    dev = device()
    g = rng(seed)
    at, bt = layout
    a, astr = make_operand(g, m, k, at, dtype, dist="uniform")
    b, bstr = make_operand(g, k, n, bt, dtype, dist="uniform")
    c, cstr = make_operand(g, m, n, False, dtype)
    da, db = dev.tensor(a, dtype), dev.tensor(b, dtype)
    dc_ref, dc_new = dev.tensor(c, dtype), dev.tensor(c, dtype)

    def desc(dc):
        return dev.gemm_desc(dtype, m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, cstr, accumulate=accumulate,
                             kernel=KERNEL_AUTO, split_k=split_k)

    plan = dev.gemm_plan(desc(dc_new))[2]
    announce("gemm_noalloc", dtype, (m, k, n), layout, "acc" if accumulate else "ovw", "split_k", split_k, plan)
    if expect_split:
        assert "splitk" in plan or plan == "gemv", plan   # the case must exercise the scratch array
    dev.gemm_noalloc(desc(dc_new))
    dev.gemm(desc(dc_ref))
    dev.synchronize()
    got_st, ref_st = dev.to_host(dc_new), dev.to_host(dc_ref)
    assert np.array_equal(got_st.view(np.uint8), ref_st.view(np.uint8)), "noalloc entry differs from dfdx_rocm_gemm"
    if check_oracle:
        A, B = values(a, dtype, (m, k), astr), values(b, dtype, (k, n), bstr)
        c_or = c.copy()
        oracle.gemm(dtype, m, k, n, accumulate, a, astr, b, bstr, c_or, cstr)
        want = values(c_or, dtype, (m, n), cstr)
        ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}[dtype]
        assert_within(dtype, k, values(got_st, dtype, (m, n), cstr), want, A, B,
                      extra=2 * ulp * float(np.max(np.abs(want))), what="noalloc vs oracle")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_weight_gradient_shape_twice_second_smaller(dtype):
    # dW-shaped products (TN, beta = 1): few output tiles, long contraction -> the planner splits k
    both_entries(dtype, 512, 8192, 768, (True, False), True, seed=11)
    both_entries(dtype, 256, 4096, 384, (True, False), True, seed=12)


def test_f32_split_twice_second_smaller():
    both_entries("f32", 256, 4096, 512, (True, False), True, seed=21)
    both_entries("f32", 128, 4096, 384, (False, True), False, seed=22)


def test_forced_split_then_unsplit_then_sliced_vector_product():
    both_entries("f16", 1024, 4096, 1024, (False, False), False, seed=31, split_k=4)
    both_entries("f16", 256, 512, 256, (False, True), False, seed=32, expect_split=False)   # no scratch use at all
    # vec.mat with the k axis sliced over the grid: partial sums of the slices go through the same array
    both_entries("f16", 1, 16384, 4096, (False, False), False, seed=33)
    both_entries("f32", 1, 8192, 2048, (False, False), True, seed=34)


def test_full_size_scratch_and_refusal_beyond_it():
    dev = device()
    # config 3's weight gradient: 1024 x 1024 output, K = 16384, 8 splits = exactly the whole array
    both_entries("f16", 1024, 16384, 1024, (True, False), True, seed=41, split_k=8, check_oracle=False)
    # one split more than fits: refused before anything is launched, C untouched, and the ordinary entry still works
    m = n = 1024
    k = 16384
    g = rng(42)
    a, astr = make_operand(g, m, k, True, "f16", dist="uniform")
    b, bstr = make_operand(g, k, n, False, "f16", dist="uniform")
    c = np.full(m * n, 3.0, np.float16)
    da, db, dc = dev.tensor(a, "f16"), dev.tensor(b, "f16"), dev.tensor(c, "f16")
    desc = dev.gemm_desc("f16", m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, (n, 1), accumulate=True, split_k=9)
    assert 9 * m * n * 4 > NOALLOC_SCRATCH_BYTES
    announce("gemm_noalloc refusal", dev.gemm_plan(desc)[2])
    with pytest.raises(RocmError) as err:
        dev.gemm_noalloc(desc)
    assert err.value.code == ERR_SCRATCH_TOO_SMALL and "scratch" in str(err.value)
    dev.synchronize()
    assert np.array_equal(dev.to_host(dc), c)
    dev.gemm(desc)
    dev.synchronize()
    assert not np.array_equal(dev.to_host(dc), c)
