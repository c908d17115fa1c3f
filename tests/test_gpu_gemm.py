"""GPU parity: the strided batched GEMM entry (`dfdx_rocm_gemm`) against the CPU oracle.

Every kernel family and every MFMA tile variant is forced in turn, over all operand
layouts the matmul path produces (NN / TN / NT / TT, row- and column-major C), with
and without accumulation, on shapes that are not multiples of the tile sizes.
Tolerance: max|err| <= 1e-5*sqrt(K)*max|a|*max|b| for f32 and 2e-3*sqrt(K)*max|a|*max|b|
for f16 / bf16 (f32 accumulate), measured against the oracle's float64 shadow result;
the oracle's own f32-accumulated result must satisfy the same bound.
"""
import numpy as np
import pytest

import oracle
from helpers import assert_within, rng
from gpu_util import announce, device, make_operand, values

pytestmark = pytest.mark.gpu

from dfdx_amd import RocmError  # noqa: E402
from dfdx_amd.rocm import KERNEL_AUTO, KERNEL_GENERIC, KERNEL_MFMA  # noqa: E402

LAYOUTS = {"nn": (False, False), "tn": (True, False), "nt": (False, True), "tt": (True, True)}


def run_case(dtype, m, k, n, layout, accumulate, kernel, variant, c_colmajor=False, bias=False, seed=1, pads=(0, 0, 0),
             split_k=0):
    dev = device()
    g = rng(seed)
    at, bt = LAYOUTS[layout]
    a, astr = make_operand(g, m, k, at, dtype, pads[0])
    b, bstr = make_operand(g, k, n, bt, dtype, pads[1])
    c, cstr = make_operand(g, m, n, c_colmajor, dtype, pads[2])
    bias_st = oracle.to_storage(g.standard_normal(n), dtype) if bias else None
    A, B, C0 = values(a, dtype, (m, k), astr), values(b, dtype, (k, n), bstr), values(c, dtype, (m, n), cstr)

    da, db, dc = dev.tensor(a, dtype), dev.tensor(b, dtype), dev.tensor(c, dtype)
    dbias = dev.tensor(bias_st, dtype) if bias else None
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, cstr, accumulate=accumulate,
                         bias=dbias.ptr if bias else None, kernel=kernel, variant=variant, split_k=split_k)
    plan_name = dev.gemm_plan(desc)[2]
    announce("gemm", dtype, (m, k, n), layout, "acc" if accumulate else "ovw", "kernel", kernel, "variant", variant,
             "ccol" if c_colmajor else "crow", "bias" if bias else "", plan_name)
    dev.gemm(desc)
    dev.synchronize()
    got_st = dev.to_host(dc)
    got = values(got_st, dtype, (m, n), cstr)

    want = A @ B + (C0 if accumulate else 0.0) + (oracle.to_f64(bias_st, dtype) if bias else 0.0)
    ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8, "f64": 2.0 ** -53}[dtype]
    assert_within(dtype, k, got, want, A, B, extra=ulp * float(np.max(np.abs(want))), what="gpu vs f64")
    if not bias:  # the oracle proper (f32 accumulate, same rounding rule) on the same inputs; it has no bias term
        c_or = c.copy()
        oracle.gemm(dtype, m, k, n, accumulate, a, astr, b, bstr, c_or, cstr)
        want_or = values(c_or, dtype, (m, n), cstr)
        assert_within(dtype, k, got, want_or, A, B, extra=2 * ulp * float(np.max(np.abs(want))), what="gpu vs oracle")
    # nothing outside the C view is touched
    mask = np.ones(c.size, dtype=bool)
    idx = values(np.arange(c.size, dtype=np.float64), "f64", (m, n), cstr).astype(np.int64)
    mask[idx.reshape(-1)] = False
    assert np.array_equal(oracle.to_f64(got_st, dtype)[mask], oracle.to_f64(c, dtype)[mask])
    return plan_name


# ------------------------------------------------------------------ generic --
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("accumulate", [False, True])
def test_generic_kernel(dtype, layout, accumulate):
    run_case(dtype, 67, 45, 83, layout, accumulate, KERNEL_GENERIC, 0, pads=(3, 1, 2))


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 7, 5), (5, 7, 1), (5, 1, 7), (1, 300, 1), (130, 2, 3)])
def test_generic_degenerate_shapes(dtype, shape):
    m, k, n = shape
    run_case(dtype, m, k, n, "nn", True, KERNEL_GENERIC, 0)
    run_case(dtype, m, k, n, "tt", False, KERNEL_GENERIC, 0, c_colmajor=True)


def test_generic_k_zero_and_empty():
    dev = device()
    c = dev.tensor(np.full(6, 7.0, np.float32), "f32")
    a = dev.tensor(np.zeros(4, np.float32), "f32")
    announce("gemm k=0")
    dev.gemm(dev.gemm_desc("f32", 2, 0, 3, a.ptr, (0, 1), a.ptr, (3, 1), c.ptr, (3, 1), accumulate=True))
    assert np.array_equal(dev.to_host(c), np.full(6, 7.0, np.float32))
    dev.gemm(dev.gemm_desc("f32", 2, 0, 3, a.ptr, (0, 1), a.ptr, (3, 1), c.ptr, (3, 1), accumulate=False))
    assert np.array_equal(dev.to_host(c), np.zeros(6, np.float32))
    dev.gemm(dev.gemm_desc("f32", 0, 4, 3, a.ptr, (4, 1), a.ptr, (3, 1), c.ptr, (3, 1)))  # m = 0: no-op


def test_doubly_strided_operand_takes_generic_path():
    """Neither stride is 1 (reachable through user permutes/slices): Cuda panics there (mod.rs:323), Cpu does not.  A small
    product takes the k-sliced 16 x 16 kernel, which reads such an operand element by element and accepts any strides; a
    large one the generic kernel."""
    dev = device()
    g = rng(5)
    for dtype, (m, k, n), family, kernel_name in (("f16", (40, 24, 16), KERNEL_MFMA, "mfma16_small_16x16_ksliced"),
                                                  ("bf16", (40, 24, 16), KERNEL_MFMA, "mfma16_small_16x16_ksliced"),
                                                  ("f32", (40, 24, 16), KERNEL_MFMA, "mfma32_small_16x16_ksliced"),
                                                  ("f64", (40, 24, 16), KERNEL_MFMA, "mfma64_small_16x16_ksliced"),
                                                  ("f16", (600, 520, 440), KERNEL_GENERIC, "generic"),
                                                  ("f32", (600, 520, 440), KERNEL_MFMA, "mfma32_small_16x16_ksliced"),
                                                  ("f32", (1200, 1040, 880), KERNEL_GENERIC, "generic")):
        a = oracle.to_storage(g.standard_normal(m * (2 * k + 3)), dtype)
        astr = (2 * k + 3, 2)
        b, bstr = make_operand(g, k, n, False, dtype)
        c = oracle.to_storage(np.zeros(m * n), dtype)
        da, db, dc = dev.tensor(a, dtype), dev.tensor(b, dtype), dev.tensor(c, dtype)
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, (n, 1))
        plan = dev.gemm_plan(desc)
        assert plan[0] == family and plan[2] == kernel_name, plan
        announce("gemm doubly strided", dtype, (m, k, n), kernel_name)
        dev.gemm(desc)
        A, B = values(a, dtype, (m, k), astr), values(b, dtype, (k, n), bstr)
        assert_within(dtype, k, oracle.to_f64(dev.to_host(dc), dtype).reshape(m, n), A @ B, A, B, extra=1e-6)


def test_aliased_output_sums_or_is_rejected():
    """A zero stride on a matrix axis of C (the gradient view of a broadcast operand) sums the elements that share an
    address; a zero BATCH stride without `reduce_batch`, or a bias on such a view, is refused."""
    from dfdx_amd import RocmError

    dev = device()
    g = rng(77)
    A, B = g.integers(-3, 4, (4, 5)).astype(np.float32), g.integers(-3, 4, (5, 6)).astype(np.float32)
    a, b = dev.tensor(A.reshape(-1), "f32"), dev.tensor(B.reshape(-1), "f32")
    P = (A @ B).astype(np.float64)
    for c_strides, want, size in (((0, 1), P.sum(axis=0), 6), ((1, 0), P.sum(axis=1), 4), ((0, 0), P.sum(keepdims=True).reshape(-1), 1)):
        c = dev.tensor(np.full(size, 2.0, np.float32), "f32")
        announce("gemm into an aliased view", c_strides)
        dev.gemm(dev.gemm_desc("f32", 4, 5, 6, a.ptr, (5, 1), b.ptr, (6, 1), c.ptr, c_strides, accumulate=True))
        assert np.array_equal(dev.to_host(c).astype(np.float64), want + 2.0)   # small integers: exact in any order
        dev.gemm(dev.gemm_desc("f32", 4, 5, 6, a.ptr, (5, 1), b.ptr, (6, 1), c.ptr, c_strides, accumulate=False))
        assert np.array_equal(dev.to_host(c).astype(np.float64), want)
    c = dev.tensor(np.zeros(64, np.float32), "f32")
    with pytest.raises(RocmError) as e:   # two batches into one matrix without reduce_batch
        dev.gemm(dev.gemm_desc("f32", 4, 5, 6, a.ptr, (5, 1), b.ptr, (6, 1), c.ptr, (6, 1), batch=(2, 1)))
    assert e.value.code == -4
    with pytest.raises(RocmError) as e:   # a bias on a view whose columns share an address
        dev.gemm(dev.gemm_desc("f32", 4, 5, 6, a.ptr, (5, 1), b.ptr, (6, 1), c.ptr, (1, 0), bias=b.ptr))
    assert e.value.code == -4
    with pytest.raises(RocmError):
        dev.gemm(dev.gemm_desc("f32", -1, 4, 4, a.ptr, (4, 1), a.ptr, (4, 1), a.ptr, (4, 1)))


# --------------------------------------------------------------------- MFMA --
MFMA_SHAPES = [(200, 136, 264), (512, 256, 256), (96, 72, 40), (264, 192, 200), (72, 64, 136), (520, 128, 72),
               (264, 64, 200), (520, 64, 136)]   # K = 64: one k tile per work item


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("variant", list(range(1, 17)))
@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_mfma_variants(dtype, variant, layout):
    if variant > device().mfma_variant_count(dtype):
        pytest.skip("no such tile variant for this dtype")
    ran = 0
    for i, (m, k, n) in enumerate(MFMA_SHAPES):
        try:
            run_case(dtype, m, k, n, layout, bool(i % 2), KERNEL_MFMA, variant, seed=10 + i, pads=(8, 16, 8))
            ran += 1
        except RocmError as e:   # a variant may not serve a shape (the LDS-DMA kernels need K % 64 == 0)
            if e.code != -2:
                raise
    assert ran >= 2


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_mfma_column_major_c(dtype, layout):
    """A permuted operand's gradient is a column-major C (cpu_kernel.rs:283-284): solved as C^T = B^T A^T."""
    run_case(dtype, 264, 72, 136, layout, True, KERNEL_MFMA, 0, c_colmajor=True, pads=(0, 8, 8))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_small_kernel_tails_bias_and_wave_counts(layout, dtype):
    """The 16 x 16 kernel that cuts k over the waves of a workgroup, the last variant of every family: extents that are no
    multiple of 16 or 4 in any direction, every wave count (k = 20 .. 4096: 1, 2, 4, 8, 16 slices, one to four passes each), bias per column and
    (column-major C) per row, beta = 1, padded rows (vector loads off / on)."""
    dev = device()
    small = dev.mfma_variant_count(dtype)
    t = dev.zeros(dtype, (16, 16))
    assert dev.gemm_plan(dev.gemm_desc(dtype, 16, 16, 16, t.ptr, (16, 1), t.ptr, (16, 1), t.ptr, (16, 1), kernel=KERNEL_MFMA,
                                       variant=small))[2].endswith("small_16x16_ksliced")
    for i, (m, k, n) in enumerate([(64, 512, 256), (19, 20, 35), (33, 70, 17), (50, 131, 49), (16, 600, 16), (1, 77, 5), (130, 258, 3),
                                   (20, 2100, 18), (17, 4096, 33)]):
        for pads in ((0, 0, 0), (3, 1, 5), (8, 4, 4)):
            run_case(dtype, m, k, n, layout, bool(i % 2), KERNEL_MFMA, small, bias=(i % 3 == 0), c_colmajor=(i % 3 == 1 and n > 1),
                     seed=60 + i, pads=pads)


def test_small_f32_products_plan_the_small_kernel():
    """Config 1's three products take the small kernel on their own; a caller that asks for the plain k order does not."""
    dev = device()
    x, w, y = dev.tensor(np.zeros(64 * 512, np.float32), "f32"), dev.tensor(np.zeros(256 * 512, np.float32), "f32"), dev.tensor(np.zeros(64 * 256, np.float32), "f32")
    for desc in (dev.gemm_desc("f32", 64, 512, 256, x.ptr, (512, 1), w.ptr, (1, 512), y.ptr, (256, 1)),
                 dev.gemm_desc("f32", 64, 256, 512, y.ptr, (256, 1), w.ptr, (512, 1), x.ptr, (512, 1), accumulate=True),
                 dev.gemm_desc("f32", 512, 64, 256, x.ptr, (1, 512), y.ptr, (256, 1), w.ptr, (1, 512), accumulate=True)):
        assert dev.gemm_plan(desc)[2] == "mfma32_small_16x16_ksliced"
    # the plain k order asked for (broadcast-rhs forward): not this kernel
    from dfdx_amd.rocm import View
    assert "small" not in dev.gemm_plan(dev.gemm_desc("f32", 64, 512, 256, x.ptr, (512, 1), w.ptr, (1, 512), y.ptr, (256, 1), no_split_k=True))[2]


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_mfma_bias_epilogue(dtype):
    run_case(dtype, 136, 64, 200, "nt", False, KERNEL_MFMA, 0, bias=True)
    run_case(dtype, 136, 64, 200, "nt", False, KERNEL_MFMA, 0, bias=True, c_colmajor=True)
    run_case(dtype, 40, 64, 72, "nn", False, KERNEL_GENERIC, 0, bias=True)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_mfma_small_integer_operands_are_exact(dtype):
    """Integer operands with exactly representable products and sums: bit-exact whatever the summation order."""
    dev = device()
    g = rng(31)
    m, n = 256, 128
    ran = 0
    for k in (512, 64):   # 64: a single k tile, the conversions of the epilogue right behind the first MFMAs
        A = g.integers(-2, 3, (m, k)).astype(np.float64)
        B = g.integers(-2, 3, (k, n)).astype(np.float64)
        a, b = oracle.to_storage(A.reshape(-1), dtype), oracle.to_storage(B.reshape(-1), dtype)
        da, db, dc = dev.tensor(a, dtype), dev.tensor(b, dtype), dev.zeros(dtype, (m, n))
        for variant in range(1, dev.mfma_variant_count(dtype) + 1):
            announce("gemm exact ints", dtype, "k", k, "variant", variant)
            try:
                dev.gemm(dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (n, 1), dc.ptr, (n, 1), kernel=KERNEL_MFMA,
                                       variant=variant))
            except RocmError as e:
                if e.code != -2:
                    raise
                continue
            ran += 1
            got = oracle.to_f64(dev.to_host(dc), dtype).reshape(m, n)
            assert np.array_equal(got, A @ B)
    assert ran == 2 * dev.mfma_variant_count(dtype)


def test_auto_dispatch_prefers_mfma_when_aligned():
    dev = device()
    a = dev.zeros("f16", (256, 256))
    d = dev.gemm_desc("f16", 256, 256, 256, a.ptr, (256, 1), a.ptr, (256, 1), a.ptr, (256, 1))
    assert dev.gemm_plan(d)[0] == KERNEL_MFMA
    d = dev.gemm_desc("f16", 255, 256, 256, a.ptr, (1, 256), a.ptr, (256, 1), a.ptr, (256, 1))
    assert dev.gemm_plan(d)[0] == KERNEL_MFMA     # M-contiguous A with M % 8 != 0: the MFMA kernel's window loads
    d = dev.gemm_desc("f16", 128, 64, 128, a.ptr, (128, 2), a.ptr, (256, 1), a.ptr, (256, 1))
    assert dev.gemm_plan(d)[2] == "mfma16_small_16x16_ksliced"  # neither stride of A is 1: no tiled kernel; small enough
    d = dev.gemm_desc("f16", 1024, 256, 1024, a.ptr, (512, 2), a.ptr, (1024, 1), a.ptr, (1024, 1))
    assert dev.gemm_plan(d)[0] == KERNEL_GENERIC  # the same at a size where 16 x 16 tiles no longer pay
    d = dev.gemm_desc("f64", 256, 256, 256, a.ptr, (256, 1), a.ptr, (256, 1), a.ptr, (256, 1))
    assert dev.gemm_plan(d)[0] == KERNEL_MFMA and dev.gemm_plan(d)[2].startswith("mfma64")


# ----------------------------------------------------------- f64 on MFMA --
@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_mfma_f64_variants(variant, layout):
    """`MatMulImpl<f64>` (cpu_kernel.rs:189-229) on v_mfma_f64_16x16x4_f64: both tiles, every operand layout, extents that
    are no multiple of anything, overwrite and accumulate, row- and column-major C, bias, a k of 1 and of one k tile."""
    shapes = [(67, 45, 83), (130, 129, 200), (256, 16, 128), (16, 1, 16), (300, 64, 17)]
    for i, (m, k, n) in enumerate(shapes):
        run_case("f64", m, k, n, layout, bool(i % 2), KERNEL_MFMA, variant, c_colmajor=(i == 2), bias=(i == 1), seed=40 + i,
                 pads=((0, 0, 0), (3, 1, 2))[i % 2])


def test_mfma_f64_exact_on_integers_and_batched_reduce():
    dev, g = device(), rng(41)
    m, k, n, nb = 96, 80, 72, 5
    A = g.integers(-3, 4, (nb, m, k)).astype(np.float64)
    B = g.integers(-3, 4, (nb, k, n)).astype(np.float64)
    da, db = dev.tensor(A.reshape(-1), "f64"), dev.tensor(B.reshape(-1), "f64")
    dc = dev.zeros("f64", (nb, m, n))
    desc = dev.gemm_desc("f64", m, k, n, da.ptr, (k, 1), db.ptr, (n, 1), dc.ptr, (n, 1), batch=(nb, 1),
                         a_batch=(m * k, 0), b_batch=(k * n, 0), c_batch=(m * n, 0))
    assert dev.gemm_plan(desc)[2].startswith("mfma64")
    announce("gemm f64 batched", dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    assert np.array_equal(dev.to_host(dc).reshape(nb, m, n), A @ B)
    # all batches summed into one C, on top of what it holds (a broadcast operand's gradient)
    dr = dev.tensor(np.ones(m * n), "f64")
    desc = dev.gemm_desc("f64", m, k, n, da.ptr, (k, 1), db.ptr, (n, 1), dr.ptr, (n, 1), accumulate=True, batch=(nb, 1),
                         a_batch=(m * k, 0), b_batch=(k * n, 0), reduce_batch=True)
    announce("gemm f64 reduce", dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    assert np.array_equal(dev.to_host(dr).reshape(m, n), (A @ B).sum(axis=0) + 1.0)


# ------------------------------------------- operands off the 16-byte grid --
UNALIGNED_SHAPES = [
    # (m, k, n): odd everything; a vocabulary-sized extent (GPT-2's 50257) as n, as k and as m; k below one MFMA step
    (67, 45, 83), (33, 50257, 24), (16, 72, 50257), (50257, 40, 24), (130, 9, 70), (8, 8, 8), (257, 129, 255),
]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", UNALIGNED_SHAPES)
def test_unaligned_operands_run_on_the_mfma_kernels(dtype, shape):
    """Leading dimensions, extents and base addresses that are not multiples of 16 bytes (an LM head with 50257 outputs,
    its two gradients, a first-layer convolution with C*K*K = 27): the register-staged MFMA kernels walk such operands
    with window loads; only a view with no unit stride at all is left to the scalar kernel."""
    m, k, n = shape
    dev = device()
    for i, layout in enumerate(LAYOUTS):
        pads = ((1, 3, 5), (0, 0, 0), (7, 1, 0), (2, 2, 2))[i]
        g = rng(900 + i)
        at, bt = LAYOUTS[layout]
        a, astr = make_operand(g, m, k, at, dtype, pads[0])
        b, bstr = make_operand(g, k, n, bt, dtype, pads[1])
        da, db = dev.tensor(a, dtype), dev.tensor(b, dtype)
        dc = dev.zeros(dtype, (m, n + pads[2]))
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, astr, db.ptr, bstr, dc.ptr, (n + pads[2], 1))
        plan = dev.gemm_plan(desc)   # (a contraction of at most eight may go to the row-streaming kernel instead)
        assert plan[0] == KERNEL_MFMA or (k <= 8 and plan[2] == "thin_k"), (shape, layout, plan)
        run_case(dtype, m, k, n, layout, bool(i % 2), KERNEL_AUTO, 0, c_colmajor=(i == 3), seed=900 + i, pads=pads)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_unaligned_base_address_and_batch_strides(dtype):
    """Operands that start one element into their allocation, batches an odd number of elements apart."""
    dev, g = device(), rng(77)
    nb, m, k, n = 3, 70, 52, 41
    es = {"f16": 2, "f32": 4}[dtype]
    a_st = oracle.to_storage(g.standard_normal(1 + nb * (m * k + 1)), dtype)
    b_st = oracle.to_storage(g.standard_normal(1 + nb * (k * n + 3)), dtype)
    da, db, dc = dev.tensor(a_st, dtype), dev.tensor(b_st, dtype), dev.zeros(dtype, (nb, m, n))
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr + es, (k, 1), db.ptr + es, (n, 1), dc.ptr, (n, 1), batch=(nb, 1),
                         a_batch=(m * k + 1, 0), b_batch=(k * n + 3, 0), c_batch=(m * n, 0))
    assert dev.gemm_plan(desc)[0] == KERNEL_MFMA
    announce("gemm unaligned base / batch strides", dtype, dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    got = oracle.to_f64(dev.to_host(dc), dtype).reshape(nb, m, n)
    A64, B64 = oracle.to_f64(a_st, dtype), oracle.to_f64(b_st, dtype)
    for i in range(nb):
        A = A64[1 + i * (m * k + 1):][:m * k].reshape(m, k)
        B = B64[1 + i * (k * n + 3):][:k * n].reshape(k, n)
        assert_within(dtype, k, got[i], A @ B, A, B, extra=1e-6, what=f"batch {i}")


# --------------------------------------------------------------------- gemv --
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(1, 4096, 4096), (1, 520, 264), (1, 8200, 64), (4096, 4096, 1), (264, 520, 1), (72, 16384, 1)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
def test_gemv(dtype, shape, layout):
    """vec.mat (M = 1) and mat.vec (N = 1): the bandwidth-bound kernels, both matrix layouts, beta = 0 / 1, bias."""
    from dfdx_amd.rocm import KERNEL_GEMV
    m, k, n = shape
    dev = device()
    a = dev.zeros(dtype, (max(m, k), max(m, k)))
    at, bt = LAYOUTS[layout]
    astr = (1, m) if at else (k, 1)
    bstr = (1, k) if bt else (n, 1)
    plan = dev.gemm_plan(dev.gemm_desc(dtype, m, k, n, a.ptr, astr, a.ptr, bstr, a.ptr, (n, 1)))
    assert plan[0] == KERNEL_GEMV, plan
    run_case(dtype, m, k, n, layout, False, KERNEL_AUTO, 0, seed=3)
    run_case(dtype, m, k, n, layout, True, KERNEL_AUTO, 0, seed=4, bias=(dtype == "f32"))


@pytest.mark.parametrize("case", [("f32", 1, 8192, 8192, "nn"), ("f32", 8192, 8192, 1, "nn"), ("f32", 1, 8192, 8192, "nt"),
                                  ("f16", 1, 16384, 8192, "nn"), ("f32", 4, 8192, 8192, "nn"), ("f32", 8192, 8192, 3, "tn"),
                                  ("bf16", 2, 8192, 16384, "nt")],
                         ids=lambda c: "-".join(map(str, c)))
def test_vector_products_with_a_streamed_matrix(case):
    """From 256 MiB of matrix on, the vector-product kernels read it with non-temporal loads (it cannot stay cached
    between two products): the same sums, one and several vectors, both layouts, beta = 0 and 1."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dtype, m, k, n, layout = case
    run_case(dtype, m, k, n, layout, False, KERNEL_GEMV, 0, seed=21)
    run_case(dtype, m, k, n, layout, True, KERNEL_GEMV, 0, seed=22)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 1024, 1032), (3, 2056, 520), (4, 4096, 1024), (5, 1032, 2048), (8, 8200, 264), (7, 264, 8200),
                                   (1032, 1024, 2), (520, 2056, 3), (2048, 1032, 8), (8200, 264, 6)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
def test_gemv_multi(dtype, shape, layout):
    """2 .. 8 vectors against one streamed matrix (a Linear layer on a batch of a few rows; the gradients of a layer with a
    few outputs): every layout the matrix can be streamed in, either operand as the small one,
    beta = 0 / 1, bias, column-major C."""
    from dfdx_amd.rocm import KERNEL_GEMV
    m, k, n = shape
    dev = device()
    a = dev.zeros(dtype, (max(m, n) * k,))
    at, bt = LAYOUTS[layout]
    astr = (1, m) if at else (k, 1)
    bstr = (1, k) if bt else (n, 1)
    # the matrix must be walkable in 16-byte pieces along its outputs ("cols") or along k ("dots": then the vectors must be
    # contiguous in k as well); of the three layouts only A.B with the few columns in B is neither.  The planner weighs
    # this kernel against the matrix-core plans by estimated time, so the kernel is FORCED here (its family on request
    # takes the product whenever the kernel supports it) and the automatic plan, whichever it is, runs beside it.
    if n <= 8 and layout == "nn":
        forced = KERNEL_AUTO
    else:
        forced = KERNEL_GEMV
        plan = dev.gemm_plan(dev.gemm_desc(dtype, m, k, n, a.ptr, astr, a.ptr, bstr, a.ptr, (n, 1), kernel=KERNEL_GEMV))
        assert plan[0] == KERNEL_GEMV and plan[2] == "gemv_multi", (shape, layout, plan)
    run_case(dtype, m, k, n, layout, False, forced, 0, seed=5, bias=True)
    run_case(dtype, m, k, n, layout, True, forced, 0, seed=6, c_colmajor=True, bias=(dtype == "f32"))
    run_case(dtype, m, k, n, layout, True, forced, 0, seed=7, pads=(8, 8, 3))
    if forced != KERNEL_AUTO:
        run_case(dtype, m, k, n, layout, True, KERNEL_AUTO, 0, seed=8, bias=True)


@pytest.mark.parametrize("shape,layout", [((10, 8192, 1024), "tn"), ((1024, 8200, 10), "tn"), ((16, 8192, 520), "nn"), ((9, 16384, 264), "tn"),
                                          ((264, 8192, 13), "tt"), ((12, 16384, 520), "nn")])
def test_gemv_multi_nine_to_sixteen_vectors_f32(shape, layout):
    """The weight gradient of a layer with ten outputs over a batch of thousands of rows (both operands stored along the
    batch): up to sixteen vectors against the streamed matrix where the contraction is long (f32 from 8192 terms, the
    16-bit types from 16384); beta, bias, column-major C.  Shorter contractions keep their matrix-core plans."""
    from dfdx_amd.rocm import KERNEL_GEMV
    m, k, n = shape
    dev = device()
    a = dev.zeros("f32", (max(m, n) * k,))
    at, bt = LAYOUTS[layout]
    astr, bstr = (1, m) if at else (k, 1), (1, k) if bt else (n, 1)
    forced = lambda dt, kk: dev.gemm_plan(dev.gemm_desc(dt, m, kk, n, a.ptr, astr, a.ptr, bstr, a.ptr, (n, 1), kernel=KERNEL_GEMV))
    plan = forced("f32", k)
    assert plan[0] == KERNEL_GEMV and plan[2] == "gemv_multi", (shape, layout, plan)
    if k >= 16384:   # the 16-bit types take the form from 16384 terms on
        assert forced("f16", k)[2] == "gemv_multi"
        for dt in ("f16", "bf16"):
            run_case(dt, m, k, n, layout, True, KERNEL_GEMV, 0, seed=18, bias=True, pads=(8, 8, 3))
            run_case(dt, m, k, n, layout, False, KERNEL_GEMV, 0, seed=19, c_colmajor=True)
            run_case(dt, m, k, n, layout, False, KERNEL_AUTO, 0, seed=20)
    else:
        with pytest.raises(RocmError):   # shorter contractions with more than eight vectors: not this kernel's
            forced("f16", k)
    with pytest.raises(RocmError):
        forced("f32", 4096)
    run_case("f32", m, k, n, layout, False, KERNEL_GEMV, 0, seed=15, bias=True)
    run_case("f32", m, k, n, layout, True, KERNEL_GEMV, 0, seed=16, c_colmajor=True, bias=True)
    run_case("f32", m, k, n, layout, True, KERNEL_GEMV, 0, seed=17, pads=(8, 8, 3))
    run_case("f32", m, k, n, layout, True, KERNEL_AUTO, 0, seed=21, bias=True)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
def test_rank1_updates(dtype):
    """k = 1 (vec (x) vec, mod.rs:139-144, and the weight gradient of a vec.mat product): the elementwise kernel that
    streams C by whole rows; wide and narrow C, extents off the 16-byte grid, padded rows, strided vectors, beta = 0 / 1,
    bias per column and (column-major C) per row.  A single product, so f32 and f64 results equal the rounded product."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dev = device()
    for i, (m, n) in enumerate([(4096, 1024), (3, 5), (130, 24), (2, 4104), (515, 257), (64, 8), (1000, 3)]):
        a = dev.zeros(dtype, (max(m, n),))
        plan = dev.gemm_plan(dev.gemm_desc(dtype, m, 1, n, a.ptr, (1, 1), a.ptr, (n, 1), a.ptr, (n, 1)))
        assert plan[0] == KERNEL_GEMV and plan[2] == "rank1", plan
        for layout in ("nn", "tt"):
            for pads in ((0, 0, 0), (3, 5, 8), (1, 1, 3)):
                run_case(dtype, m, 1, n, layout, bool(i % 2), KERNEL_AUTO, 0, bias=(i % 3 == 0), c_colmajor=(i % 3 == 1), seed=90 + i, pads=pads)
                run_case(dtype, m, 1, n, layout, not (i % 2), KERNEL_GEMV, 0, bias=(i % 3 == 1), seed=70 + i, pads=pads)
    if dtype in ("f32", "f64"):
        g = rng(8)
        np_t = np.float32 if dtype == "f32" else np.float64
        x, y = g.standard_normal(300).astype(np_t), g.standard_normal(200).astype(np_t)
        dx, dy, dc = dev.tensor(x, dtype), dev.tensor(y, dtype), dev.zeros(dtype, (300, 200))
        dev.gemm(dev.gemm_desc(dtype, 300, 1, 200, dx.ptr, (1, 1), dy.ptr, (200, 1), dc.ptr, (200, 1)))
        assert np.array_equal(dev.to_host(dc).reshape(300, 200), np.outer(x, y))


@pytest.mark.parametrize("case", [("f32", 8192, 1, 8192), ("f32", 8192, 4, 8192), ("f16", 16384, 1, 8192), ("f64", 4096, 2, 8192)],
                         ids=lambda c: "-".join(map(str, c)))
def test_rank1_update_into_a_streamed_output(case):
    """Accumulating into 256 MiB of C or more, the row-streaming kernel reads and writes C with non-temporal accesses:
    the same sums as the cached form (and, for comparison, the overwriting product of the same shape, which stays cached)."""
    dtype, m, k, n = case
    dev = device()
    a = dev.zeros(dtype, (8,))
    plan = dev.gemm_plan(dev.gemm_desc(dtype, m, k, n, a.ptr, (k, 1), a.ptr, (n, 1), a.ptr, (n, 1), accumulate=True))
    if k == 1 or dtype == "f64":   # (f32 with k = 4 goes to the matrix-core form of the thin kernel: checked all the same)
        assert plan[2] in ("rank1", "thin_k"), plan
    run_case(dtype, m, k, n, "nn", True, KERNEL_AUTO, 0, seed=31)
    run_case(dtype, m, k, n, "nn", False, KERNEL_AUTO, 0, seed=32)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("k", [2, 3, 4, 5, 8])
def test_thin_contractions(dtype, k):
    """k = 2 .. 8 (a Linear layer on a handful of input features, the input gradient of a layer with a handful of outputs):
    the row-streaming kernel with the sum over k ascending; all four operand layouts, tails, padded rows, beta, bias."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dev = device()
    for i, (m, n) in enumerate([(2048, 1024), (3, 5), (130, 24), (515, 257), (1000, 3)]):
        a = dev.zeros(dtype, (max(m, n) * k,))
        plan = dev.gemm_plan(dev.gemm_desc(dtype, m, k, n, a.ptr, (k, 1), a.ptr, (n, 1), a.ptr, (n, 1)))
        if i == 0 and dtype != "f64" and k >= 3:   # a large row-major output: the thin contraction on the matrix cores
            assert plan[0] == KERNEL_GEMV and plan[2] == "thin_k_mfma", plan
        elif dtype in ("f32", "f64") or k <= 4:   # 16-bit types: up to k = 4 (beyond, the matrix-core kernels are as fast)
            assert plan[0] == KERNEL_GEMV and plan[2] == "thin_k", plan
        else:
            assert plan[2] != "thin_k", plan
        for layout in LAYOUTS:
            run_case(dtype, m, k, n, layout, bool(i % 2), KERNEL_AUTO, 0, bias=(i % 3 == 0), c_colmajor=(i % 3 == 1), seed=40 + i, pads=(i % 3, 2 * (i % 2), 3 * (i % 2)))
    a = dev.zeros(dtype, (4096,))
    assert dev.gemm_plan(dev.gemm_desc(dtype, 64, 9, 64, a.ptr, (9, 1), a.ptr, (64, 1), a.ptr, (64, 1)))[2] != "thin_k"


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("k", [3, 9, 16, 17, 31, 32])
def test_thin_contractions_on_matrix_cores(dtype, k):
    """k <= 32 with an output of megabytes (a low-rank factor applied to a batch of rows, the product that follows a
    projection to a handful of features): the row-streaming matrix-core kernel -- all four operand layouts, rows and
    columns that end inside a strip, rows of C on and off the 16-byte grid, a last piece that n cuts, beta, bias along the columns and (column-major C) along the rows."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dev = device()
    big = dtype == "f32" and k > 16   # f32 takes two rounds of MFMAs there and is planned for outputs of 64 MB and more
    shapes = [(4096, 4096), (4104, 4099)] if big else [(2048, 1024), (1030, 2056), (4100, 520), (520, 8200), (2048, 1029), (1031, 2050)]
    for i, (m, n) in enumerate(shapes):
        a = dev.zeros(dtype, (max(m, n) * k,))
        c = dev.zeros(dtype, (m * n,))
        d = dev.gemm_desc(dtype, m, k, n, a.ptr, (k, 1), a.ptr, (n, 1), c.ptr, (n, 1))
        plan = dev.gemm_plan(d)
        assert plan[0] == KERNEL_GEMV and plan[2] == "thin_k_mfma", plan
        del a, c
        for j, layout in enumerate(LAYOUTS):
            if big and j % 2 != i % 2:
                continue
            colmajor = (i + j) % 4 == 3
            # rows of C on the 16-byte grid (pad 0 or 8) and off it (pad 3: unaligned pieces; n = 1029: a cut last piece)
            run_case(dtype, m, k, n, layout, bool((i + j) % 2), KERNEL_AUTO, 0, bias=(j % 3 != 1), c_colmajor=colmajor,
                     seed=90 + 4 * i + j, pads=(j % 3, 2 * (i % 2), (0, 8, 3, 5)[(i + j) % 4]))
    # small outputs stay with the other kernels
    a = dev.zeros(dtype, (65536,))
    assert dev.gemm_plan(dev.gemm_desc(dtype, 256, 16, 256, a.ptr, (16, 1), a.ptr, (256, 1), a.ptr, (256, 1)))[2] != "thin_k_mfma"


# ------------------------------------------------------------------ split-k --
@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("layout", ["tn", "nt", "nn"])
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_split_k_forced(dtype, layout, splits):
    """k split over several workgroups, f32 partials combined in a fixed order; with beta = 1, bias, ragged edges."""
    run_case(dtype, 264, 1024, 200, layout, True, KERNEL_MFMA, 0, split_k=splits, pads=(8, 8, 8))
    run_case(dtype, 136, 512, 72, layout, False, KERNEL_MFMA, 0, split_k=splits, bias=True)
    run_case(dtype, 264, 576, 136, layout, True, KERNEL_MFMA, 0, split_k=splits, c_colmajor=True)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("splits", [0, 2, 5])
def test_split_k_register_staged_family(dtype, splits):
    """k not a multiple of 64, or operands off the 16-byte grid, with few output tiles and a long contraction (an LM head's
    dX): the register-staged kernels split the k loop as well; forced piece counts and the planner's own."""
    dev = device()
    for i, (m, k, n, layout, pads) in enumerate([(264, 1000, 200, "nn", (8, 8, 8)), (130, 2057, 72, "nt", (1, 3, 5)),
                                                 (96, 4104, 256, "tn", (0, 8, 0))]):
        run_case(dtype, m, k, n, layout, bool(i % 2), KERNEL_MFMA, 0, split_k=splits, seed=700 + i, pads=pads)
    a = dev.zeros(dtype, (512, 4104))   # (at 256 x 4104 x 256 the small-product kernel is the faster plan)
    d = dev.gemm_desc(dtype, 512, 4104, 512, a.ptr, (4104, 1), a.ptr, (1, 4104), a.ptr, (512, 1))
    assert "splitk" in dev.gemm_plan(d)[2] and "dma" not in dev.gemm_plan(d)[2], dev.gemm_plan(d)


def test_split_k_is_planned_for_weight_gradients_and_is_deterministic():
    dev = device()
    g = rng(77)
    m, k, n, dtype = 512, 8192, 512, "f16"      # dW-shaped: few output tiles, long contraction
    a = oracle.to_storage(g.standard_normal(k * m), dtype)      # stored (k, m): the transposed lhs of a weight gradient
    b = oracle.to_storage(g.standard_normal(k * n), dtype)
    c0 = oracle.to_storage(g.standard_normal(m * n), dtype)
    da, db = dev.tensor(a, dtype), dev.tensor(b, dtype)
    outs = []
    for _ in range(2):
        dc = dev.tensor(c0, dtype)
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (1, m), db.ptr, (n, 1), dc.ptr, (n, 1), accumulate=True)
        name = dev.gemm_plan(desc)[2]
        assert "splitk" in name, name
        announce("planned split-k", name)
        dev.gemm(desc)
        outs.append(dev.to_host(dc))
    assert np.array_equal(outs[0], outs[1])
    A, B = oracle.to_f64(a, dtype).reshape(k, m).T, oracle.to_f64(b, dtype).reshape(k, n)
    want = A @ B + oracle.to_f64(c0, dtype).reshape(m, n)
    assert_within(dtype, k, oracle.to_f64(outs[0], dtype).reshape(m, n), want, A, B, extra=2.0 ** -11 * np.abs(want).max())
    # NO_SPLIT_K keeps the plain kernel
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (1, m), db.ptr, (n, 1), dc.ptr, (n, 1), accumulate=True, no_split_k=True)
    assert "splitk" not in dev.gemm_plan(desc)[2]


def test_split_k_f32_planned_for_long_reductions():
    """f32: a small output with a long contraction (weight gradient, reduce-over-batch) is cut along k, gives the
    same bits on every run and stays within the f32 tolerance; NO_SPLIT_K switches it off."""
    dev, g = device(), rng(78)
    m, k, n, nb, dtype = 64, 3136, 576, 8, "f32"
    a = oracle.to_storage(g.standard_normal(nb * m * k), dtype)
    b = oracle.to_storage(g.standard_normal(nb * n * k), dtype)     # stored (nb, n, k): B^T per batch
    da, db = dev.tensor(a, dtype), dev.tensor(b, dtype)
    outs = []
    for _ in range(2):
        dc = dev.zeros(dtype, (m, n))
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (1, k), dc.ptr, (n, 1), accumulate=True,
                             batch=(nb, 1), a_batch=(m * k, 0), b_batch=(n * k, 0), reduce_batch=True)
        name = dev.gemm_plan(desc)[2]
        assert "mfma32" in name and "splitk" in name, name
        announce("planned f32 split-k", name)
        dev.gemm(desc)
        outs.append(dev.to_host(dc))
    assert np.array_equal(outs[0], outs[1])
    A, B = oracle.to_f64(a, dtype).reshape(nb, m, k), oracle.to_f64(b, dtype).reshape(nb, n, k)
    want = np.einsum("bmk,bnk->mn", A, B)
    assert_within(dtype, nb * k, oracle.to_f64(outs[0], dtype).reshape(m, n), want, A, B)
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (1, k), dc.ptr, (n, 1), accumulate=True,
                         batch=(nb, 1), a_batch=(m * k, 0), b_batch=(n * k, 0), reduce_batch=True, no_split_k=True)
    assert "splitk" not in dev.gemm_plan(desc)[2]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_split_k_many_ways_for_filter_gradient_shapes(dtype):
    """A convolution's filter gradient: one or two output tiles and a reduction over batch x pixels.  The planner cuts
    it into more than 16 pieces; forced counts beyond the planner's candidates (40, 64, 100) work too; every count
    gives the same bits on every run and stays within tolerance."""
    dev, g = device(), rng(79)
    m, k, n, nb = 64, 1024, 192, 48
    a = oracle.to_storage(g.standard_normal(nb * m * k), dtype)
    b = oracle.to_storage(g.standard_normal(nb * n * k), dtype)     # stored (nb, n, k): B^T per batch
    da, db = dev.tensor(a, dtype), dev.tensor(b, dtype)
    A, B = oracle.to_f64(a, dtype).reshape(nb, m, k), oracle.to_f64(b, dtype).reshape(nb, n, k)
    want = np.einsum("bmk,bnk->mn", A, B)
    ulp = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8, "f32": 2.0 ** -24}[dtype]
    for split_k in (0, 40, 64, 100):
        outs = []
        for _ in range(2):
            dc = dev.zeros(dtype, (m, n))
            desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (1, k), dc.ptr, (n, 1), accumulate=True,
                                 batch=(nb, 1), a_batch=(m * k, 0), b_batch=(n * k, 0), reduce_batch=True, split_k=split_k)
            name = dev.gemm_plan(desc)[2]
            announce("filter-gradient split-k", dtype, split_k, name)
            splits = int(name.rsplit("splitk", 1)[1]) if "splitk" in name else 1
            assert 16 < splits <= (split_k or 256), name     # a forced count shrinks until no piece is empty; the f32 planner goes up to 256
            dev.gemm(desc)
            outs.append(dev.to_host(dc))
        assert np.array_equal(outs[0], outs[1])
        assert_within(dtype, nb * k, oracle.to_f64(outs[0], dtype).reshape(m, n), want, A, B, extra=ulp * np.abs(want).max())


# ------------------------------------------------------- planner's choices --
@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_auto_dispatch_seeded_shape_sweep(dtype):
    """Whatever kernel, tile and split count the planner picks for a shape, the result is the oracle's: 48 seeded
    shapes per dtype through KERNEL_AUTO -- extents from 1 to ~700 (aligned to the MFMA kernels' 8 / 64 granules or
    not), contractions up to 4096, every operand layout, row- and column-major C, padded leading dimensions, with
    and without accumulation, with and without the fused bias."""
    g = rng(20240 + len(dtype))
    for i in range(48):
        kind = i % 4
        if kind == 0:      # everything aligned: the LDS-DMA family (16-bit) / the f32 MFMA kernel
            m, n, k = int(g.integers(1, 88)) * 8, int(g.integers(1, 88)) * 8, int(g.integers(1, 17)) * 64
        elif kind == 1:    # aligned rows / columns, k not a multiple of 64: the register-staged family
            m, n, k = int(g.integers(1, 88)) * 8, int(g.integers(1, 88)) * 8, int(g.integers(1, 130)) * 8
        elif kind == 2:    # few output tiles, long contraction: split-k candidates
            m, n, k = int(g.integers(4, 40)) * 8, int(g.integers(4, 40)) * 8, int(g.integers(16, 65)) * 64
        else:              # nothing aligned: the generic kernel (or GEMV when an extent is 1)
            m, n, k = int(g.integers(1, 300)), int(g.integers(1, 300)), int(g.integers(1, 500))
        layout = list(LAYOUTS)[int(g.integers(0, 4))]
        pads = tuple(int(g.integers(0, 3)) * 8 for _ in range(3)) if kind != 3 else tuple(int(g.integers(0, 5)) for _ in range(3))
        accumulate, ccol, bias = bool(g.integers(0, 2)), bool(g.integers(0, 4) == 0), bool(g.integers(0, 3) == 0)
        run_case(dtype, m, k, n, layout, accumulate, KERNEL_AUTO, 0, c_colmajor=ccol, bias=bias, seed=500 + i, pads=pads)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_auto_dispatch_few_rows_or_columns_sweep(dtype):
    """The corner of the planner where five kernel families compete: products of 1 ... 64 rows (or columns) against a
    matrix of 0.5 ... 32 MB -- a Linear layer on a handful of tokens and its gradients.  24 seeded shapes per dtype
    through KERNEL_AUTO (vector-product kernels, the k-sliced small kernel, LDS-DMA tiles with and without split-k, the
    split 64 x 64 tile), every operand layout, aligned and unaligned extents, with and without accumulation and bias;
    the kernels taken are counted so that a sweep that only ever reached one family fails."""
    g = rng(31000 + ["f16", "bf16", "f32"].index(dtype))
    few_choices = [1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 32, 48, 64]
    taken = {}
    for i in range(24):
        few = few_choices[int(g.integers(0, len(few_choices)))]
        aligned = i % 3 != 2
        gran = 8 if aligned else 1
        wide = int(g.integers(64, 1025)) * gran if aligned else int(g.integers(500, 4100))
        k = int(g.integers(4, 257)) * 64 if aligned else int(g.integers(300, 9000))
        while wide * k > (1 << 24):
            k //= 2
        m, n = (few, wide) if g.integers(0, 2) else (wide, few)
        layout = list(LAYOUTS)[int(g.integers(0, 4))]
        pads = tuple(int(g.integers(0, 2)) * 8 for _ in range(3)) if aligned else tuple(int(g.integers(0, 3)) for _ in range(3))
        accumulate, bias = bool(g.integers(0, 2)), bool(g.integers(0, 4) == 0)
        name = run_case(dtype, m, k, n, layout, accumulate, KERNEL_AUTO, 0, bias=bias, seed=900 + i, pads=pads)
        family = name.split("_")[0] + ("_small" if "small" in name else "_dma" if "dma" in name else "")
        taken[family] = taken.get(family, 0) + 1
    announce("few rows / columns sweep", dtype, taken)
    assert len(taken) >= 3, f"the sweep reached only {taken}"


def test_thin_contraction_with_more_than_2_31_output_elements():
    """70000 x 16 x 32768 in f16: 2.29 G elements of C (4.6 GB), so element offsets pass 2^31 (and byte offsets 2^32) --
    sampled row blocks, the last rows included, against the f64 product."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dev, g = device(), rng(97)
    m, k, n, dtype = 70000, 16, 32768, "f16"
    a = oracle.to_storage(g.standard_normal(m * k), dtype)
    b = oracle.to_storage(g.standard_normal(k * n), dtype)
    da, db, dc = dev.tensor(a, dtype), dev.tensor(b, dtype), dev.zeros(dtype, (m * n,))
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (n, 1), dc.ptr, (n, 1))
    plan = dev.gemm_plan(desc)
    announce("gemm beyond 2^31 elements", dtype, (m, k, n), plan[2])
    assert plan[0] == KERNEL_GEMV and plan[2] == "thin_k_mfma", plan
    dev.gemm(desc)
    dev.synchronize()
    A, B = oracle.to_f64(a, dtype).reshape(m, k), oracle.to_f64(b, dtype).reshape(k, n)
    for r0 in (0, 1008, 32768, 65520, 65536, m - 16):   # 65536 rows x 32768 columns = 2^31 elements
        raw = dc.storage[r0 * n * 2:(r0 + 16) * n * 2].cpu().numpy().view(np.float16)
        got = raw.astype(np.float64).reshape(16, n)
        want = A[r0:r0 + 16] @ B
        assert_within(dtype, k, got, want, A[r0:r0 + 16], B, extra=2.0 ** -11 * float(np.abs(want).max()), what=f"rows {r0}..")


# ------------------------------------------------------------------ batched --
@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("k", [12, 32])
def test_batched_thin_contractions(dtype, k):
    """Attention scores with a head dimension of 32 or less: two batch axes, head-interleaved rows of A, B stored along k
    (the transposed view of the keys), per batch or shared; beta = 1 and a bias; the row-streaming matrix-core kernel."""
    from dfdx_amd.rocm import KERNEL_GEMV
    dev = device()
    g = rng(43 + k)
    b1, b2, m, n = 2, 4, 520, 1024 if (dtype == "f32" and k > 16) else 512
    if dtype == "f32" and k > 16:
        b1 = 16     # planned for outputs of 64 MB and more there
    a = oracle.to_storage(g.standard_normal(b1 * m * b2 * k), dtype)   # stored (b1, m, b2, k)
    a_rs, a_cs, a_b1, a_b2 = b2 * k, 1, m * b2 * k, k
    A = values(a, dtype, (b1, b2, m, k), (a_b1, a_b2, a_rs, a_cs))
    da = dev.tensor(a, dtype)
    for shared in (False, True):
        nbm = 1 if shared else b1 * b2
        bmat = oracle.to_storage(g.standard_normal(nbm * n * k), dtype)   # stored (batches, n, k)
        B = oracle.to_f64(bmat, dtype).reshape((n, k) if shared else (b1, b2, n, k)).swapaxes(-1, -2)
        bias = oracle.to_storage(g.standard_normal(n), dtype)
        c0 = oracle.to_storage(g.standard_normal(b1 * b2 * m * n), dtype)
        db, dbias, dc = dev.tensor(bmat, dtype), dev.tensor(bias, dtype), dev.tensor(c0, dtype)
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (a_rs, a_cs), db.ptr, (1, k), dc.ptr, (n, 1), batch=(b1, b2),
                             a_batch=(a_b1, a_b2), b_batch=(0, 0) if shared else (b2 * n * k, n * k), c_batch=(b2 * m * n, m * n),
                             accumulate=shared, bias=dbias.ptr)
        plan = dev.gemm_plan(desc)
        announce("batched thin", dtype, k, "shared" if shared else "per batch", plan[2])
        assert plan[0] == KERNEL_GEMV and plan[2] == "thin_k_mfma", plan
        dev.gemm(desc)
        want = A @ B + oracle.to_f64(bias, dtype) + (oracle.to_f64(c0, dtype).reshape(b1, b2, m, n) if shared else 0.0)
        got = oracle.to_f64(dev.to_host(dc), dtype).reshape(b1, b2, m, n)
        ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}[dtype]
        assert_within(dtype, k, got, want, A, B, extra=2 * ulp * np.abs(want).max())


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("kernel", [KERNEL_GENERIC, KERNEL_MFMA])
def test_batched_and_reduce(dtype, kernel):
    """Two batch axes with head-interleaved strides, a broadcast (stride 0) B, and the reduce-over-batch mode."""
    dev = device()
    g = rng(41)
    b1, b2, m, k, n = 3, 4, 72, 64, 40
    # A stored (b1, m, b2, k): batch-2 stride (k) smaller than the row stride (b2*k)
    a = oracle.to_storage(g.standard_normal(b1 * m * b2 * k), dtype)
    a_rs, a_cs, a_b1, a_b2 = b2 * k, 1, m * b2 * k, k
    bmat = oracle.to_storage(g.standard_normal(k * n), dtype)  # shared by all batches
    c = np.zeros(b1 * b2 * m * n, oracle.NP_DTYPES[dtype])
    da, db, dc = dev.tensor(a, dtype), dev.tensor(bmat, dtype), dev.tensor(c, dtype)
    desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (a_rs, a_cs), db.ptr, (n, 1), dc.ptr, (n, 1), batch=(b1, b2),
                         a_batch=(a_b1, a_b2), b_batch=(0, 0), c_batch=(b2 * m * n, m * n), kernel=kernel)
    announce("batched", dtype, kernel, dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    A = values(a, dtype, (b1, b2, m, k), (a_b1, a_b2, a_rs, a_cs))
    B = oracle.to_f64(bmat, dtype).reshape(k, n)
    got = oracle.to_f64(dev.to_host(dc), dtype).reshape(b1, b2, m, n)
    assert_within(dtype, k, got, A @ B, A, B, extra=2.0 ** -10 * np.abs(A @ B).max())

    # reduce: G (k x n) += sum over batches A[b]^T (k x m) . D[b] (m x n)
    dmat = oracle.to_storage(g.standard_normal(b1 * b2 * m * n), dtype)
    gacc = oracle.to_storage(g.standard_normal(k * n), dtype)
    dd, dg = dev.tensor(dmat, dtype), dev.tensor(gacc, dtype)
    desc = dev.gemm_desc(dtype, k, m, n, da.ptr, (a_cs, a_rs), dd.ptr, (n, 1), dg.ptr, (n, 1), accumulate=True,
                         batch=(b1, b2), a_batch=(a_b1, a_b2), b_batch=(b2 * m * n, m * n), reduce_batch=True, kernel=kernel,
                         split_k=3 if (kernel == KERNEL_MFMA and dtype == "f16") else 0)
    announce("reduce", dtype, kernel, dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    D = oracle.to_f64(dmat, dtype).reshape(b1, b2, m, n)
    want = oracle.to_f64(gacc, dtype).reshape(k, n) + np.einsum("xymk,xymn->kn", A, D)
    got = oracle.to_f64(dev.to_host(dg), dtype).reshape(k, n)
    assert_within(dtype, b1 * b2 * m, got, want, A, D, extra=2.0 ** -10 * np.abs(want).max())
