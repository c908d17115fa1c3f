"""Pin what the golden literals leave open: other dtypes, strided / batched
operands, accumulation, and the conversion routines -- against things the
mathematics fixes (float64 BLAS products, exact small-integer products, the
identities the reference's tests assert in matmul/mod.rs:413-527)."""
import numpy as np
import pytest
import torch

from helpers import assert_within, logical, permute, rng, row_major_strides


# ------------------------------------------------------------- conversions --
def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_to_f32(bits.view(np.float16))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_matches_ieee_rne(oracle):
    g = rng(11)
    x = np.concatenate([
        g.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** g.integers(-9, 6, 200000).astype(np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),            # every f16 value
        np.nextafter(np.arange(1, 2048, dtype=np.float32) * np.float32(2 ** -25), np.float32(1)),  # subnormal ties +ulp
        np.arange(1, 4096, dtype=np.float32) * np.float32(2 ** -25),                      # exact subnormal ties
        np.array([65504, 65519.99, 65520, 65536, 1e30, -1e30, np.inf, -np.inf, 0.0, -0.0, 2 ** -24, 2 ** -25, 2 ** -26], np.float32),
    ])
    x = x[np.isfinite(x) | np.isinf(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = oracle.f32_to_f16(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_bf16_conversions_match_torch(oracle):
    g = rng(12)
    x = g.standard_normal(300000).astype(np.float32) * np.float32(10.0) ** g.integers(-20, 20, 300000).astype(np.float32)
    x = np.concatenate([x, np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 1.00390625, 1.005859375, 3.3895314e38], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16)
    got = oracle.f32_to_bf16(x)
    assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16))
    back = oracle.bf16_to_f32(got)
    assert np.array_equal(back.view(np.uint32), want.to(torch.float32).numpy().view(np.uint32))


# -------------------------------------------------------------------- gemm --
LAYOUTS = ["nn", "tn", "nt", "tt", "c_colmajor", "strided"]


def make_view(g, rows, cols, layout_t, dtype, oracle, pad=0, scale=1.0):
    """A (rows, cols) matrix view over fresh storage; layout_t stores it transposed."""
    if layout_t:
        st = g.standard_normal((cols, rows + pad)) * scale
        strides = [1, rows + pad]
    else:
        st = g.standard_normal((rows, cols + pad)) * scale
        strides = [cols + pad, 1]
    return oracle.to_storage(st.reshape(-1), dtype), strides


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("accum", [False, True])
def test_gemm_against_f64_blas(oracle, dtype, layout, accum):
    g = rng(100 + LAYOUTS.index(layout))
    m, k, n = 37, 53, 29
    a, astr = make_view(g, m, k, layout in ("tn", "tt"), dtype, oracle, pad=3 if layout == "strided" else 0)
    b, bstr = make_view(g, k, n, layout in ("nt", "tt"), dtype, oracle, pad=5 if layout == "strided" else 0)
    if layout == "strided":  # neither stride is 1: every second column of a wider matrix
        astr = [2 * k + 3, 2]
        a = oracle.to_storage(g.standard_normal(m * astr[0]), dtype)
    c, cstr = make_view(g, m, n, layout == "c_colmajor", dtype, oracle, pad=2)
    A = logical(oracle.to_f64(a, dtype), (m, k), astr)
    B = logical(oracle.to_f64(b, dtype), (k, n), bstr)
    C0 = logical(oracle.to_f64(c, dtype), (m, n), cstr)
    untouched = oracle.to_f64(c, dtype).copy()
    want = A @ B + (C0 if accum else 0.0)
    oracle.gemm(dtype, m, k, n, accum, a, astr, b, bstr, c, cstr)
    got = logical(oracle.to_f64(c, dtype), (m, n), cstr)
    # storage rounding of the result itself: half an ulp of the output dtype
    ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8, "f64": 2.0 ** -53}[dtype]
    assert_within(dtype, k, got, want, A, B, extra=ulp * float(np.max(np.abs(want))), what=f"{dtype}/{layout}")
    # elements of C's storage outside the view (the padding) are not written
    mask = np.ones(untouched.shape, dtype=bool)
    idx = logical(np.arange(untouched.size, dtype=np.float64), (m, n), cstr).astype(np.int64)
    mask[idx.reshape(-1)] = False
    assert np.array_equal(oracle.to_f64(c, dtype)[mask], untouched[mask])


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16", "f64"])
def test_gemm_small_integers_exact(oracle, dtype):
    """Integer operands whose products and sums are exact in every dtype: bit-exact result expected."""
    g = rng(7)
    m, k, n = 24, 40, 17
    A = g.integers(-3, 4, (m, k)).astype(np.float64)
    B = g.integers(-3, 4, (k, n)).astype(np.float64)
    C0 = g.integers(-8, 9, (m, n)).astype(np.float64)
    want = A @ B + C0  # |.| <= 40*9 + 8 = 368 < 2^9: exact in bf16's 8 bits only if small; keep check on magnitude
    a, b, c = (oracle.to_storage(x.reshape(-1), dtype) for x in (A, B, C0))
    oracle.gemm(dtype, m, k, n, True, a, [k, 1], b, [n, 1], c, [n, 1])
    got = oracle.to_f64(c, dtype).reshape(m, n)
    if dtype == "bf16":  # bf16 holds integers exactly only up to 256: compare against RNE-rounded truth
        want = oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32))).astype(np.float64)
    assert np.array_equal(got, want)


def test_gemm_accumulate_twice_is_double(oracle):
    g = rng(8)
    m, k, n = 8, 16, 8
    a = g.integers(-2, 3, m * k).astype(np.float32)
    b = g.integers(-2, 3, k * n).astype(np.float32)
    c = np.zeros(m * n, np.float32)
    oracle.gemm("f32", m, k, n, True, a, [k, 1], b, [n, 1], c, [n, 1])
    once = c.copy()
    oracle.gemm("f32", m, k, n, True, a, [k, 1], b, [n, 1], c, [n, 1])
    assert np.array_equal(c, 2 * once)
    oracle.gemm("f32", m, k, n, False, a, [k, 1], b, [n, 1], c, [n, 1])  # overwrite ignores old contents
    assert np.array_equal(c, once)


def test_gemm_identity_and_permutation(oracle):
    g = rng(9)
    n = 33
    x = g.standard_normal((n, n)).astype(np.float32)
    eye = np.eye(n, dtype=np.float32)
    perm = eye[g.permutation(n)]
    c = np.empty(n * n, np.float32)
    oracle.gemm("f32", n, n, n, False, x.reshape(-1), [n, 1], eye.reshape(-1), [n, 1], c, [n, 1])
    assert np.array_equal(c.reshape(n, n), x)
    oracle.gemm("f32", n, n, n, False, perm.reshape(-1), [n, 1], x.reshape(-1), [n, 1], c, [n, 1])
    assert np.array_equal(c.reshape(n, n), perm @ x)


def test_gemm_degenerate_dims(oracle):
    c = np.full(6, 7.0, np.float32)
    a = np.zeros(1, np.float32)
    oracle.gemm("f32", 2, 0, 3, False, a, [0, 1], a, [3, 1], c, [3, 1])  # K = 0: overwrite with zeros
    assert np.array_equal(c, np.zeros(6, np.float32))
    c[:] = 7.0
    oracle.gemm("f32", 2, 0, 3, True, a, [0, 1], a, [3, 1], c, [3, 1])  # K = 0, accumulate: unchanged
    assert np.array_equal(c, np.full(6, 7.0, np.float32))
    oracle.gemm("f32", 0, 4, 3, False, a, [4, 1], a, [3, 1], c, [3, 1])  # M = 0: nothing written
    assert np.array_equal(c, np.full(6, 7.0, np.float32))


# ---------------------------------------------------------- kernel drivers --
def _rand_storage(g, n, dtype, oracle):
    return oracle.to_storage(g.standard_normal(n), dtype)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_transpose_identity_with_grads(oracle, dtype):
    """(A.B)^T == B^T.A^T, gradients included (matmul/mod.rs:413-426)."""
    g = rng(21)
    m, k, n = 4, 3, 2
    a, b = _rand_storage(g, m * k, dtype, oracle), _rand_storage(g, k * n, dtype, oracle)
    go = _rand_storage(g, m * n, dtype, oracle)
    out1 = oracle.matmat_forward(dtype, m, k, n, a, [k, 1], b, [n, 1])
    ga1, gb1 = np.zeros_like(a), np.zeros_like(b)
    oracle.matmat_backward(dtype, m, k, n, a, [k, 1], ga1, b, [n, 1], gb1, go)
    # second form: lhs = b permuted (n,k) strides [1,n]; rhs = a permuted (k,m) strides [1,k]
    out2 = oracle.matmat_forward(dtype, n, k, m, b, [1, n], a, [1, k])
    go_t = np.ascontiguousarray(go.reshape(m, n).T).reshape(-1)
    ga2, gb2 = np.zeros_like(a), np.zeros_like(b)
    oracle.matmat_backward(dtype, n, k, m, b, [1, n], gb2, a, [1, k], ga2, go_t)
    assert np.array_equal(out1.reshape(m, n), out2.reshape(n, m).T)
    assert np.array_equal(ga1, ga2) and np.array_equal(gb1, gb2)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_broadcast_equals_per_slice_and_stacked(oracle, dtype):
    """Br == loop of 2-D products; grad_rhs == sum over slices (mod.rs:429-457);
    Br == Batch3 with a stacked rhs, exactly, for out and grad_lhs (mod.rs:460-473)."""
    g = rng(22)
    bsz, m, k, n = 5, 4, 3, 2
    a, b = _rand_storage(g, bsz * m * k, dtype, oracle), _rand_storage(g, k * n, dtype, oracle)
    go = _rand_storage(g, bsz * m * n, dtype, oracle)
    ls = row_major_strides((bsz, m, k))
    out = oracle.matmat_br_forward(dtype, bsz, m, k, n, a, ls, b, [n, 1])
    ga, gb = np.zeros_like(a), np.zeros_like(b)
    oracle.matmat_br_backward(dtype, bsz, m, k, n, a, ls, ga, b, [n, 1], gb, go)

    gb_sum = np.zeros(k * n)
    for i in range(bsz):
        sub_a, sub_go = a[i * m * k:(i + 1) * m * k].copy(), go[i * m * n:(i + 1) * m * n].copy()
        sub_out = oracle.matmat_forward(dtype, m, k, n, sub_a, [k, 1], b, [n, 1])
        assert np.array_equal(sub_out, out[i * m * n:(i + 1) * m * n])
        sga, sgb = np.zeros_like(sub_a), np.zeros_like(b)
        oracle.matmat_backward(dtype, m, k, n, sub_a, [k, 1], sga, b, [n, 1], sgb, sub_go)
        assert np.array_equal(sga, ga[i * m * k:(i + 1) * m * k])
        gb_sum += oracle.to_f64(sgb, dtype)
    A = oracle.to_f64(a, dtype).reshape(bsz * m, k)
    G = oracle.to_f64(go, dtype).reshape(bsz * m, n)
    assert_within(dtype, bsz * m, oracle.to_f64(gb, dtype), gb_sum, A, G, extra=2.0 ** -7 * np.abs(gb_sum).max())

    b_up = np.tile(b, bsz)
    out3 = oracle.matmat_batch3_forward(dtype, bsz, m, k, n, a, ls, b_up, row_major_strides((bsz, k, n)))
    ga3, gb3 = np.zeros_like(a), np.zeros_like(b_up)
    oracle.matmat_batch3_backward(dtype, bsz, m, k, n, a, ls, ga3, b_up, row_major_strides((bsz, k, n)), gb3, go)
    assert np.array_equal(out3, out) and np.array_equal(ga3, ga)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_batched_equal_loops_of_2d(oracle, dtype):
    """Batch3 / Batch4 == loop of 2-D products, head-interleaved strides included (mod.rs:476-527)."""
    g = rng(23)
    B, S, m, k, n = 3, 5, 3, 2, 4
    # lhs stored (B, m, S, k) and viewed (B, S, m, k): batch-2 stride smaller than the row stride
    lhs = _rand_storage(g, B * m * S * k, dtype, oracle)
    lshape, ls = permute((B, m, S, k), row_major_strides((B, m, S, k)), (0, 2, 1, 3))
    # rhs stored (B, n, S, k) viewed (B, S, k, n): a transposed K matrix per head
    rhs = _rand_storage(g, B * n * S * k, dtype, oracle)
    rshape, rs = permute((B, n, S, k), row_major_strides((B, n, S, k)), (0, 2, 3, 1))
    go = _rand_storage(g, B * S * m * n, dtype, oracle)
    out = oracle.matmat_batch4_forward(dtype, B, S, m, k, n, lhs, ls, rhs, rs)
    gl, gr = np.zeros_like(lhs), np.zeros_like(rhs)
    oracle.matmat_batch4_backward(dtype, B, S, m, k, n, lhs, ls, gl, rhs, rs, gr, go)
    L = logical(oracle.to_f64(lhs, dtype), lshape, ls)
    R = logical(oracle.to_f64(rhs, dtype), rshape, rs)
    G = oracle.to_f64(go, dtype).reshape(B, S, m, n)
    assert_within(dtype, k, oracle.to_f64(out, dtype).reshape(B, S, m, n), L @ R, L, R, extra=2.0 ** -10 * 8)
    assert_within(dtype, n, logical(oracle.to_f64(gl, dtype), lshape, ls), G @ R.transpose(0, 1, 3, 2), G, R, extra=2.0 ** -10 * 8)
    assert_within(dtype, m, logical(oracle.to_f64(gr, dtype), rshape, rs), L.transpose(0, 1, 3, 2) @ G, L, G, extra=2.0 ** -10 * 8)
    # Batch3 over the flattened (B*S) batch of contiguous copies gives the same bits
    lc = oracle.to_storage(L.reshape(-1), dtype)
    rc = oracle.to_storage(R.reshape(-1), dtype)
    out3 = oracle.matmat_batch3_forward(dtype, B * S, m, k, n, lc, row_major_strides((B * S, m, k)), rc, row_major_strides((B * S, k, n)))
    assert np.array_equal(out3, out)


def test_grad_buffers_accumulate(oracle):
    """Backward adds into whatever the gradient buffers already hold (cpu_kernel.rs:268,278)."""
    g = rng(24)
    m, k, n = 3, 4, 5
    a, b, go = (g.integers(-2, 3, s).astype(np.float32) for s in (m * k, k * n, m * n))
    ga, gb = np.ones(m * k, np.float32), np.full(k * n, 2.0, np.float32)
    oracle.matmat_backward("f32", m, k, n, a, [k, 1], ga, b, [n, 1], gb, go)
    A, Bm, G = a.reshape(m, k), b.reshape(k, n), go.reshape(m, n)
    assert np.array_equal(ga.reshape(m, k), 1 + G @ Bm.T)
    assert np.array_equal(gb.reshape(k, n), 2 + A.T @ G)
