"""GPU parity on the five benchmark configurations, at their full sizes.

Where the whole result is too large for the CPU oracle to finish in seconds, the oracle is run on a
seeded sample of output rows / batch slices (same inputs, same code path), plus size-independent
properties: linearity (accumulating twice doubles), agreement between the three operand layouts of
the same product, and column-sum checksums in float64."""
import numpy as np
import pytest

import oracle
from helpers import assert_within, logical, rng, row_major_strides, tolerance
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

ULP = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}


def host(dev, view):
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


# ---- config 1: Linear<512,256> forward + backward, f32 -----------------------------------------
def test_config1_linear_512_256_f32():
    """x [64,512] ~ N(0,1); W [256,512], b [256] ~ U(+-1/sqrt(512)); loss = sum(y) so dy = 1.
    y, dW, db, dx against the oracle's MatMat drivers (linear.rs:65-89, bias1d.rs:62-78)."""
    dev, g = device(), rng(1001)
    dtype, (rows, i, o) = "f32", (64, 512, 256)
    bound = 1.0 / np.sqrt(i)
    x = upload(dev, g.standard_normal((rows, i)), dtype)
    w = upload(dev, g.uniform(-bound, bound, (o, i)), dtype)
    b = upload(dev, g.uniform(-bound, bound, (o,)), dtype)
    wt = w.permute(1, 0)
    announce("config1 forward")
    y = dev.linear_forward(x, w, b)
    x_h, w_h, b_h = dev.to_host(x), dev.to_host(w), dev.to_host(b)
    want = oracle.matmat_forward(dtype, rows, i, o, x_h, x.strides, w_h, wt.strides).reshape(rows, o) + b_h
    X, W = host(dev, x), host(dev, wt)
    assert_within(dtype, i, host(dev, y), want.astype(np.float64), X, W, extra=ULP[dtype] * 8, what="y")
    announce("config1 backward")
    dy = upload(dev, np.ones((rows, o)), dtype)
    gx, gw = dev.zeros_like_storage(x), dev.zeros_like_storage(wt)
    dev.backward(x, gx, wt, gw, dy)
    wgx, wgw = np.zeros_like(x_h), np.zeros_like(w_h)
    oracle.matmat_backward(dtype, rows, i, o, x_h, x.strides, wgx, w_h, wt.strides, wgw, dev.to_host(dy))
    ones = np.ones((rows, o))
    assert_within(dtype, o, oracle.to_f64(dev.to_host(gx), dtype), wgx.astype(np.float64), ones, W, what="dx")
    assert_within(dtype, rows, oracle.to_f64(dev.to_host(gw), dtype), wgw.astype(np.float64), X, ones, what="dW")
    # db = column sum of dy = 64 for every output feature (utilities/cpu_kernels.rs:188-200)
    assert np.array_equal(host(dev, dy).sum(axis=0), np.full(o, float(rows)))


# ---- config 2: 4096^3, f32 and f16, A.B / A^T.B / A.B^T ------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_config2_square_4096(dtype):
    dev, g = device(), rng(2002)
    n = 4096
    a = upload(dev, g.uniform(-1, 1, (n, n)).astype(np.float32), dtype)
    b = upload(dev, g.uniform(-1, 1, (n, n)).astype(np.float32), dtype)
    a_h, b_h = dev.to_host(a), dev.to_host(b)
    A, B = oracle.to_f64(a_h, dtype).reshape(n, n), oracle.to_f64(b_h, dtype).reshape(n, n)
    rows = np.sort(rng(7).choice(n, 48, replace=False))
    results = {}
    for name, lhs, rhs, La, Lb in (("A.B", a, b, A, B), ("At.B", a.permute(1, 0), b, A.T, B), ("A.Bt", a, b.permute(1, 0), A, B.T)):
        announce("config2", dtype, name)
        c = dev.forward(lhs, rhs)
        C = oracle.to_f64(dev.to_host(c), dtype).reshape(n, n)
        results[name] = C
        # sampled rows through the oracle (same storage, same strides, row offset applied to the lhs view)
        for r in rows[:16]:
            want = oracle.gemm(dtype, 1, n, n, False, a_h, (lhs.strides[0], lhs.strides[1]), b_h, rhs.strides,
                               np.zeros(n, oracle.NP_DTYPES[dtype]), (n, 1), a_off=int(r) * lhs.strides[0])
            assert_within(dtype, n, C[r], oracle.to_f64(want, dtype), La, Lb, extra=2 * ULP[dtype] * 64, what=f"{name} row {r} vs oracle")
        want64 = La[rows] @ Lb
        assert_within(dtype, n, C[rows], want64, La, Lb, extra=ULP[dtype] * np.abs(want64).max(), what=f"{name} rows vs f64")
        # checksum of checksums over the whole result: 1^T C 1 == (1^T A)(B 1)
        total, want_total = C.sum(), float(La.sum(axis=0) @ Lb.sum(axis=1))
        assert abs(total - want_total) <= tolerance(dtype, n, 1.0, 1.0) * n * 8, (total, want_total)
        col = C.sum(axis=0)
        want_col = La.sum(axis=0) @ Lb
        assert np.max(np.abs(col - want_col)) <= tolerance(dtype, n, 1.0, 1.0) * np.sqrt(n) * 8
    # linearity: accumulating the same product into C doubles it (beta = 1 path at full size)
    announce("config2", dtype, "accumulate")
    c = dev.forward(a, b)
    before = oracle.to_f64(dev.to_host(c), dtype)
    dev.gemm(dev.gemm_desc(dtype, n, n, n, a.ptr, a.strides, b.ptr, b.strides, c.ptr, (n, 1), accumulate=True))
    after = oracle.to_f64(dev.to_host(c), dtype)
    assert np.max(np.abs(after - 2 * before)) <= 2 * ULP[dtype] * np.abs(after).max() + 1e-30


# ---- config 3: [32,512,1024] x [1024,1024] f16, forward + both backward GEMMs ---------------------
def test_config3_batched_broadcast_rhs_f16():
    dev, g = device(), rng(3003)
    dtype, (bsz, m, k, n) = "f16", (32, 512, 1024, 1024)
    lhs = upload(dev, g.standard_normal((bsz, m, k)).astype(np.float32), dtype)
    rhs = upload(dev, (g.standard_normal((k, n)) / 32.0).astype(np.float32), dtype)
    go = upload(dev, g.standard_normal((bsz, m, n)).astype(np.float32), dtype)
    announce("config3 forward")
    out = dev.forward(lhs, rhs)
    announce("config3 backward")
    gl, gr = dev.zeros_like_storage(lhs), dev.zeros_like_storage(rhs)
    dev.backward(lhs, gl, rhs, gr, go)
    l_h, r_h, go_h = dev.to_host(lhs), dev.to_host(rhs), dev.to_host(go)
    L, R, G = (oracle.to_f64(x, dtype) for x in (l_h, r_h, go_h))
    L, R, G = L.reshape(bsz, m, k), R.reshape(k, n), G.reshape(bsz, m, n)
    # forward and dX: oracle on 3 sampled batch slices (the Br driver with batch = 1 on a slice)
    for i in (0, 13, 31):
        sl, sg = l_h[i * m * k:(i + 1) * m * k], go_h[i * m * n:(i + 1) * m * n]
        want = oracle.matmat_forward(dtype, m, k, n, sl, (k, 1), r_h, (n, 1))
        got = oracle.to_f64(dev.to_host(out), dtype).reshape(bsz, m, n)[i]
        assert_within(dtype, k, got, oracle.to_f64(want, dtype).reshape(m, n), L[i], R, extra=2 * ULP[dtype] * 8, what=f"out[{i}]")
        wgl, wgr = np.zeros(m * k, np.float16), np.zeros(k * n, np.float16)
        oracle.matmat_backward(dtype, m, k, n, sl, (k, 1), wgl, r_h, (n, 1), wgr, sg)
        got = oracle.to_f64(dev.to_host(gl), dtype).reshape(bsz, m, k)[i]
        assert_within(dtype, n, got, oracle.to_f64(wgl, dtype).reshape(m, k), G[i], R, extra=2 * ULP[dtype] * 256, what=f"dX[{i}]")
    # dW: the full oracle driver re-rounds the shared accumulator to f16 after each of the 32 slices
    # (cpu_kernel.rs:339-348); the GPU rounds once.  Compare both against float64 on sampled columns.
    announce("config3 dW oracle")
    cols = np.sort(rng(9).choice(n, 32, replace=False))
    want64 = np.einsum("bmk,bmn->kn", L, G[:, :, cols])
    got = oracle.to_f64(dev.to_host(gr), dtype).reshape(k, n)[:, cols]
    assert_within(dtype, bsz * m, got, want64, L, G, extra=ULP[dtype] * np.abs(want64).max(), what="dW vs f64")
    wgl, wgr = np.zeros_like(l_h), np.zeros_like(r_h)
    oracle.matmat_br_backward(dtype, bsz, m, k, n, l_h, (m * k, k, 1), wgl, r_h, (n, 1), wgr, go_h)
    full = oracle.to_f64(dev.to_host(gr), dtype).reshape(k, n)
    assert_within(dtype, bsz * m, full, oracle.to_f64(wgr, dtype).reshape(k, n), L, G,
                  extra=bsz * ULP[dtype] * np.abs(want64).max(), what="dW vs oracle driver")
    assert_within(dtype, n, oracle.to_f64(dev.to_host(gl), dtype), oracle.to_f64(wgl, dtype), G, R, extra=2 * ULP[dtype] * 256, what="dX full")


# ---- config 4: attention-shaped Rank4, f16 ---------------------------------------------------------
def test_config4_attention_rank4_f16():
    """Q,K,V [8,16,1024,64]; scores = Q.K^T / 8 -> softmax (host, float64, CPU-equivalent glue:
    softmax.rs:70-83) -> out = P.V; backward through both matmuls with dO ~ N(0,1)."""
    dev, g = device(), rng(4004)
    dtype, (B, H, S, D) = "f16", (8, 16, 1024, 64)
    q, k, v, d_o = (upload(dev, g.standard_normal((B, H, S, D)).astype(np.float32), dtype) for _ in range(4))
    kt = k.permute(0, 1, 3, 2)
    announce("config4 scores")
    scores = dev.forward(q, kt)
    s_h = dev.to_host(scores)
    q_h, k_h, v_h, do_h = (dev.to_host(t) for t in (q, k, v, d_o))
    sample = [(0, 0), (3, 7), (7, 15)]
    sl = lambda arr, b, h, per: arr[(b * H + h) * per:(b * H + h + 1) * per]
    Q, K = oracle.to_f64(q_h, dtype).reshape(B, H, S, D), oracle.to_f64(k_h, dtype).reshape(B, H, S, D)
    for b, h in sample:
        want = oracle.matmat_forward(dtype, S, D, S, sl(q_h, b, h, S * D), (D, 1), sl(k_h, b, h, S * D), (1, D))
        assert_within(dtype, D, oracle.to_f64(sl(s_h, b, h, S * S), dtype), oracle.to_f64(want, dtype), Q[b, h], K[b, h],
                      extra=2 * ULP[dtype] * 64, what=f"scores[{b},{h}]")
    # glue on the host in float64, stored back as f16 (the reference's softmax is elementwise + reductions)
    sc = oracle.to_f64(s_h, dtype).reshape(B, H, S, S) / 8.0
    sc -= sc.max(axis=-1, keepdims=True)
    p64 = np.exp(sc)
    p64 /= p64.sum(axis=-1, keepdims=True)
    p = upload(dev, p64.astype(np.float32), dtype)
    del sc, p64
    announce("config4 out")
    out = dev.forward(p, v)
    p_h, o_h = dev.to_host(p), dev.to_host(out)
    P, V = oracle.to_f64(p_h, dtype).reshape(B, H, S, S), oracle.to_f64(v_h, dtype).reshape(B, H, S, D)
    for b, h in sample:
        want = oracle.matmat_forward(dtype, S, S, D, sl(p_h, b, h, S * S), (S, 1), sl(v_h, b, h, S * D), (D, 1))
        assert_within(dtype, S, oracle.to_f64(sl(o_h, b, h, S * D), dtype), oracle.to_f64(want, dtype), P[b, h], V[b, h],
                      extra=2 * ULP[dtype] * 4, what=f"out[{b},{h}]")
    announce("config4 backward of P.V")
    gp, gv = dev.zeros_like_storage(p), dev.zeros_like_storage(v)
    dev.backward(p, gp, v, gv, d_o)
    announce("config4 backward of Q.K^T")
    gq, gk = dev.zeros_like_storage(q), dev.zeros_like_storage(kt)
    dev.backward(q, gq, kt, gk, gp)   # dS := dP as a stand-in for the softmax backward glue
    gp_h, gv_h, gq_h, gk_h = (dev.to_host(t) for t in (gp, gv, gq, gk))
    DO = oracle.to_f64(do_h, dtype).reshape(B, H, S, D)
    DS = oracle.to_f64(gp_h, dtype).reshape(B, H, S, S)
    for b, h in sample:
        wgp, wgv = np.zeros(S * S, np.float16), np.zeros(S * D, np.float16)
        oracle.matmat_backward(dtype, S, S, D, sl(p_h, b, h, S * S), (S, 1), wgp, sl(v_h, b, h, S * D), (D, 1), wgv, sl(do_h, b, h, S * D))
        assert_within(dtype, D, oracle.to_f64(sl(gp_h, b, h, S * S), dtype), oracle.to_f64(wgp, dtype), DO[b, h], V[b, h], extra=2 * ULP[dtype] * 64, what="dP")
        assert_within(dtype, S, oracle.to_f64(sl(gv_h, b, h, S * D), dtype), oracle.to_f64(wgv, dtype), P[b, h], DO[b, h], extra=2 * ULP[dtype] * 8, what="dV")
        wgq, wgk = np.zeros(S * D, np.float16), np.zeros(S * D, np.float16)
        oracle.matmat_backward(dtype, S, D, S, sl(q_h, b, h, S * D), (D, 1), wgq, sl(k_h, b, h, S * D), (1, D), wgk, sl(gp_h, b, h, S * S))
        assert_within(dtype, S, oracle.to_f64(sl(gq_h, b, h, S * D), dtype), oracle.to_f64(wgq, dtype), DS[b, h], K[b, h], extra=2 * ULP[dtype] * 2048, what="dQ")
        assert_within(dtype, S, oracle.to_f64(sl(gk_h, b, h, S * D), dtype), oracle.to_f64(wgk, dtype), Q[b, h], DS[b, h], extra=2 * ULP[dtype] * 2048, what="dK")
