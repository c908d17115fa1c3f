"""GPU parity on the five benchmark configurations, at their full sizes.

Where the whole result is too large for the CPU oracle to finish in seconds, the oracle is run on a
seeded sample of output rows / batch slices (same inputs, same code path), plus size-independent
properties: linearity (accumulating twice doubles), agreement between the three operand layouts of
the same product, and column-sum checksums in float64."""
import numpy as np
import pytest

import oracle
from oracle import nn_ops
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
    gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros_like_storage(b)
    dev.linear_backward(x, gx, w, gw, gb, dy)   # dx, dW and db all come from the device
    wgx, wgw = np.zeros_like(x_h), np.zeros_like(w_h)
    oracle.matmat_backward(dtype, rows, i, o, x_h, x.strides, wgx, w_h, wt.strides, wgw, dev.to_host(dy))
    ones = np.ones((rows, o))
    assert_within(dtype, o, oracle.to_f64(dev.to_host(gx), dtype), wgx.astype(np.float64), ones, W, what="dx")
    assert_within(dtype, rows, oracle.to_f64(dev.to_host(gw), dtype), wgw.astype(np.float64), X, ones, what="dW")
    # db: the broadcast add's backward sums dy down the rows (utilities/cpu_kernels.rs:188-200); with dy = 1 every
    # partial sum is a small integer, so the reference's row-after-row f32 order and any other order agree exactly: 64
    want_db = nn_ops.bias_backward(dev.to_host(dy).reshape(rows, o), np.zeros(o), dtype, faithful=True)
    got_db = oracle.to_f64(dev.to_host(gb), dtype)
    assert np.array_equal(want_db, np.full(o, float(rows)))
    assert np.array_equal(got_db, want_db), np.max(np.abs(got_db - want_db))
    # a second backward with a random dy accumulates into all three (beta = 1 everywhere, db included)
    announce("config1 backward, random dy, accumulating")
    dy2 = upload(dev, g.standard_normal((rows, o)), dtype)
    dev.linear_backward(x, gx, w, gw, gb, dy2)
    oracle.matmat_backward(dtype, rows, i, o, x_h, x.strides, wgx, w_h, wt.strides, wgw, dev.to_host(dy2))
    DY2 = host(dev, dy2)
    assert_within(dtype, o, oracle.to_f64(dev.to_host(gx), dtype), wgx.astype(np.float64), DY2, W, extra=ULP[dtype] * 64, what="dx (2)")
    assert_within(dtype, rows, oracle.to_f64(dev.to_host(gw), dtype), wgw.astype(np.float64), X, DY2, extra=ULP[dtype] * 256, what="dW (2)")
    want_db = nn_ops.bias_backward(dev.to_host(dy2).reshape(rows, o), want_db, dtype, faithful=True)
    assert_within(dtype, rows, oracle.to_f64(dev.to_host(gb), dtype), want_db, DY2, np.ones(1), extra=ULP[dtype] * 128, what="db (2)")


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
    """Q,K,V [8,16,1024,64]; scores = Q.K^T, P = softmax(scores / 8) (the scale folded into the device softmax:
    multi_head_attention.rs:129-134 over softmax.rs:70-83), out = P.V; backward through both matmuls AND the softmax
    with dO ~ N(0,1), everything on the device.  Each GEMM is compared with the oracle's MatMat driver run on that
    GEMM's own device-produced operands for sampled (batch, head) slices -- the Batch4 driver is a loop of exactly
    these calls (cpu_kernel.rs:432-447,461-484) --, each softmax step with the numpy restatement."""
    dev, g = device(), rng(4004)
    dtype, (B, H, S, D) = "f16", (8, 16, 1024, 64)
    scale = 0.125
    q, k, v, d_o = (upload(dev, g.standard_normal((B, H, S, D)).astype(np.float32), dtype) for _ in range(4))
    kt = k.permute(0, 1, 3, 2)
    announce("config4 forward: scores, softmax, P.V")
    scores = dev.forward(q, kt)
    p = dev.softmax_forward(scores, scale)
    out = dev.forward(p, v)
    announce("config4 backward: P.V, softmax, Q.K^T")
    gp, gv = dev.zeros_like_storage(p), dev.zeros_like_storage(v)
    dev.backward(p, gp, v, gv, d_o)
    gs = dev.zeros_like_storage(scores)
    dev.softmax_backward(p, gs, gp, scale)
    gq, gk = dev.zeros_like_storage(q), dev.zeros_like_storage(kt)
    dev.backward(q, gq, kt, gk, gs)
    dev.synchronize()
    announce("config4 checks")
    q_h, k_h, v_h, do_h, s_h, p_h, o_h, gp_h, gv_h, gs_h, gq_h, gk_h = (
        dev.to_host(t) for t in (q, k, v, d_o, scores, p, out, gp, gv, gs, gq, gk))
    sample = [(0, 0), (3, 7), (7, 15)]
    sl = lambda arr, b, h, per: arr[(b * H + h) * per:(b * H + h + 1) * per]
    f = lambda arr, b, h, r, c: oracle.to_f64(sl(arr, b, h, r * c), dtype).reshape(r, c)
    e = ULP[dtype]
    for b, h in sample:
        Q, K, V, DO = (f(t, b, h, S, D) for t in (q_h, k_h, v_h, do_h))
        SC, P, GP, GS = (f(t, b, h, S, S) for t in (s_h, p_h, gp_h, gs_h))
        want = oracle.matmat_forward(dtype, S, D, S, sl(q_h, b, h, S * D), (D, 1), sl(k_h, b, h, S * D), (1, D))
        assert_within(dtype, D, SC, oracle.to_f64(want, dtype).reshape(S, S), Q, K, extra=2 * e * 64, what=f"scores[{b},{h}]")
        # softmax of the device's own scores: the exact formula rounded once, +-1 ulp of the largest probability
        once = nn_ops.softmax_forward(SC * scale, dtype, faithful=False)
        np.testing.assert_allclose(P, once, rtol=0, atol=2 * e * float(once.max()) + 1e-7)
        want = oracle.matmat_forward(dtype, S, S, D, sl(p_h, b, h, S * S), (S, 1), sl(v_h, b, h, S * D), (D, 1))
        assert_within(dtype, S, f(o_h, b, h, S, D), oracle.to_f64(want, dtype).reshape(S, D), P, V, extra=2 * e * 4, what=f"out[{b},{h}]")
        wgp, wgv = np.zeros(S * S, np.float16), np.zeros(S * D, np.float16)
        oracle.matmat_backward(dtype, S, S, D, sl(p_h, b, h, S * S), (S, 1), wgp, sl(v_h, b, h, S * D), (D, 1), wgv, sl(do_h, b, h, S * D))
        assert_within(dtype, D, GP, oracle.to_f64(wgp, dtype).reshape(S, S), DO, V, extra=2 * e * 64, what="dP")
        assert_within(dtype, S, f(gv_h, b, h, S, D), oracle.to_f64(wgv, dtype).reshape(S, D), P, DO, extra=2 * e * 8, what="dV")
        # softmax backward from the saved output, on the device's own dP: scale * p * (g - sum g p)
        want = scale * P * (GP - (GP * P).sum(axis=-1, keepdims=True))
        np.testing.assert_allclose(GS, want, rtol=0, atol=2 * e * float(np.abs(want).max()) + 1e-6)
        wgq, wgk = np.zeros(S * D, np.float16), np.zeros(S * D, np.float16)
        oracle.matmat_backward(dtype, S, D, S, sl(q_h, b, h, S * D), (D, 1), wgq, sl(k_h, b, h, S * D), (1, D), wgk, sl(gs_h, b, h, S * S))
        assert_within(dtype, S, f(gq_h, b, h, S, D), oracle.to_f64(wgq, dtype).reshape(S, D), GS, K, extra=2 * e * 16, what="dQ")
        assert_within(dtype, S, f(gk_h, b, h, S, D), oracle.to_f64(wgk, dtype).reshape(S, D), Q, GS, extra=2 * e * 16, what="dK")
    # the softmax backward's row identity over the WHOLE tensor: every row of dS sums to 0 (up to rounding of 1024 terms)
    GS_all = oracle.to_f64(gs_h, dtype).reshape(-1, S)
    assert float(np.max(np.abs(GS_all.sum(axis=-1)))) <= 1024 * e * float(np.max(np.abs(GS_all))) + 1e-6
