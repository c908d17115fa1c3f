"""GPU parity at the kernel-trait level: the `Rocm` device's forward / backward for the four
matmul kernel traits against (a) the literals the reference's own tests assert, (b) the CPU oracle on
seeded inputs, (c) the identities the reference's tests assert (matmul/mod.rs:413-527).
These tests read like the reference's: build tensors, call matmul forward, push a loss gradient
through backward, compare."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import assert_within, logical, rng, row_major_strides
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
MATMUL = json.load(open(os.path.join(GOLD, "matmul_literals.json")))
LINEAR = json.load(open(os.path.join(GOLD, "linear_literals.json")))


def loss_grad(kind, out):
    out = out.astype(np.float64)
    return {"exp_mean": np.exp(out) / out.size, "exp_sum": np.exp(out), "square_mean": 2.0 * out / out.size}[kind]


def host(dev, view):
    """Logical float64 contents of a device view."""
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


# ------------------------------------------------------------ golden literals --
@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("case", MATMUL["cases"], ids=lambda c: c["name"])
def test_matmul_literals(case, dtype):
    dev = device()
    announce("literal", case["name"], dtype)
    a, b = upload(dev, case["a"], dtype), upload(dev, case["b"], dtype)
    lhs = a.permute(1, 0) if case.get("permute_a") else a
    rhs = b.permute(1, 0) if case.get("permute_b") else b
    tol = case.get("tol", 1e-6)
    r = dev.forward(lhs, rhs)
    np.testing.assert_allclose(host(dev, r), case["out"], rtol=0, atol=tol)
    g = upload(dev, loss_grad(case["loss"], host(dev, r)), dtype)
    ga, gb = dev.zeros_like_storage(lhs), dev.zeros_like_storage(rhs)
    dev.backward(lhs, ga, rhs, gb, g)
    # gradients live in the operand's physical layout == the literal's own shape
    np.testing.assert_allclose(oracle.to_f64(dev.to_host(ga), dtype).reshape(np.shape(case["grad_a"])), case["grad_a"], rtol=0, atol=tol)
    np.testing.assert_allclose(oracle.to_f64(dev.to_host(gb), dtype).reshape(np.shape(case["grad_b"])), case["grad_b"], rtol=0, atol=tol)


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("case", LINEAR["cases"], ids=lambda c: c["name"])
def test_linear_literals(case, dtype, fused):
    """Linear = x.matmul(weight.permute()) + bias (linear.rs:82-89); `fused` uses the bias epilogue."""
    dev = device()
    announce("linear literal", case["name"], dtype, "fused" if fused else "unfused")
    w, bias = upload(dev, LINEAR["weight"], dtype), upload(dev, LINEAR["bias"], dtype)
    x = upload(dev, case["x"], dtype)
    wt = w.permute(1, 0)
    if fused:
        y = host(dev, dev.linear_forward(x, w, bias))
    else:
        y = host(dev, dev.forward(x, wt)) + np.asarray(LINEAR["bias"])
    np.testing.assert_allclose(y, case["y"], rtol=0, atol=1e-6)
    gy = loss_grad("square_mean", y)
    if fused:   # the whole backward through the Linear entry point, grad_bias included (f64 too: the reference's CI runs in f64)
        gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros_like_storage(bias)
        dev.linear_backward(x, gx, w, gw, gb, upload(dev, gy, dtype))
    else:       # MatMat backward on the permuted view + Bias1D's backward
        gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(wt), dev.zeros_like_storage(bias)
        gyv = upload(dev, gy, dtype)
        dev.backward(x, gx, wt, gw, gyv)
        dev.bias_backward(gyv, gb)
    np.testing.assert_allclose(oracle.to_f64(dev.to_host(gw), dtype).reshape(2, 5), case["grad_weight"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(oracle.to_f64(dev.to_host(gb), dtype), case["grad_bias"], rtol=0, atol=1e-6)


# ------------------------------------------------------------------ identities --
def sample(dev, g, shape, dtype, scale=1.0):
    return upload(dev, g.standard_normal(shape) * scale, dtype)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("dims", [(4, 3, 2), (136, 72, 200)])
def test_matmul_transpose(dtype, dims):
    """(A.B)^T == B^T.A^T including gradients (mod.rs:413-426); exact, the summation order is the same."""
    dev, g = device(), rng(61)
    m, k, n = dims
    announce("transpose identity", dtype, dims)
    a, b, go = sample(dev, g, (m, k), dtype), sample(dev, g, (k, n), dtype), sample(dev, g, (m, n), dtype)
    c1 = dev.forward(a, b)
    ga1, gb1 = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
    dev.backward(a, ga1, b, gb1, go)
    c2 = dev.forward(b.permute(1, 0), a.permute(1, 0))
    go_t = upload(dev, host(dev, go).T, dtype)
    ga2, gb2 = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
    dev.backward(b.permute(1, 0), gb2.permute(1, 0), a.permute(1, 0), ga2.permute(1, 0), go_t)
    tol = {"f32": 1e-5, "f16": 2e-3}[dtype] * np.sqrt(max(m, k, n)) * 16
    np.testing.assert_allclose(host(dev, c1), host(dev, c2).T, rtol=0, atol=tol)
    np.testing.assert_allclose(dev.to_host(ga1).astype(np.float64), dev.to_host(ga2).astype(np.float64), rtol=0, atol=tol)
    np.testing.assert_allclose(dev.to_host(gb1).astype(np.float64), dev.to_host(gb2).astype(np.float64), rtol=0, atol=tol)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("dims", [(5, 4, 3, 2), (6, 40, 64, 72), (3, 200, 136, 264), (8, 512, 16, 1024), (4, 1024, 24, 1024)])
def test_matmul_broadcast(dtype, dims):
    """Br == per-slice 2-D products, grad_rhs == sum over slices (mod.rs:429-457); and Br == Batch3 with
    the rhs stacked, EXACTLY, for out and grad_lhs (mod.rs:460-473)."""
    dev, g = device(), rng(62)
    bsz, m, k, n = dims
    announce("broadcast identity", dtype, dims)
    a, b, go = sample(dev, g, (bsz, m, k), dtype), sample(dev, g, (k, n), dtype), sample(dev, g, (bsz, m, n), dtype)
    r = dev.forward(a, b)
    ga, gb = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
    dev.backward(a, ga, b, gb, go)
    A, B, G = host(dev, a), host(dev, b), host(dev, go)
    ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}[dtype]
    assert_within(dtype, k, host(dev, r), A @ B, A, B, extra=ulp * np.abs(A @ B).max(), what="out")
    assert_within(dtype, n, host(dev, ga), G @ B.T, G, B, extra=ulp * np.abs(G @ B.T).max(), what="grad_lhs")
    want_gb = np.einsum("bmk,bmn->kn", A, G)
    assert_within(dtype, bsz * m, host(dev, gb), want_gb, A, G, extra=ulp * np.abs(want_gb).max(), what="grad_rhs")

    b_up = upload(dev, np.broadcast_to(B, (bsz, k, n)), dtype)
    r3 = dev.forward(a, b_up)
    ga3, gb3 = dev.zeros_like_storage(a), dev.zeros_like_storage(b_up)
    dev.backward(a, ga3, b_up, gb3, go)
    assert np.array_equal(dev.to_host(r3), dev.to_host(r)), "Br and Batch3 forward differ bitwise"
    assert np.array_equal(dev.to_host(ga3), dev.to_host(ga)), "Br and Batch3 grad_lhs differ bitwise"
    assert_within(dtype, bsz * m, host(dev, gb3).sum(axis=0), want_gb, A, G, extra=bsz * ulp * np.abs(want_gb).max())


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("dims", [(2, 4, 4096, 4096), (2, 1, 4096, 4096), (16, 1, 16384, 4096), (3, 2, 8192, 1024), (2, 5, 64, 16384)])
def test_matmul_broadcast_few_rows_exact(dtype, dims):
    """The reference's exact identity Br == Batch3 with the rhs stacked (mod.rs:460-473) where the broadcast form folds to
    a FEW rows against a large matrix: a Linear layer on a handful of tokens.  Those shapes would otherwise go to the
    vector-product kernels, which cut the contraction into grid slices; the broadcast entry points ask for the tiled
    kernels' contraction order, so forward and grad_lhs must equal the batched product bit for bit whatever the row
    count.  The stacked rhs is built on the device (up to 4 GiB in f32)."""
    dev, g = device(), rng(66)
    bsz, m, k, n = dims
    announce("broadcast identity, few rows", dtype, dims)
    from dfdx_amd.rocm import View
    a, b, go = sample(dev, g, (bsz, m, k), dtype), sample(dev, g, (k, n), dtype, scale=k ** -0.5), sample(dev, g, (bsz, m, n), dtype)
    r = dev.forward(a, b)
    ga, gb = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
    dev.backward(a, ga, b, gb, go)
    A, B, G = host(dev, a), host(dev, b), host(dev, go)
    ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}[dtype]
    assert_within(dtype, k, host(dev, r), A @ B, A, B, extra=ulp * np.abs(A @ B).max(), what="out")
    assert_within(dtype, n, host(dev, ga), G @ B.T, G, B, extra=ulp * np.abs(G @ B.T).max(), what="grad_lhs")
    want_gb = np.einsum("bmk,bmn->kn", A, G)
    assert_within(dtype, bsz * m, host(dev, gb), want_gb, A, G, extra=ulp * np.abs(want_gb).max(), what="grad_rhs")
    del A, G, want_gb

    b_up = View(b.storage.repeat(bsz), dtype, (bsz, k, n), row_major_strides((bsz, k, n)))
    r3 = dev.forward(a, b_up)
    ga3, gb3 = dev.zeros_like_storage(a), dev.zeros_like_storage(b_up)
    dev.backward(a, ga3, b_up, gb3, go)
    assert np.array_equal(dev.to_host(r3), dev.to_host(r)), "Br and Batch3 forward differ bitwise"
    assert np.array_equal(dev.to_host(ga3), dev.to_host(ga)), "Br and Batch3 grad_lhs differ bitwise"


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_matmul_batched_3d_and_4d(dtype):
    """Batched == loop of 2-D products incl. gradients (mod.rs:476-527), against the oracle's drivers."""
    dev, g = device(), rng(63)
    for shape_l, shape_r in (((5, 3, 2), (5, 2, 4)), ((7, 5, 3, 2), (7, 5, 2, 4)), ((2, 3, 72, 64), (2, 3, 64, 40))):
        announce("batched", dtype, shape_l, shape_r)
        a, b = sample(dev, g, shape_l, dtype), sample(dev, g, shape_r, dtype)
        go = sample(dev, g, shape_l[:-1] + shape_r[-1:], dtype)
        c = dev.forward(a, b)
        ga, gb = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
        dev.backward(a, ga, b, gb, go)
        a_h, b_h, go_h = dev.to_host(a), dev.to_host(b), dev.to_host(go)
        dims = shape_l + shape_r[-1:]
        fwd = oracle.matmat_batch3_forward if len(shape_l) == 3 else oracle.matmat_batch4_forward
        bwd = oracle.matmat_batch3_backward if len(shape_l) == 3 else oracle.matmat_batch4_backward
        want = fwd(dtype, *dims, a_h, row_major_strides(shape_l), b_h, row_major_strides(shape_r))
        wga, wgb = np.zeros_like(a_h), np.zeros_like(b_h)
        bwd(dtype, *dims, a_h, row_major_strides(shape_l), wga, b_h, row_major_strides(shape_r), wgb, go_h)
        A, B, G = host(dev, a), host(dev, b), host(dev, go)
        k, m, n = shape_l[-1], shape_l[-2], shape_r[-1]
        ulp = {"f32": 2.0 ** -23, "f16": 2.0 ** -10}[dtype]
        assert_within(dtype, k, oracle.to_f64(dev.to_host(c), dtype), oracle.to_f64(want, dtype), A, B, extra=ulp * 8)
        assert_within(dtype, n, oracle.to_f64(dev.to_host(ga), dtype), oracle.to_f64(wga, dtype), G, B, extra=ulp * 8)
        assert_within(dtype, m, oracle.to_f64(dev.to_host(gb), dtype), oracle.to_f64(wgb, dtype), A, G, extra=ulp * 8)


def test_attention_shaped_permuted_views():
    """Head-interleaved Q/K/V views as MultiHeadAttention builds them (multi_head_attention.rs:123-141):
    storage (B, S, H, D); Q, V viewed (B, H, S, D), K viewed (B, H, D, S); forward and backward vs the oracle."""
    dev, g = device(), rng(64)
    dtype, (B, S, H, D) = "f16", (2, 64, 4, 32)
    announce("attention views", dtype, (B, S, H, D))
    q, kk, v = (sample(dev, g, (B, S, H, D), dtype) for _ in range(3))
    qv, kv, vv = q.permute(0, 2, 1, 3), kk.permute(0, 2, 3, 1), v.permute(0, 2, 1, 3)
    scores = dev.forward(qv, kv)               # (B, H, S, S)
    q_h, k_h, v_h = dev.to_host(q), dev.to_host(kk), dev.to_host(v)
    want_s = oracle.matmat_batch4_forward(dtype, B, H, S, D, S, q_h, qv.strides, k_h, kv.strides)
    Q, K = host(dev, qv), host(dev, kv)
    assert_within(dtype, D, oracle.to_f64(dev.to_host(scores), dtype), oracle.to_f64(want_s, dtype), Q, K, extra=2.0 ** -10 * 64)
    p = upload(dev, g.uniform(0, 1, (B, H, S, S)) / S, dtype)   # stand-in for softmax output
    out = dev.forward(p, vv)                   # (B, H, S, D)
    p_h = dev.to_host(p)
    want_o = oracle.matmat_batch4_forward(dtype, B, H, S, S, D, p_h, p.strides, v_h, vv.strides)
    P, V = host(dev, p), host(dev, vv)
    assert_within(dtype, S, oracle.to_f64(dev.to_host(out), dtype), oracle.to_f64(want_o, dtype), P, V, extra=2.0 ** -10)
    # backward through Q.K^T: dQ lands in (B,S,H,D) storage through the permuted strides, dK through a column-major view
    go = sample(dev, g, (B, H, S, S), dtype)
    gq, gk = dev.zeros_like_storage(qv), dev.zeros_like_storage(kv)
    dev.backward(qv, gq, kv, gk, go)
    wgq, wgk = np.zeros_like(q_h), np.zeros_like(k_h)
    oracle.matmat_batch4_backward(dtype, B, H, S, D, S, q_h, qv.strides, wgq, k_h, kv.strides, wgk, dev.to_host(go))
    G = host(dev, go)
    assert_within(dtype, S, oracle.to_f64(dev.to_host(gq), dtype), oracle.to_f64(wgq, dtype), G, K, extra=2.0 ** -10 * 64)
    assert_within(dtype, S, oracle.to_f64(dev.to_host(gk), dtype), oracle.to_f64(wgk, dtype), Q, G, extra=2.0 ** -10 * 64)


def test_backward_accumulates_into_existing_gradients():
    """Gradient buffers are added to, never overwritten (cpu_kernel.rs:268,278): the same `x` feeding
    three Linear layers receives three accumulations (multi_head_attention.rs:123-131)."""
    dev, g = device(), rng(65)
    m, k, n = 64, 72, 40
    a, b, go = sample(dev, g, (m, k), "f32"), sample(dev, g, (k, n), "f32"), sample(dev, g, (m, n), "f32")
    ga, gb = dev.zeros_like_storage(a), dev.zeros_like_storage(b)
    for _ in range(3):
        dev.backward(a, ga, b, gb, go)
    A, B, G = host(dev, a), host(dev, b), host(dev, go)
    np.testing.assert_allclose(host(dev, ga), 3 * (G @ B.T), rtol=0, atol=1e-3)
    np.testing.assert_allclose(host(dev, gb), 3 * (A.T @ G), rtol=0, atol=1e-3)


# -------------------------------------------------------------- shape checks --
@pytest.mark.parametrize("shapes,msg", [
    (((3, 3), (4, 4)), "left: 3\n right: 4"),            # mod.rs:704-711
    (((1, 3, 3), (4, 4)), "left: 3\n right: 4"),         # mod.rs:713-720
    (((1, 3, 3), (1, 4, 4)), "left: 3\n right: 4"),      # mod.rs:722-729
    (((1, 5, 3, 3), (1, 5, 4, 4)), "left: 3\n right: 4"),  # mod.rs:731-740
    (((1, 2, 3), (2, 3, 4)), "left: 1\n right: 2"),      # mod.rs:742-749
    (((1, 1, 2, 3), (2, 1, 3, 4)), "left: 1\n right: 2"),  # mod.rs:751-758
    (((1, 1, 2, 3), (1, 2, 3, 4)), "left: 1\n right: 2"),  # mod.rs:760-767
])
def test_shape_mismatch_panics_before_the_kernel(shapes, msg):
    dev = device()
    x, y = dev.zeros("f32", shapes[0]), dev.zeros("f32", shapes[1])
    with pytest.raises(AssertionError) as e:
        dev.forward(x, y)
    assert msg in str(e.value)


# -------------------------------------------- broadcast views: a zero stride on a MATRIX axis --
@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("shape", [(48, 40, 72), (200, 136, 264), (5, 3, 7)])
@pytest.mark.parametrize("which", ["lhs_k", "lhs_m", "rhs_k", "rhs_n", "lhs_both", "ones"])
def test_matmul_broadcast_matrix_axes(dtype, shape, which):
    """`matrix_strides` lets views through whose matrix strides are [1,0], [0,1] or [1,1] (matmul/mod.rs:316-325): a
    vector broadcast along one matrix axis (`broadcast_to.rs:68-75` shares the tensor id, so the gradient buffer has
    the VECTOR's length and is written through the zero stride), or a size-1 tensor broadcast along both.  Forward is an
    ordinary product of the logical matrices; backward must SUM the logical gradient over the broadcast axis (the
    gradient of a broadcast).  Checked against float64 on the logical matrices; forward also against the oracle."""
    dev, g = device(), rng(907)
    m, k, n = shape
    announce("broadcast matrix axis", dtype, shape, which)
    vec = lambda length: upload(dev, g.standard_normal(length), dtype)
    full = lambda r, c: upload(dev, g.standard_normal((r, c)), dtype)
    from dfdx_amd.rocm import View
    if which == "lhs_k":      # lhs[i, kk] = v[i]: strides [1, 0]
        v = vec(m); lhs = View(v.storage, dtype, (m, k), (1, 0)); rhs = full(k, n)
    elif which == "lhs_m":    # lhs[i, kk] = v[kk]: strides [0, 1]
        v = vec(k); lhs = View(v.storage, dtype, (m, k), (0, 1)); rhs = full(k, n)
    elif which == "rhs_k":    # rhs[kk, j] = v[kk]: strides [1, 0]
        v = vec(k); rhs = View(v.storage, dtype, (k, n), (1, 0)); lhs = full(m, k)
    elif which == "rhs_n":    # rhs[kk, j] = v[j]: strides [0, 1]
        v = vec(n); rhs = View(v.storage, dtype, (k, n), (0, 1)); lhs = full(m, k)
    elif which == "lhs_both":  # a one-element tensor broadcast along both axes: strides [0, 0]
        v = vec(1); lhs = View(v.storage, dtype, (m, k), (0, 0)); rhs = full(k, n)
    else:                      # strides [1, 1]: a (1, 1) matrix -- the arm exists for size-1 axes
        m, k = 1, 1
        v = vec(1); lhs = View(v.storage, dtype, (1, 1), (1, 1)); rhs = full(1, n)
    out = dev.forward(lhs, rhs)
    go = upload(dev, g.standard_normal((m, n)), dtype)
    gl, gr = dev.zeros_like_storage(lhs), dev.zeros_like_storage(rhs)
    dev.backward(lhs, gl, rhs, gr, go)
    dev.synchronize()
    L, R, G = host(dev, lhs), host(dev, rhs), host(dev, go)
    ulp = {"f32": 2.0 ** -24, "f16": 2.0 ** -11}[dtype]
    want = L @ R
    assert_within(dtype, k, host(dev, out), want, L, R, extra=ulp * np.abs(want).max(), what="forward vs f64")
    want_or = oracle.matmat_forward(dtype, m, k, n, dev.to_host(lhs), lhs.strides, dev.to_host(rhs), rhs.strides)
    assert_within(dtype, k, host(dev, out), oracle.to_f64(want_or, dtype).reshape(m, n), L, R,
                  extra=2 * ulp * np.abs(want).max(), what="forward vs oracle")
    # logical gradients, then summed over the axes the storage does not have
    GL, GR = G @ R.T, L.T @ G

    def fold(grad, view):
        for ax, st in enumerate(view.strides):
            if st == 0 and view.shape[ax] > 1:
                grad = grad.sum(axis=ax, keepdims=True)
        return grad.reshape(-1)

    # a sum over up to max(m, k, n) products of sums over up to max(m, k, n) terms
    terms = max(m, k, n) ** 2
    for name, got, want_g, a_, b_ in (("grad_lhs", gl, fold(GL, lhs), G, R), ("grad_rhs", gr, fold(GR, rhs), L, G)):
        got64 = oracle.to_f64(dev.to_host(got), dtype)[: want_g.size]
        assert_within(dtype, terms, got64, want_g, a_, b_, extra=ulp * np.abs(want_g).max(), what=name)
