"""Pin the CPU oracle against the literals the reference's own tests hold.

The reference asserts these values for its Cpu device (and every other device)
in dfdx-core/src/tensor_ops/matmul/mod.rs:368-703 and
dfdx/src/nn/layers/linear.rs:97-204.  The scalar loss wrapped round the matmul
(exp().mean(), exp().sum(), square().mean()) is elementwise glue evaluated here
in float64; everything between the operands and `out` / the gradients goes
through the oracle's MatMat* drivers, rank-1 operands included (they are
reshapes to M=1 / N=1 / K=1 products, mod.rs:133-175).
"""
import json
import os

import numpy as np
import pytest

from helpers import row_major_strides

GOLD = os.path.join(os.path.dirname(__file__), "golden")
MATMUL = json.load(open(os.path.join(GOLD, "matmul_literals.json")))
LINEAR = json.load(open(os.path.join(GOLD, "linear_literals.json")))


def loss_grad(kind, out):
    out = out.astype(np.float64)
    if kind == "exp_mean":
        return np.exp(out) / out.size
    if kind == "exp_sum":
        return np.exp(out)
    if kind == "square_mean":
        return 2.0 * out / out.size
    raise KeyError(kind)


def as_matrix_view(arr, role, permuted):
    """Return (storage, (rows, cols), strides) of the 2-D operand the kernel sees.

    role 'lhs': rank-1 (K,) -> (1,K); role 'rhs': rank-1 (K,) -> (K,1); for the
    outer product the caller reshapes itself.  `permuted` applies dfdx's
    zero-copy permute to a rank-2 literal.
    """
    a = np.asarray(arr, dtype=np.float64)
    if a.ndim == 1:
        shape = (1, a.shape[0]) if role == "lhs" else (a.shape[0], 1)
        return a, shape, row_major_strides(shape)
    shape, strides = a.shape, row_major_strides(a.shape)
    if permuted:
        shape, strides = (shape[1], shape[0]), [strides[1], strides[0]]
    return a, tuple(shape), strides


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("case", MATMUL["cases"], ids=lambda c: c["name"])
def test_matmul_literals(oracle, case, dtype):
    np_dt = oracle.NP_DTYPES[dtype]
    a_lit, b_lit = np.asarray(case["a"]), np.asarray(case["b"])
    if a_lit.ndim == 1 and b_lit.ndim == 1:  # vec (M,) x vec (N,) -> outer product, K = 1 (mod.rs:139-144)
        a, ashape, astr = a_lit, (a_lit.shape[0], 1), [1, 1]
        b, bshape, bstr = b_lit, (1, b_lit.shape[0]), [b_lit.shape[0], 1]
    else:
        a, ashape, astr = as_matrix_view(a_lit, "lhs", case.get("permute_a", False))
        b, bshape, bstr = as_matrix_view(b_lit, "rhs", case.get("permute_b", False))
    (m, k), (k2, n) = ashape, bshape
    assert k == k2
    a_st = np.ascontiguousarray(a, dtype=np_dt).reshape(-1)
    b_st = np.ascontiguousarray(b, dtype=np_dt).reshape(-1)
    tol = case.get("tol", 1e-6)

    out = oracle.matmat_forward(dtype, m, k, n, a_st, astr, b_st, bstr)
    np.testing.assert_allclose(out.reshape(np.asarray(case["out"]).shape), case["out"], rtol=0, atol=tol)

    g = loss_grad(case["loss"], out).astype(np_dt)
    ga = np.zeros_like(a_st)
    gb = np.zeros_like(b_st)
    oracle.matmat_backward(dtype, m, k, n, a_st, astr, ga, b_st, bstr, gb, g)
    # gradients live in the operand's physical layout, i.e. the literal's own shape
    np.testing.assert_allclose(ga.reshape(a_lit.shape), case["grad_a"], rtol=0, atol=tol)
    np.testing.assert_allclose(gb.reshape(b_lit.shape), case["grad_b"], rtol=0, atol=tol)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("case", LINEAR["cases"], ids=lambda c: c["name"])
def test_linear_literals(oracle, case, dtype):
    """Linear = x.matmul(weight.permute()) + bias (linear.rs:82-89); db = column sum of dy."""
    np_dt = oracle.NP_DTYPES[dtype]
    w = np.asarray(LINEAR["weight"], dtype=np_dt)  # (O, I) storage
    bias = np.asarray(LINEAR["bias"], dtype=np.float64)
    o, i = w.shape
    wt_strides = [1, i]  # the (I, O) view of the (O, I) storage
    x = np.asarray(case["x"], dtype=np_dt)
    x_st, w_st = x.reshape(-1).copy(), w.reshape(-1).copy()
    gx, gw = np.zeros_like(x_st), np.zeros_like(w_st)
    if x.ndim <= 2:
        m = 1 if x.ndim == 1 else x.shape[0]
        xs = [i, 1]
        y = oracle.matmat_forward(dtype, m, i, o, x_st, xs, w_st, wt_strides)
        y = y.reshape(m, o).astype(np.float64) + bias
        gy = loss_grad("square_mean", y)
        oracle.matmat_backward(dtype, m, i, o, x_st, xs, gx, w_st, wt_strides, gw, gy.astype(np_dt).reshape(-1))
    else:
        b, m = x.shape[0], x.shape[1]
        xs = row_major_strides(x.shape)
        y = oracle.matmat_br_forward(dtype, b, m, i, o, x_st, xs, w_st, wt_strides)
        y = y.reshape(b, m, o).astype(np.float64) + bias
        gy = loss_grad("square_mean", y)
        oracle.matmat_br_backward(dtype, b, m, i, o, x_st, xs, gx, w_st, wt_strides, gw, gy.astype(np_dt).reshape(-1))
    np.testing.assert_allclose(y.reshape(np.asarray(case["y"]).shape), case["y"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(gw.reshape(o, i), case["grad_weight"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(gy.reshape(-1, o).sum(axis=0), case["grad_bias"], rtol=0, atol=1e-6)
