"""The numpy restatement of the module-level ops (oracle/nn_ops.py) against the reference's own literals."""
import json
import os

import numpy as np
import pytest

from oracle import nn_ops

GOLD = os.path.join(os.path.dirname(__file__), "golden")
LINEAR = json.load(open(os.path.join(GOLD, "linear_literals.json")))


@pytest.mark.parametrize("case", LINEAR["cases"], ids=lambda c: c["name"])
def test_bias_ops_on_linear_literals(case):
    """linear.rs:97-204: y = x.W^T + b and db under the test's loss; dy is recovered from the literals' y."""
    w = np.asarray(LINEAR["weight"], np.float64)
    b = np.asarray(LINEAR["bias"], np.float64)
    x = np.asarray(case["x"], np.float64)
    y = np.asarray(case["y"], np.float64)
    pre = x @ w.T
    np.testing.assert_allclose(nn_ops.bias_forward(pre, b, "f32"), y, rtol=0, atol=2e-6)
    gy = 2.0 * y / y.size  # loss = square().mean()
    for faithful in (True, False):
        db = nn_ops.bias_backward(nn_ops.round_to(gy, "f32"), np.zeros_like(b), "f32", faithful=faithful)
        np.testing.assert_allclose(db, case["grad_bias"], rtol=0, atol=1e-6)


def test_bias_backward_sequential_rounding_is_visible():
    """The faithful variant rounds after every row: with f16 a long column of ones stalls at 2048."""
    go = np.ones((4096, 3))
    seq = nn_ops.bias_backward(go, np.zeros(3), "f16", faithful=True)
    wide = nn_ops.bias_backward(go, np.zeros(3), "f16", faithful=False)
    assert (seq == 2048).all() and (wide == 4096).all()


def test_bias_backward_accumulates_and_matches_brute_force():
    rng = np.random.default_rng(5)
    go = nn_ops.round_to(rng.standard_normal((7, 5)), "f32")
    gb0 = nn_ops.round_to(rng.standard_normal(5), "f32")
    want = gb0.copy()
    for r in range(7):
        for c in range(5):
            want[c] = np.float64(np.float32(want[c] + go[r, c]))
    np.testing.assert_array_equal(nn_ops.bias_backward(go, gb0, "f32"), want)


GLUE = json.load(open(os.path.join(GOLD, "attention_glue_literals.json")))


@pytest.mark.parametrize("case", GLUE["softmax"], ids=lambda c: c["name"])
@pytest.mark.parametrize("faithful", [True, False])
def test_softmax_literals(case, faithful):
    """softmax.rs:113-166: forward values and the gradient under loss = mean(out * mask)."""
    x, mask = np.asarray(case["x"]), np.asarray(case["mask"])
    out = nn_ops.softmax_forward(x, "f32", faithful=faithful)
    np.testing.assert_allclose(out, case["out"], rtol=0, atol=1e-6)
    g = nn_ops.round_to(mask / mask.size, "f32")
    gx = nn_ops.softmax_backward(x, g, "f32", faithful=faithful)
    np.testing.assert_allclose(gx, case["grad_x"], rtol=0, atol=1e-6)


def test_softmax_backward_finite_differences():
    """The two restatements of the gradient against central differences of the forward (float64)."""
    g = np.random.default_rng(11)
    x, w = g.standard_normal((3, 7)), g.standard_normal((3, 7))
    f = lambda t: float((nn_ops.softmax_forward(t, "f64", faithful=False) * w).sum())
    fd = np.zeros_like(x)
    for i in np.ndindex(*x.shape):
        d = np.zeros_like(x); d[i] = 1e-6
        fd[i] = (f(x + d) - f(x - d)) / 2e-6
    for faithful in (True, False):
        np.testing.assert_allclose(nn_ops.softmax_backward(x, w, "f64", faithful=faithful), fd, rtol=0, atol=1e-8)


def test_softmax_rows_sum_to_one_and_shift_invariance():
    g = np.random.default_rng(12)
    x = nn_ops.round_to(g.standard_normal((5, 33)) * 4, "f16")
    p = nn_ops.softmax_forward(x, "f16")
    assert np.all(np.abs(p.sum(axis=-1) - 1.0) < 33 * 2.0 ** -11)
    np.testing.assert_array_equal(p, nn_ops.softmax_forward(x + 8.0, "f16"))  # t - max is what enters exp


@pytest.mark.parametrize("case", GLUE["reshape"], ids=lambda c: c["name"])
def test_reshape_literals(case):
    """reshape_to/mod.rs:197-228: the copy of a permuted / broadcast view and, where given, its gradient."""
    st = np.asarray(case["storage"])
    out = nn_ops.reshape_forward(st, case["shape"], case["strides"])
    np.testing.assert_allclose(out, case["out"], rtol=0, atol=1e-7)
    if "grad_storage" in case:
        go = nn_ops.round_to(np.exp(out) / out.size, "f32")
        gi = nn_ops.reshape_backward(case["shape"], case["strides"], np.zeros_like(st), go, "f32")
        np.testing.assert_allclose(gi, case["grad_storage"], rtol=0, atol=1e-6)


def test_reshape_backward_broadcast_accumulates():
    gi = nn_ops.reshape_backward([2, 3], [0, 1], np.zeros(3), np.arange(6.0), "f32")
    np.testing.assert_array_equal(gi, [3.0, 5.0, 7.0])


@pytest.mark.parametrize("case", GLUE["scalar_mul"], ids=lambda c: c["name"])
def test_scalar_mul_literals(case):
    x = np.asarray(case["x"])
    out = nn_ops.scalar_mul_forward(x, case["scalar"], "f32")
    np.testing.assert_allclose(out, case["out"], rtol=0, atol=1e-7)
    gx = nn_ops.scalar_mul_backward(case["scalar"], np.zeros_like(x), nn_ops.round_to(np.exp(out), "f32"), "f32")
    np.testing.assert_allclose(gx, case["grad_x"], rtol=0, atol=1e-6)
