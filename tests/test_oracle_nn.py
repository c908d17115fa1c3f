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


ENC = json.load(open(os.path.join(GOLD, "encoder_glue_literals.json")))


@pytest.mark.parametrize("case", ENC["normalize"], ids=lambda c: c["name"].split()[0])
@pytest.mark.parametrize("faithful", [True, False])
def test_normalize_literals(case, faithful):
    """normalize.rs:57-117: values, and the gradient of r.exp().mean() through the closed-form backward."""
    a = np.atleast_2d(np.asarray(case["a"], np.float64))
    r = nn_ops.normalize_forward(a, 1e-5, "f32", faithful=faithful)
    np.testing.assert_allclose(r, np.atleast_2d(case["r"]), rtol=0, atol=2e-6)
    ones, zeros = np.ones(a.shape[-1]), np.zeros(a.shape[-1])
    g = nn_ops.round_to(np.exp(r) / r.size, "f32")
    gx, _, _ = nn_ops.layer_norm_backward(a, ones, g, 1e-5, "f32", np.zeros_like(a), zeros, zeros)
    np.testing.assert_allclose(gx, np.atleast_2d(case["grad_a"]), rtol=0, atol=2e-6)


def test_normalize_of_constant_rows_is_zero():
    """normalize.rs:119-127: all-ones input -> zeros, zero gradient."""
    a = np.ones((4, 2, 3))
    for faithful in (True, False):
        assert not nn_ops.normalize_forward(a, 1e-5, "f32", faithful=faithful).any()
    gx, gg, gb = nn_ops.layer_norm_backward(a, np.ones(3), np.full(a.shape, 1 / 24), 1e-5, "f32", np.zeros_like(a), np.zeros(3), np.zeros(3))
    assert not gx.any() and not gg.any()
    np.testing.assert_allclose(gb, 8 / 24)


def test_layer_norm_literals():
    """layer_norm1d.rs:159-180: with gamma = 1, beta = 0 the module's output rows r are normalized rows, so feeding r
    itself reproduces r (to the 1e-5 epsilon) and the literal gradients of r.mean(): grad_gamma = sum_rows r / 15,
    grad_beta = 3 / 15."""
    ln = ENC["layer_norm_2d"]
    r = np.asarray(ln["r"], np.float64)
    ones, zeros = np.ones(5), np.zeros(5)
    for faithful in (True, False):
        out = nn_ops.layer_norm_forward(r, ones, zeros, 1e-5, "f32", faithful=faithful)
        np.testing.assert_allclose(out, r, rtol=0, atol=2e-5)
    g = np.full(r.shape, 1.0 / r.size)
    gx, gg, gb = nn_ops.layer_norm_backward(r, ones, g, 1e-5, "f32", np.zeros_like(r), zeros, zeros)
    np.testing.assert_allclose(gg, ln["grad_gamma"], rtol=0, atol=2e-6)
    np.testing.assert_allclose(gb, ln["grad_beta"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(gx, 0.0, atol=1e-6)   # a constant gradient has no component a normalized row can feel


def test_layer_norm_backward_against_finite_differences():
    rng = np.random.default_rng(21)
    x, gamma, beta = rng.standard_normal((3, 7)), rng.standard_normal(7), rng.standard_normal(7)
    g = rng.standard_normal((3, 7))
    loss = lambda x_, gm_, bt_: float((nn_ops.layer_norm_forward(x_, gm_, bt_, 1e-5, "f64") * g).sum())
    gx, gg, gb = nn_ops.layer_norm_backward(x, gamma, g, 1e-5, "f64", np.zeros_like(x), np.zeros(7), np.zeros(7))
    h = 1e-6
    for idx in [(0, 0), (1, 3), (2, 6)]:
        d = np.zeros_like(x); d[idx] = h
        assert abs((loss(x + d, gamma, beta) - loss(x - d, gamma, beta)) / (2 * h) - gx[idx]) < 1e-6
    for j in (0, 4):
        d = np.zeros(7); d[j] = h
        assert abs((loss(x, gamma + d, beta) - loss(x, gamma - d, beta)) / (2 * h) - gg[j]) < 1e-6
        assert abs((loss(x, gamma, beta + d) - loss(x, gamma, beta - d)) / (2 * h) - gb[j]) < 1e-6
    # accumulation into non-zero gradients
    gx2, gg2, gb2 = nn_ops.layer_norm_backward(x, gamma, g, 1e-5, "f64", np.ones_like(x), np.ones(7), np.ones(7))
    np.testing.assert_allclose(gx2 - 1, gx, atol=1e-12)
    np.testing.assert_allclose(gg2 - 1, gg, atol=1e-12)
    np.testing.assert_allclose(gb2 - 1, gb, atol=1e-12)


def test_layer_norm_faithful_f16_is_close_to_the_exact_formula():
    rng = np.random.default_rng(22)
    x = nn_ops.round_to(rng.standard_normal((5, 64)) * 3 + 1, "f16")
    gamma, beta = nn_ops.round_to(rng.standard_normal(64), "f16"), nn_ops.round_to(rng.standard_normal(64), "f16")
    a = nn_ops.layer_norm_forward(x, gamma, beta, 1e-5, "f16", faithful=True)
    b = nn_ops.layer_norm_forward(x, gamma, beta, 1e-5, "f16", faithful=False)
    assert np.abs(a - b).max() <= 8 * 2.0 ** -11 * np.abs(b).max()


def test_relu_literals():
    """relu/mod.rs:48-59."""
    rl = ENC["relu"]
    x = np.asarray(rl["x"], np.float64)
    r = nn_ops.relu_forward(x, "f32")
    np.testing.assert_array_equal(r, rl["r"])
    g = nn_ops.round_to(np.exp(r) / r.size, "f32")
    np.testing.assert_allclose(nn_ops.relu_backward(x, np.zeros(5), g, "f32"), rl["grad_x"], rtol=0, atol=1e-6)


def test_add_forward_and_backward():
    a, b = np.asarray([1.0, 2.0, 2048.0]), np.asarray([0.5, -2.0, 1.0])
    np.testing.assert_array_equal(nn_ops.add_forward(a, b, "f16"), [1.5, 0.0, 2048.0])   # 2049 is not an f16
    gl, gr = nn_ops.add_backward(np.asarray([1.0, 1.0, 1.0]), np.zeros(3), np.asarray([0.25, 0.5, 1.0]), "f32")
    np.testing.assert_array_equal(gl, [1.25, 1.5, 2.0])
    np.testing.assert_array_equal(gr, [0.25, 0.5, 1.0])
