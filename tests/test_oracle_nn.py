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
