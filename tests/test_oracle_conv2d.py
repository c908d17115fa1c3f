"""The conv2d restatement (oracle/conv2d.py) against the PyTorch-produced literals the reference's tests hold
(conv2d/tests.rs) and against a direct-summation convolution."""
import json
import os

import numpy as np
import pytest

import oracle
from oracle.conv2d import Conv2DOp, conv2d_backward, conv2d_forward

GOLD = os.path.join(os.path.dirname(__file__), "golden")
CONV = json.load(open(os.path.join(GOLD, "conv2d_literals.json")))


def op_of(case, batch=1):
    x, w = np.asarray(case["x"]), np.asarray(case["weight"])
    return Conv2DOp.make(batch, x.shape[0], w.shape[0], x.shape[1], x.shape[2], w.shape[2], case["stride"],
                         case["padding"], case["dilation"], case["groups"])


def loss_grad(kind, out):
    return {"exp_mean": np.exp(out) / out.size, "mean": np.full(out.shape, 1.0 / out.size)}[kind]


def direct_conv(op: Conv2DOp, x, w):
    """Seven nested loops, float64: out[b,o,oh,ow] = sum_{c,k1,k2} x[b, g*C/G + c, y, x] * w[o, c, k1, k2]."""
    x = x.reshape(op.batch, op.chan_in, op.h_in, op.w_in)
    w = w.reshape(op.chan_out, op.chan_in // op.groups, op.kernel, op.kernel)
    out = np.zeros((op.batch, op.chan_out, op.h_out, op.w_out))
    cg, og = op.chan_in // op.groups, op.chan_out // op.groups
    for b in range(op.batch):
        for o in range(op.chan_out):
            g = o // og
            for oh in range(op.h_out):
                for ow in range(op.w_out):
                    s = 0.0
                    for c in range(cg):
                        for k1 in range(op.kernel):
                            for k2 in range(op.kernel):
                                y = oh * op.stride + op.dilation * k1 - op.padding
                                xx = ow * op.stride + op.dilation * k2 - op.padding
                                if 0 <= y < op.h_in and 0 <= xx < op.w_in:
                                    s += x[b, g * cg + c, y, xx] * w[o, c, k1, k2]
                    out[b, o, oh, ow] = s
    return out


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("case", CONV["cases"], ids=lambda c: c["name"])
def test_conv2d_literals(case, dtype):
    op = op_of(case)
    x = oracle.to_storage(np.asarray(case["x"], np.float64).reshape(-1), dtype)
    w = oracle.to_storage(np.asarray(case["weight"], np.float64).reshape(-1), dtype)
    y = oracle.to_f64(conv2d_forward(dtype, op, x, w), dtype).reshape(op.chan_out, op.h_out, op.w_out)
    if "bias" in case:
        y = y + np.asarray(case["bias"]).reshape(-1, 1, 1)
    np.testing.assert_allclose(y, case["out"], rtol=0, atol=2e-6)
    gy = loss_grad(case["loss"], y)
    gx, gw = np.zeros_like(x), np.zeros_like(w)
    conv2d_backward(dtype, op, x, gx, w, gw, oracle.to_storage(gy.reshape(-1), dtype))
    np.testing.assert_allclose(oracle.to_f64(gx, dtype).reshape(np.shape(case["x"])), case["grad_x"], rtol=0, atol=2e-6)
    np.testing.assert_allclose(oracle.to_f64(gw, dtype).reshape(np.shape(case["weight"])), case["grad_weight"], rtol=0, atol=2e-6)
    if "bias" in case:
        np.testing.assert_allclose(gy.sum(axis=(1, 2)), case["grad_bias"], rtol=0, atol=2e-6)


@pytest.mark.parametrize("cfg", [
    dict(batch=2, chan_in=4, chan_out=6, h_in=7, w_in=6, kernel=3, stride=2, padding=1, dilation=1, groups=2),
    dict(batch=1, chan_in=3, chan_out=5, h_in=9, w_in=8, kernel=2, stride=1, padding=2, dilation=3, groups=1),
    dict(batch=3, chan_in=6, chan_out=3, h_in=5, w_in=5, kernel=1, stride=1, padding=0, dilation=1, groups=3),
    dict(batch=1, chan_in=5, chan_out=3, h_in=7, w_in=6, kernel=2, stride=4, padding=3, dilation=1, groups=1),
])
def test_conv2d_against_direct_summation(cfg):
    """Forward equals the seven-loop definition; the backward is the transpose of the (linear) forward:
    <conv(x, w), g> differentiates to <x, grad_x> and <w, grad_w> exactly (float64)."""
    op = Conv2DOp.make(**cfg)
    g = np.random.default_rng(21)
    x = g.standard_normal(op.batch * op.chan_in * op.h_in * op.w_in)
    w = g.standard_normal(op.chan_out * (op.chan_in // op.groups) * op.kernel ** 2)
    y = conv2d_forward("f64", op, x, w)
    np.testing.assert_allclose(y.reshape(op.batch, op.chan_out, op.h_out, op.w_out), direct_conv(op, x, w), rtol=0, atol=1e-12)
    go = g.standard_normal(y.size)
    gx, gw = np.zeros_like(x), np.zeros_like(w)
    conv2d_backward("f64", op, x, gx, w, gw, go)
    dx, dw = g.standard_normal(x.size), g.standard_normal(w.size)
    np.testing.assert_allclose(np.dot(conv2d_forward("f64", op, dx, w), go), np.dot(dx, gx), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(np.dot(conv2d_forward("f64", op, x, dw), go), np.dot(dw, gw), rtol=1e-11, atol=1e-11)


def test_batched_equals_unbatched_broadcast():
    """conv2d/tests.rs:219-250: a batch of 10 copies gives 10 copies of y, the same filter gradient x10 ... here
    with the sum loss, the filter gradient of the batch is 10x and every image gradient equals the single one."""
    g = np.random.default_rng(22)
    op1 = Conv2DOp.make(1, 3, 5, 10, 10, 4, stride=3, padding=2)
    opb = Conv2DOp.make(4, 3, 5, 10, 10, 4, stride=3, padding=2)
    x, w = g.standard_normal(3 * 100).astype(np.float32), g.standard_normal(5 * 3 * 16).astype(np.float32)
    y1 = conv2d_forward("f32", op1, x, w)
    yb = conv2d_forward("f32", opb, np.tile(x, 4), w)
    np.testing.assert_array_equal(yb.reshape(4, -1), np.tile(y1, (4, 1)))
    go = g.standard_normal(y1.size).astype(np.float32)
    gx1, gw1 = np.zeros_like(x), np.zeros_like(w)
    conv2d_backward("f32", op1, x, gx1, w, gw1, go)
    gxb, gwb = np.zeros(4 * x.size, np.float32), np.zeros_like(w)
    conv2d_backward("f32", opb, np.tile(x, 4), gxb, w, gwb, np.tile(go, 4))
    np.testing.assert_array_equal(gxb.reshape(4, -1), np.tile(gx1, (4, 1)))
    np.testing.assert_allclose(gwb, 4 * gw1, rtol=1e-5, atol=1e-5)
