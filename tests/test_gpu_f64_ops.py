"""GPU: the ops around the matmuls in f64, the reference's fourth element type (`Device<f64>`; its CI runs every test in
f64 as well, .github/workflows/cargo-test.yml:28-32).  f64 leaves no room for tolerance arguments: every op is compared
with the numpy restatement to a few ulp, and a whole encoder block -- every op on the device -- with the host-glue +
CPU-oracle path to 1e-11 of the largest value, which pins the composition itself (what feeds what, which gradient
accumulates where) far more sharply than the 16-bit runs can."""
import numpy as np
import pytest

import oracle
from oracle import nn_ops
from helpers import logical, rng
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

D = "f64"
ULP = 2.0 ** -52


def up(dev, values):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(values.reshape(-1).copy(), D, values.shape)


def host(dev, view):
    return logical(dev.to_host(view).astype(np.float64), view.shape, view.strides, view.offset)


def close(got, want, ulps=64):
    scale = float(np.abs(want).max()) + 1e-300
    assert np.abs(got - want).max() <= ulps * ULP * scale, (np.abs(got - want).max(), scale)


def test_elementwise_ops_f64():
    dev, g = device(), rng(801)
    for n in (1, 7, 1000, 4099, 1 << 18):
        announce("f64 elementwise", n)
        x, y, go = (g.standard_normal(n) for _ in range(3))
        np.testing.assert_array_equal(host(dev, dev.scalar_mul_forward(up(dev, x), 0.3)), 0.3 * x)
        np.testing.assert_array_equal(host(dev, dev.relu_forward(up(dev, x))), np.maximum(x, 0.0))
        np.testing.assert_array_equal(host(dev, dev.add_forward(up(dev, x), up(dev, y))), x + y)
        gi = up(dev, y)
        dev.scalar_mul_backward(0.3, gi, up(dev, go))
        close(host(dev, gi), y + 0.3 * go, 2)
        gx = up(dev, y)
        dev.relu_backward(up(dev, x), gx, up(dev, go))
        np.testing.assert_array_equal(host(dev, gx), y + np.where(x > 0, go, 0.0))
        gl, gr = up(dev, x), up(dev, y)
        dev.add_backward(gl, gr, up(dev, go))
        np.testing.assert_array_equal(host(dev, gl), x + go)
        np.testing.assert_array_equal(host(dev, gr), y + go)
        gt = up(dev, x)
        dev.add_backward(gt, gt, up(dev, go))          # t + t
        np.testing.assert_array_equal(host(dev, gt), (x + go) + go)


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (7, 64), (5, 1000), (33, 517), (1031, 72)])
def test_softmax_f64(shape):
    dev, g = device(), rng(802)
    announce("f64 softmax", shape)
    rows, cols = shape
    x, go, gx0 = g.standard_normal(shape) * 6, g.standard_normal(shape), g.standard_normal(shape)
    scale = 0.125
    p = dev.softmax_forward(up(dev, x), scale)
    z = x * scale
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    want = e / e.sum(axis=-1, keepdims=True)
    got = host(dev, p)
    close(got, want, 8 + cols // 8)
    gx = up(dev, gx0)
    dev.softmax_backward(p, gx, up(dev, go), scale)
    close(host(dev, gx), gx0 + scale * got * (go - (go * got).sum(axis=-1, keepdims=True)), 16 + cols // 4)


@pytest.mark.parametrize("shape", [(1, 2), (4, 24), (70, 136), (9, 1000), (300, 64)])
def test_layer_norm_f64(shape):
    dev, g = device(), rng(803)
    announce("f64 layer norm", shape)
    rows, cols = shape
    x = g.standard_normal(shape) * 2 + 0.5
    gamma, beta = 1 + 0.1 * g.standard_normal(cols), 0.1 * g.standard_normal(cols)
    out = host(dev, dev.layer_norm_forward(up(dev, x), up(dev, gamma), up(dev, beta), 1e-5))
    close(out, nn_ops.layer_norm_forward(x, gamma, beta, 1e-5, D, faithful=False), 64 + cols)
    go, gx0, gg0, gb0 = g.standard_normal(shape), g.standard_normal(shape), g.standard_normal(cols), g.standard_normal(cols)
    gx, gg, gb = up(dev, gx0), up(dev, gg0), up(dev, gb0)
    dev.layer_norm_backward(up(dev, x), up(dev, gamma), gx, gg, gb, up(dev, go), 1e-5)
    wx, wg, wb = nn_ops.layer_norm_backward(x, gamma, go, 1e-5, D, gx0, gg0, gb0)
    close(host(dev, gx), wx, 256 + 4 * cols)
    close(host(dev, gg), wg, 256 + 4 * rows)
    close(host(dev, gb), wb, 64 + 4 * rows)


def test_reshape_and_bias_f64():
    from dfdx_amd.rocm import View

    dev, g = device(), rng(804)
    announce("f64 reshape / bias")
    B, H, S, Dh = 2, 3, 20, 8
    t = g.standard_normal((B, H, S, Dh))
    tv = up(dev, t)
    out = dev.reshape_forward(tv.permute(0, 2, 1, 3), (B, S, H * Dh))
    np.testing.assert_array_equal(host(dev, out), t.transpose(0, 2, 1, 3).reshape(B, S, H * Dh))
    go, gt0 = g.standard_normal((B, S, H * Dh)), g.standard_normal((B, H, S, Dh))
    gt = up(dev, gt0)
    dev.reshape_backward(tv.permute(0, 2, 1, 3), gt, up(dev, go))
    np.testing.assert_array_equal(host(dev, gt), gt0 + go.reshape(B, S, H, Dh).transpose(0, 2, 1, 3))
    # a broadcast axis in the input view: the gradient is the sum over it
    small = up(dev, g.standard_normal(5))
    bro = View(small.storage, D, (4, 5), (0, 1))
    gsmall0 = g.standard_normal(5)
    gsmall, gbro = up(dev, gsmall0), g.standard_normal((4, 5))
    dev.reshape_backward(bro, gsmall, up(dev, gbro.reshape(20)))
    close(host(dev, gsmall), gsmall0 + gbro.sum(axis=0), 8)
    x, b, gb0, gy = g.standard_normal((70, 24)), g.standard_normal(24), g.standard_normal(24), g.standard_normal((70, 24))
    np.testing.assert_array_equal(host(dev, dev.bias_forward(up(dev, x), up(dev, b))), x + b)
    gb = up(dev, gb0)
    dev.bias_backward(up(dev, gy), gb)
    close(host(dev, gb), gb0 + gy.sum(axis=0), 128)


@pytest.mark.parametrize("dims", [(2, 32, 64, 4, 128), (2, 24, 96, 4, 160)])
def test_small_encoder_block_entirely_on_the_device_f64(dims):
    """Head dimension 16: 1/sqrt(16) is a float, the scale rides in the softmax kernel.  Head dimension 24: it is not,
    and the block multiplies by the double scalar in an op of its own (multi_head_attention.rs:133-134)."""
    from dfdx_amd.encoder import EncoderBlock
    from encoder_ref import OracleBackend, encoder_block, init_params, val

    dev, g = device(), rng(805)
    B, S, d, H, ff = dims
    p = init_params(g, d, ff, D, std=0.2)
    for name in ("g1", "g2", "be1", "be2"):
        p[name] = val(p[name], D) + 0.1 * g.standard_normal(d)
    x = g.standard_normal((B * S, d))
    gout = g.standard_normal((B * S, d)) / (B * S)
    out_o, grads_o, dx_o = encoder_block(OracleBackend(D), D, p, x, B, S, d, H, ff, gout)
    announce("f64 encoder block on the device", (B, S, d, H, ff))
    shapes = {"wq": (d, d), "wk": (d, d), "wv": (d, d), "wo": (d, d), "w1": (ff, d), "w2": (d, ff)}
    params = {n: dev.tensor(np.asarray(v, np.float64).reshape(-1).copy(), D, shapes.get(n, (np.size(v),))) for n, v in p.items()}
    for deferred in (False, True):
        blk = EncoderBlock(dev, D, d, H, ff, params, deferred_zeros=deferred)
        out_v, saved = blk.forward(up(dev, x.reshape(B, S, d)))
        grads_v, gx_v = blk.backward(saved, up(dev, gout.reshape(B, S, d)))
        tol = lambda ref: 1e-11 * float(np.abs(ref).max()) + 1e-300
        assert np.abs(host(dev, out_v).reshape(B * S, d) - out_o).max() <= tol(out_o)
        assert np.abs(host(dev, gx_v).reshape(B * S, d) - dx_o).max() <= tol(dx_o)
        scale_b = float(np.abs(val(grads_o["bq"], D)).max())
        for name in grads_o:
            want = val(grads_o[name], D).reshape(-1)
            got = host(dev, grads_v[name]).reshape(-1)
            # the key bias shifts every score of a row alike: its gradient is zero up to rounding
            assert np.abs(got - want).max() <= (tol(want) if name != "bk" else 1e-11 * scale_b), name
