"""GPU parity of the ops between a transformer encoder block's GEMMs (transformer.rs:24-48): LayerNorm1D over the
last axis, ReLU and the residual add -- against the reference's literals and the numpy restatement."""
import json
import os

import numpy as np
import pytest

import oracle
from oracle import nn_ops
from helpers import logical, rng
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
ENC = json.load(open(os.path.join(GOLD, "encoder_glue_literals.json")))
EPS = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}  # half an ulp at 1.0


def host(dev, view):
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


# ------------------------------------------------------------------ literals --
@pytest.mark.parametrize("case", ENC["normalize"], ids=lambda c: c["name"].split()[0])
def test_normalize_literals(case):
    """normalize.rs:57-117 through the layer-norm entry with gamma = 1, beta = 0."""
    dev = device()
    announce("normalize literal", case["name"])
    a = np.atleast_2d(np.asarray(case["a"], np.float64))
    n = a.shape[-1]
    x, gamma, beta = upload(dev, a, "f32"), upload(dev, np.ones(n), "f32"), upload(dev, np.zeros(n), "f32")
    r = dev.layer_norm_forward(x, gamma, beta, 1e-5)
    np.testing.assert_allclose(host(dev, r), np.atleast_2d(case["r"]), rtol=0, atol=2e-6)
    gx, gg, gb = dev.zeros("f32", a.shape), dev.zeros("f32", (n,)), dev.zeros("f32", (n,))
    dev.layer_norm_backward(x, gamma, gx, gg, gb, upload(dev, np.exp(host(dev, r)) / a.size, "f32"), 1e-5)
    np.testing.assert_allclose(host(dev, gx), np.atleast_2d(case["grad_a"]), rtol=0, atol=2e-6)


def test_layer_norm_literals():
    """layer_norm1d.rs:159-180: the module's output rows fed back in (see the oracle test of the same name)."""
    dev = device()
    announce("layer norm literal")
    ln = ENC["layer_norm_2d"]
    r = np.asarray(ln["r"], np.float64)
    x, gamma, beta = upload(dev, r, "f32"), upload(dev, np.ones(5), "f32"), upload(dev, np.zeros(5), "f32")
    np.testing.assert_allclose(host(dev, dev.layer_norm_forward(x, gamma, beta, 1e-5)), r, rtol=0, atol=2e-5)
    gx, gg, gb = dev.zeros("f32", r.shape), dev.zeros("f32", (5,)), dev.zeros("f32", (5,))
    dev.layer_norm_backward(x, gamma, gx, gg, gb, upload(dev, np.full(r.shape, 1.0 / r.size), "f32"), 1e-5)
    np.testing.assert_allclose(host(dev, gg), ln["grad_gamma"], rtol=0, atol=2e-6)
    np.testing.assert_allclose(host(dev, gb), ln["grad_beta"], rtol=0, atol=1e-6)


def test_relu_literals():
    """relu/mod.rs:48-59."""
    dev = device()
    announce("relu literal")
    rl = ENC["relu"]
    x = upload(dev, rl["x"], "f32")
    r = dev.relu_forward(x)
    np.testing.assert_array_equal(host(dev, r), rl["r"])
    gx = dev.zeros("f32", x.shape)
    dev.relu_backward(x, gx, upload(dev, np.exp(host(dev, r)) / 5, "f32"))
    np.testing.assert_allclose(host(dev, gx), rl["grad_x"], rtol=0, atol=1e-6)


# ---------------------------------------------------------------- layer norm --
LN_SHAPES = [(1, 1), (3, 5), (7, 64), (33, 512), (5, 1000), (64, 1024), (9, 2048), (3, 4096), (2, 5000), (2, 1001),
             (1031, 72), (8192, 1024),
             # long rows, 256 threads each: 2 / 4 / 8 vectors per thread, more rows than workgroups, then the row-walking form
             (5, 5120), (1100, 4096), (3, 8192), (2, 16384), (6, 4104), (2, 20000)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", LN_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_layer_norm_seeded(shape, dtype):
    """Forward against the formula evaluated exactly and rounded once (what an f32 row pass targets) and against the
    reference's op-by-op composition; backward, accumulated into non-zero gradient buffers, against the closed form."""
    dev, g = device(), rng(501)
    rows, cols = shape
    announce("layer norm", shape, dtype)
    x = upload(dev, g.standard_normal((rows, cols)) * 2 + 0.5, dtype)
    gamma, beta = upload(dev, 1 + 0.1 * g.standard_normal(cols), dtype), upload(dev, 0.1 * g.standard_normal(cols), dtype)
    x64, gm64, bt64 = host(dev, x), host(dev, gamma), host(dev, beta)
    out = host(dev, dev.layer_norm_forward(x, gamma, beta, 1e-5))
    exact = nn_ops.layer_norm_forward(x64, gm64, bt64, 1e-5, dtype, faithful=False)
    scale = float(np.abs(exact).max()) + 1.0
    assert np.abs(out - exact).max() <= 2 * EPS[dtype] * scale + 1e-6
    # The op-by-op composition rounds about nine times per element; its running sums in a 16-bit type drift with the
    # row length (a sum of 1000 bf16 terms is good to two digits), so that comparison is for short rows there (and in f32
    # for rows of up to 5000: over 20000 terms the composition's own running sums are 4e-6 off).
    if rows * cols <= 1 << 16 and cols > 1 and ((dtype == "f32" and cols <= 5000) or cols <= 72):
        faithful = nn_ops.layer_norm_forward(x64, gm64, bt64, 1e-5, dtype, faithful=True)
        assert np.abs(out - faithful).max() <= (16 * EPS[dtype] + (0 if dtype == "f32" else 2e-3)) * scale
    go = upload(dev, g.standard_normal((rows, cols)), dtype)
    gx0, gg0, gb0 = (upload(dev, g.standard_normal(s), dtype) for s in ((rows, cols), (cols,), (cols,)))
    gx, gg, gb = (dev.tensor(dev.to_host(t), dtype, t.shape) for t in (gx0, gg0, gb0))
    dev.layer_norm_backward(x, gamma, gx, gg, gb, go, 1e-5)
    wx, wg, wb = nn_ops.layer_norm_backward(x64, gm64, host(dev, go), 1e-5, dtype, host(dev, gx0), host(dev, gg0), host(dev, gb0))
    # f32 sums of `rows` (columns) or `cols` (rows) terms of O(1): a few ulp of the largest partial sum
    tol_x = 4 * EPS[dtype] * (float(np.abs(wx).max()) + 1.0) + 1e-5 * np.sqrt(cols)
    assert np.abs(host(dev, gx) - wx).max() <= tol_x
    col_tol = 4 * EPS[dtype] * (float(np.abs(wg).max()) + 1.0) + 4e-6 * rows ** 0.5 * (float(np.abs(x64).max()) + 1.0)
    assert np.abs(host(dev, gg) - wg).max() <= col_tol
    assert np.abs(host(dev, gb) - wb).max() <= 4 * EPS[dtype] * (float(np.abs(wb).max()) + 1.0) + 4e-6 * rows ** 0.5 * 5


def test_layer_norm_constant_rows_and_unaligned_views():
    """Rows of equal values normalize to beta (normalize.rs:119-127); operands at odd element offsets take the
    element-wise path."""
    dev, g = device(), rng(502)
    announce("layer norm constant rows")
    x, gamma, beta = upload(dev, np.ones((4, 24)), "f16"), upload(dev, np.full(24, 2.0), "f16"), upload(dev, np.full(24, 0.25), "f16")
    np.testing.assert_array_equal(host(dev, dev.layer_norm_forward(x, gamma, beta, 1e-5)), np.full((4, 24), 0.25))
    from dfdx_amd.rocm import View
    announce("layer norm unaligned")
    base = upload(dev, g.standard_normal(3 * 40 + 1), "bf16")
    xv = View(base.storage, "bf16", (3, 40), (40, 1), 1)          # 2 bytes past a 16-byte boundary
    gm, bt = upload(dev, np.ones(40), "bf16"), upload(dev, np.zeros(40), "bf16")
    out = dev.layer_norm_forward(dev.reshape_forward(View(base.storage, "bf16", (3, 40), (40, 1), 1), (3, 40)), gm, bt)
    want = nn_ops.layer_norm_forward(host(dev, xv), np.ones(40), np.zeros(40), 1e-5, "bf16", faithful=False)
    assert np.abs(host(dev, out) - want).max() <= 2 * EPS["bf16"] * 4


# --------------------------------------------------------------- relu / add --
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("n", [1, 7, 64, 1000, 4099, 1 << 20])
def test_relu_and_add_seeded(n, dtype):
    """Exact ops: one rounding in the reference, one here -- bit-identical."""
    dev, g = device(), rng(503)
    announce("relu / add", n, dtype)
    x, y, go, g0, g1 = (upload(dev, g.standard_normal(n), dtype) for _ in range(5))
    x64, y64, go64 = host(dev, x), host(dev, y), host(dev, go)
    np.testing.assert_array_equal(host(dev, dev.relu_forward(x)), nn_ops.relu_forward(x64, dtype))
    gx = dev.tensor(dev.to_host(g0), dtype)
    dev.relu_backward(x, gx, go)
    np.testing.assert_array_equal(host(dev, gx), nn_ops.relu_backward(x64, host(dev, g0), go64, dtype))
    np.testing.assert_array_equal(host(dev, dev.add_forward(x, y)), nn_ops.add_forward(x64, y64, dtype))
    gl, gr = dev.tensor(dev.to_host(g0), dtype), dev.tensor(dev.to_host(g1), dtype)
    dev.add_backward(gl, gr, go)
    wl, wr = nn_ops.add_backward(host(dev, g0), host(dev, g1), go64, dtype)
    np.testing.assert_array_equal(host(dev, gl), wl)
    np.testing.assert_array_equal(host(dev, gr), wr)
    # t + t: one gradient buffer receives grad_out twice, one add after the other
    gt = dev.tensor(dev.to_host(g0), dtype)
    dev.add_backward(gt, gt, go)
    once, _ = nn_ops.add_backward(host(dev, g0), host(dev, g0), go64, dtype)
    twice, _ = nn_ops.add_backward(once, once, go64, dtype)
    np.testing.assert_array_equal(host(dev, gt), twice)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_relu_add_and_scalar_mul_on_streamed_inputs(dtype):
    """From 128 MiB of read-only input per launch on, the element-wise kernels load it non-temporally: same bits.
    2^25 elements: every op in f32 (128 MiB per tensor), the two-input ops (ReLU backward, add forward) in bf16."""
    dev, g = device(), rng(504)
    n = 1 << 25
    announce("relu / add / scalar mul, streamed inputs", n, dtype)
    small = g.standard_normal(1 << 16)
    x, y, go = (upload(dev, np.tile(np.roll(small, 17 * i), n >> 16), dtype) for i in range(3))
    x64, y64, go64 = host(dev, x), host(dev, y), host(dev, go)
    np.testing.assert_array_equal(host(dev, dev.relu_forward(x)), nn_ops.relu_forward(x64, dtype))
    gx = dev.tensor(dev.to_host(y), dtype)
    dev.relu_backward(x, gx, go)
    np.testing.assert_array_equal(host(dev, gx), nn_ops.relu_backward(x64, y64, go64, dtype))
    del gx
    np.testing.assert_array_equal(host(dev, dev.add_forward(x, y)), nn_ops.add_forward(x64, y64, dtype))
    gl, gr = dev.tensor(dev.to_host(x), dtype), dev.tensor(dev.to_host(y), dtype)
    dev.add_backward(gl, gr, go)
    wl, wr = nn_ops.add_backward(x64, y64, go64, dtype)
    np.testing.assert_array_equal(host(dev, gl), wl)
    np.testing.assert_array_equal(host(dev, gr), wr)
    del gl, gr, wl, wr
    s = 0.25   # a power of two: the product is exact, so a fused and an unfused multiply-add round alike
    np.testing.assert_array_equal(host(dev, dev.scalar_mul_forward(x, s)), nn_ops.scalar_mul_forward(x64, s, dtype))
    gi = dev.tensor(dev.to_host(y), dtype)
    dev.scalar_mul_backward(s, gi, go)
    np.testing.assert_array_equal(host(dev, gi), nn_ops.scalar_mul_backward(s, y64, go64, dtype))


def test_relu_signed_zero_and_nan():
    dev = device()
    announce("relu special values")
    x = upload(dev, [-0.0, 0.0, np.inf, -np.inf, 1e-30], "f32")
    np.testing.assert_array_equal(host(dev, dev.relu_forward(x)), [0.0, 0.0, np.inf, 0.0, np.float64(np.float32(1e-30))])
    gx = dev.zeros("f32", (5,))
    dev.relu_backward(x, gx, upload(dev, np.ones(5), "f32"))
    np.testing.assert_array_equal(host(dev, gx), [0.0, 0.0, 1.0, 0.0, 1.0])
