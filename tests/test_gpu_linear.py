"""GPU parity of the Linear / Bias1D entry points that sit on top of the matmul kernels: the bias add, its
backward (column sums of grad_out) and the combined Linear backward, against the reference's literals
(dfdx/src/nn/layers/linear.rs:97-204) and the CPU restatement."""
import json
import os

import numpy as np
import pytest

import oracle
from oracle import nn_ops
from helpers import TOL_COEF, logical, rng
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
LINEAR = json.load(open(os.path.join(GOLD, "linear_literals.json")))


def host(dev, view):
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("case", LINEAR["cases"], ids=lambda c: c["name"])
def test_linear_backward_literals(case, dtype):
    """y, dW and db of the reference's Linear tests through linear_forward / linear_backward."""
    dev = device()
    announce("linear backward literal", case["name"], dtype)
    tol = 1e-6 if dtype == "f32" else 2e-3
    w, bias, x = upload(dev, LINEAR["weight"], dtype), upload(dev, LINEAR["bias"], dtype), upload(dev, case["x"], dtype)
    y = host(dev, dev.linear_forward(x, w, bias))
    np.testing.assert_allclose(y, case["y"], rtol=0, atol=tol)
    gy = upload(dev, 2.0 * y / y.size, dtype)  # loss = square().mean()
    gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros_like_storage(bias)
    dev.linear_backward(x, gx, w, gw, gb, gy)
    np.testing.assert_allclose(host(dev, gw), case["grad_weight"], rtol=0, atol=tol)
    np.testing.assert_allclose(host(dev, gb), case["grad_bias"], rtol=0, atol=tol)
    np.testing.assert_allclose(host(dev, gx), host(dev, gy) @ host(dev, w), rtol=0, atol=tol)


SHAPES = [(1, 1), (3, 5), (7, 8), (64, 256), (33, 1000), (1000, 1023), (4099, 264), (8192, 4096), (16384, 1024), (200000, 8)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_forward(shape, dtype):
    """One add in the element type per output: bit-exact against the restatement."""
    dev, g = device(), rng(301)
    rows, cols = shape
    announce("bias forward", shape, dtype)
    x, b = upload(dev, g.standard_normal((rows, cols)), dtype), upload(dev, g.standard_normal(cols), dtype)
    got = host(dev, dev.bias_forward(x, b))
    np.testing.assert_array_equal(got, nn_ops.bias_forward(host(dev, x), host(dev, b), dtype))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_backward(shape, dtype):
    """Column sums accumulated into grad_bias: within the summation tolerance of the exact (float64) sums, the same
    bits on every run, and -- where the reference's row-after-row rounding is still harmless -- equal to it."""
    dev, g = device(), rng(302)
    rows, cols = shape
    announce("bias backward", shape, dtype)
    go = upload(dev, g.standard_normal((rows, cols)), dtype)
    gb0 = upload(dev, g.standard_normal(cols), dtype)
    gb = dev.tensor(dev.to_host(gb0), dtype)
    dev.bias_backward(go, gb)
    got = host(dev, gb)
    go64, gb64 = host(dev, go), host(dev, gb0)
    exact = gb64 + go64.sum(axis=0)
    amax = float(np.abs(go64).max())
    # accumulation error bound + one rounding of the result to the storage type
    eps = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}[dtype]
    tol = TOL_COEF["f32"] * np.sqrt(rows) * amax + eps * float(np.abs(exact).max())
    err = float(np.abs(got - exact).max())
    assert err <= tol, f"max|err| {err:.3e} > {tol:.3e}"
    gb2 = dev.tensor(dev.to_host(gb0), dtype)
    dev.bias_backward(go, gb2)
    np.testing.assert_array_equal(host(dev, gb2), got)
    if rows <= 8 and dtype == "f32":
        np.testing.assert_allclose(got, nn_ops.bias_backward(go64, gb64, dtype, faithful=True), rtol=0, atol=4 * eps * (rows + 1) * amax)


def test_bias_backward_small_integers_exact():
    """Integer-valued inputs whose sums stay exactly representable: every dtype must return them bit-exactly."""
    dev, g = device(), rng(303)
    for dtype, rows in (("f32", 5000), ("f16", 300), ("bf16", 60)):
        announce("bias backward exact", dtype, rows)
        go = g.integers(-3, 4, size=(rows, 72)).astype(np.float64)
        gb = upload(dev, np.arange(72) % 5, dtype)
        dev.bias_backward(upload(dev, go, dtype), gb)
        np.testing.assert_array_equal(host(dev, gb), (np.arange(72) % 5) + go.sum(axis=0))


@pytest.mark.parametrize("dtype,rows,i,o", [("f32", 64, 512, 256), ("f16", 2048, 1024, 1024), ("bf16", 1000, 264, 136)])
def test_linear_backward_seeded(dtype, rows, i, o):
    """Config-1-shaped Linear (x[64,512], W(256,512), f32) and two larger ones: all three gradients against the
    oracle's MatMat backward on the permuted weight view plus the exact column sums."""
    from helpers import assert_within
    dev, g = device(), rng(304)
    announce("linear backward seeded", dtype, rows, i, o)
    x = upload(dev, g.standard_normal((rows, i)), dtype)
    w = upload(dev, g.uniform(-1, 1, (o, i)) / np.sqrt(i), dtype)
    go = upload(dev, g.standard_normal((rows, o)), dtype)
    gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros(dtype, (o,))
    dev.linear_backward(x, gx, w, gw, gb, go)
    xs, ws_, gos = dev.to_host(x), dev.to_host(w), dev.to_host(go)
    ogx, ogw = np.zeros_like(xs), np.zeros_like(ws_)
    oracle.matmat_backward(dtype, rows, i, o, xs, (i, 1), ogx, ws_, (1, i), ogw, gos)
    x64, w64, go64 = host(dev, x), host(dev, w), host(dev, go)
    assert_within(dtype, o, host(dev, gx), oracle.to_f64(ogx, dtype).reshape(rows, i), go64, w64, what="grad_x")
    assert_within(dtype, rows, host(dev, gw), oracle.to_f64(ogw, dtype).reshape(o, i), go64, x64, what="grad_weight")
    assert_within(dtype, rows, host(dev, gb), go64.sum(axis=0), go64, np.ones(1), what="grad_bias")


# Shapes whose weight-gradient product x^T . grad_out runs on the LDS-DMA kernels (rows % 64 == 0, 16-bit): there the bias
# gradient is produced by the same launch (one more MFMA per A fragment in the work items of tile column 0) instead of
# by the reduction kernels.  Both tile families, split and unsplit contractions, edge tiles in either direction.
FUSED_SHAPES = [(8192, 1024, 1024), (4096, 1024, 4096), (512, 256, 512), (640, 264, 1000), (128, 64, 8), (2048, 4096, 1024),
                (64, 1024, 1024), (2048, 128, 256), (4096, 128, 256), (4096, 256, 4096), (8192, 1024, 4096)]


def test_fused_shapes_reach_every_tile_family_that_sums_rows():
    """The weight-gradient products of FUSED_SHAPES are planned on all four LDS-DMA tiles that can carry the row sums
    (the 256 x 64 tile serves outputs of at most 64 columns: too few tile columns to share an A tile)."""
    dev = device()
    seen = set()
    probe = dev.zeros("f16", (16,))
    for rows, i, o in FUSED_SHAPES:
        d = dev.gemm_desc("f16", i, rows, o, probe.ptr, (1, i), probe.ptr, (o, 1), probe.ptr, (1, i), accumulate=True)
        name = dev.gemm_plan(d)[2]
        if "_dma_" in name and "splitk" in name:
            seen.add(name.split("_dma_")[1].split("x64_")[0])
    assert {"256x256", "256x128", "128x128", "128x64"} <= seen, seen


# f32: the k-sliced small kernel produces the row sums (config 1's Linear and smaller)
FUSED_F32 = [("f32", 64, 512, 256), ("f32", 100, 40, 24), ("f32", 17, 33, 9), ("f32", 300, 16, 130), ("f32", 12, 2048, 1024)]
# the small-product kernel in the other element types (its row sums come from the tile column 0 workgroups)
FUSED_SMALL = [(d, *shape) for d in ("f16", "bf16", "f64") for shape in ((64, 512, 256), (100, 40, 24), (17, 33, 9), (300, 16, 130),
                                                                             (24, 2048, 1024))]   # (a handful of rows, a large weight: the thin-contraction kernel, row sums apart)


@pytest.mark.parametrize("dtype,rows,i,o", [(d, *shape) for d in ("f16", "bf16") for shape in FUSED_SHAPES] + FUSED_F32 + FUSED_SMALL)
def test_linear_backward_bias_gradient_from_the_weight_gradient_launch(dtype, rows, i, o):
    """grad_bias: exact on small integers (sums below 2^8 for bf16, 2^11 for f16 are representable), and twice the
    value after a second call (the first call finds the gradient fresh when its zeros are deferred, the second adds)."""
    from helpers import assert_within
    dev, g = device(), rng(305)
    announce("linear backward, fused bias gradient", dtype, rows, i, o)
    x = upload(dev, g.standard_normal((rows, i)), dtype)
    w = upload(dev, g.uniform(-1, 1, (o, i)) / np.sqrt(i), dtype)
    # mostly zeros, a few +-1: column sums stay small integers whatever the number of rows
    go_host = (g.random((rows, o)) < 4.0 / rows) * g.choice([-1.0, 1.0], size=(rows, o))
    go_host[0, :] += np.arange(o) % 3
    go = upload(dev, go_host, dtype)
    start = (np.arange(o) % 4).astype(np.float64)
    for deferred in (False, True):
        gx, gw = dev.zeros_like_storage(x), dev.zeros_like_storage(w)
        if deferred:   # NaN patterns that are only DECLARED zero: a read of the old contents would show
            import torch
            from dfdx_amd.rocm import View
            es = {"f64": 8, "f32": 4}.get(dtype, 2)
            raw = torch.full((o * es,), 0xFF, dtype=torch.uint8, device="cuda")
            dev.zero_deferred(raw.data_ptr(), o * es)
            gb, base = View(raw, dtype, (o,), (1,)), np.zeros(o)
        else:
            gb, base = upload(dev, start, dtype), start
        dev.linear_backward(x, gx, w, gw, gb, go)
        np.testing.assert_array_equal(host(dev, gb), base + go_host.sum(axis=0))
        dev.linear_backward(x, gx, w, gw, gb, go)
        np.testing.assert_array_equal(host(dev, gb), base + 2 * go_host.sum(axis=0))
    # the products themselves are unchanged by the extra result
    xs, ws_, gos = dev.to_host(x), dev.to_host(w), dev.to_host(go)
    gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros(dtype, (o,))
    dev.linear_backward(x, gx, w, gw, gb, go)
    gx2, gw2 = dev.zeros_like_storage(x), dev.zeros_like_storage(w)
    dev.linear_backward(x, gx2, w, gw2, None, go)
    assert np.array_equal(dev.to_host(gw).view(np.uint8), dev.to_host(gw2).view(np.uint8))
    assert np.array_equal(dev.to_host(gx).view(np.uint8), dev.to_host(gx2).view(np.uint8))
    ogx, ogw = np.zeros_like(xs), np.zeros_like(ws_)
    oracle.matmat_backward(dtype, rows, i, o, xs, (i, 1), ogx, ws_, (1, i), ogw, gos)
    assert_within(dtype, rows, host(dev, gw), oracle.to_f64(ogw, dtype).reshape(o, i), host(dev, go), host(dev, x), what="grad_weight")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_linear_backward_fused_bias_gradient_random(dtype):
    """Random grad_out: against the f64 column sums within the tolerance of one f32-accumulated reduction."""
    from helpers import assert_within
    dev, g = device(), rng(306)
    for rows, i, o in ((8192, 1024, 1024), (1024, 512, 2048), (640, 264, 1000)):
        announce("linear backward, fused bias gradient, random", dtype, rows, i, o)
        x = upload(dev, g.standard_normal((rows, i)), dtype)
        w = upload(dev, g.uniform(-1, 1, (o, i)) / np.sqrt(i), dtype)
        go = upload(dev, g.standard_normal((rows, o)), dtype)
        gx, gw, gb = dev.zeros_like_storage(x), dev.zeros_like_storage(w), dev.zeros(dtype, (o,))
        dev.linear_backward(x, gx, w, gw, gb, go)
        go64 = host(dev, go)
        assert_within(dtype, rows, host(dev, gb), go64.sum(axis=0), go64, np.ones(1), what="grad_bias")
