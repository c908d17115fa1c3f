"""GPU parity of conv2d (unfold kernels + the library's batched GEMM) against the PyTorch-produced literals of
the reference's tests (conv2d/tests.rs) and the CPU restatement of cpu_kernel.rs on seeded inputs."""
import json
import os

import numpy as np
import pytest

import oracle
from oracle.conv2d import Conv2DOp, conv2d_backward, conv2d_forward
from helpers import assert_within, logical, rng
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
CONV = json.load(open(os.path.join(GOLD, "conv2d_literals.json")))
ULP = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}


def host(dev, view):
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


@pytest.mark.parametrize("case", CONV["cases"], ids=lambda c: c["name"])
def test_conv2d_literals(case):
    dev = device()
    announce("conv2d literal", case["name"])
    x, w = upload(dev, case["x"], "f32"), upload(dev, case["weight"], "f32")
    kw = dict(stride=case["stride"], padding=case["padding"], dilation=case["dilation"], groups=case["groups"])
    y = host(dev, dev.conv2d_forward(x, w, **kw))
    if "bias" in case:
        y = y + np.asarray(case["bias"]).reshape(-1, 1, 1)
    np.testing.assert_allclose(y, case["out"], rtol=0, atol=2e-6)
    gy = {"exp_mean": np.exp(y) / y.size, "mean": np.full(y.shape, 1.0 / y.size)}[case["loss"]]
    gx, gw = dev.zeros_like_storage(x), dev.zeros_like_storage(w)
    dev.conv2d_backward(x, gx, w, gw, upload(dev, gy, "f32"), **kw)
    np.testing.assert_allclose(host(dev, gx), case["grad_x"], rtol=0, atol=2e-6)
    np.testing.assert_allclose(host(dev, gw), case["grad_weight"], rtol=0, atol=2e-6)


CONFIGS = [
    # batch, chan_in, chan_out, h, w, kernel, stride, padding, dilation, groups
    (2, 4, 6, 7, 6, 3, 2, 1, 1, 2),
    (1, 3, 5, 9, 8, 2, 1, 2, 3, 1),
    (3, 6, 3, 5, 5, 1, 1, 0, 1, 3),
    (1, 5, 3, 7, 6, 2, 4, 3, 1, 1),
    (10, 3, 5, 28, 28, 6, 3, 2, 1, 1),     # the shape of the reference's batched test (conv2d/tests.rs:219-250)
    (2, 9, 15, 14, 14, 3, 1, 0, 1, 3),     # the shape of its grouped-slices test (:405-464)
    (4, 64, 64, 28, 28, 3, 1, 1, 1, 1),    # k = 576, n = 784: the MFMA kernels
    (2, 64, 128, 32, 32, 3, 2, 1, 1, 2),
    (3, 16, 24, 16, 16, 3, 1, 1, 1, 1),    # unit stride, output width a multiple of 8: forward without a patch matrix
    (2, 32, 32, 12, 24, 3, 1, 2, 2, 2),    # the same with dilation and groups
    (2, 8, 16, 12, 20, 5, 1, 0, 1, 1),     # the same, no padding, k = 200 (a k tail in the 64-wide steps)
    (2, 64, 64, 56, 56, 3, 1, 1, 1, 1),    # the same at a ResNet shape
    (2, 16, 16, 9, 28, 3, 1, 1, 1, 1),     # the same with rows of 28 pixels: windows that straddle two image rows
    (2, 8, 8, 5, 30, 3, 1, 0, 1, 1),       # output 3 x 28 = 84 pixels (n % 8 = 4), no padding
    (4, 64, 128, 8, 8, 1, 1, 0, 1, 1),     # 1x1 filters: the image / grad_out are the patch matrices, no gather
    (2, 64, 64, 16, 16, 1, 1, 0, 1, 2),    # the same with groups
    (4, 64, 64, 14, 14, 3, 1, 1, 1, 1),    # n = 196: rows padded to the vector width inside the patch buffer
    (2, 32, 48, 7, 7, 3, 1, 1, 1, 1),      # n = 49
    (2, 16, 32, 15, 13, 3, 2, 1, 1, 1),    # input 195 and output 56 positions: only the backward side is padded
    (3, 32, 64, 24, 40, 5, 1, 2, 2, 1),
    (2, 3, 64, 32, 32, 3, 1, 1, 1, 1),     # a first layer: C*K*K = 27, a contraction no 16-byte load can walk (window loads)
    (2, 3, 64, 30, 30, 3, 2, 1, 1, 1),     # the same through the patch matrix (stride 2), 15 x 15 = 225 output pixels
    (3, 128, 96, 20, 14, 3, 1, 1, 1, 1),   # image gradient on the band kernel (two blocks of 64 channels out of 3 chunks of 32), forward on the tiles
    (2, 64, 32, 9, 112, 3, 1, 1, 1, 1),    # the same with one chunk, rows of 112 pixels; H * W = 1008 is off the 64-element grid of the filter gradient
    (9, 20, 24, 6, 10, 5, 1, 2, 1, 1),     # small images as one product over the batch: 9 images (a group of 8 and one), channels off the workgroups' groups
    (3, 16, 16, 10, 10, 3, 1, 2, 2, 1),    # the same with dilation
    (5, 32, 32, 7, 7, 3, 1, 1, 1, 1),      # 7 x 7: rows of 49 padded to 56 / 64 inside the folded matrices; tiled filter transposes
    (2, 16, 32, 48, 48, 3, 2, 1, 1, 1),    # stride 2, 576 output positions: both gradients from the forward patch matrix (position-major gather), 2 x 2 cells
    (2, 8, 8, 17, 18, 3, 2, 2, 2, 1),      # the same with dilation 2 and an odd height (cells cut by the image's edge)
    (2, 4, 8, 23, 19, 3, 5, 1, 1, 1),      # stride 5: the per-pixel form of the gather
    (2, 3, 16, 70, 66, 7, 2, 3, 1, 1),     # a first layer (7 x 7, stride 2, 3 channels): patches gathered from image rows staged in LDS, several bands per plane
    (3, 6, 9, 20, 21, 4, 3, 2, 1, 3),      # stride 3, three groups, an even kernel
    (1, 64, 64, 4, 224, 3, 1, 1, 1, 1),    # rows of 224 pixels: the image gradient on the band kernel's wide-row form, the filter gradient over the patch matrix
    (2, 8, 8, 12, 14, 3, 1, 1, 1, 8),      # depthwise (one input channel per group): the direct kernels
    (3, 6, 12, 9, 11, 3, 2, 1, 1, 6),      # depthwise with a channel multiplier of 2, stride 2
    (2, 4, 4, 20, 18, 5, 1, 4, 2, 4),      # depthwise, 5 x 5, dilation 2; more than 256 positions per plane
    (5, 3, 3, 8, 9, 2, 1, 1, 1, 3),        # depthwise with a 2 x 2 kernel: the filter-gradient kernel for any kernel size
    (2, 6, 12, 11, 13, 3, 1, 1, 1, 6),     # depthwise 3 x 3 at unit stride, multiplier 2, a width off the quads: four pixels per thread
    (2, 4, 4, 9, 16, 3, 1, 0, 1, 4),       # the same without padding (output 7 x 14), and with padding 2 below
    (1, 4, 4, 6, 8, 3, 1, 2, 1, 4),
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: "x".join(map(str, c)))
def test_conv2d_seeded(cfg, dtype):
    dev, g = device(), rng(501)
    batch, cin, cout, h, w_, kernel, stride, padding, dilation, groups = cfg
    announce("conv2d", cfg, dtype)
    op = Conv2DOp.make(batch, cin, cout, h, w_, kernel, stride, padding, dilation, groups)
    kw = dict(stride=stride, padding=padding, dilation=dilation, groups=groups)
    x = upload(dev, g.standard_normal((batch, cin, h, w_)), dtype)
    w = upload(dev, g.standard_normal((cout, cin // groups, kernel, kernel)) / np.sqrt(cin // groups * kernel * kernel), dtype)
    y = dev.conv2d_forward(x, w, **kw)
    assert y.shape == (batch, cout, op.h_out, op.w_out)
    x_h, w_h = dev.to_host(x).reshape(-1), dev.to_host(w).reshape(-1)
    X, W = oracle.to_f64(x_h, dtype), oracle.to_f64(w_h, dtype)
    want = oracle.to_f64(conv2d_forward(dtype, op, x_h, w_h), dtype)
    kf = cin // groups * kernel * kernel
    assert_within(dtype, kf, host(dev, y).reshape(-1), want, X, W, extra=ULP[dtype] * float(np.abs(want).max()), what="out")
    go = upload(dev, g.standard_normal(y.shape), dtype)
    gx0, gw0 = upload(dev, g.standard_normal(x.shape), dtype), upload(dev, g.standard_normal(w.shape), dtype)
    gx, gw = dev.tensor(dev.to_host(gx0), dtype), dev.tensor(dev.to_host(gw0), dtype)
    dev.conv2d_backward(x, gx, w, gw, go, **kw)
    go_h = dev.to_host(go).reshape(-1)
    ogx, ogw = dev.to_host(gx0).reshape(-1).copy(), dev.to_host(gw0).reshape(-1).copy()
    conv2d_backward(dtype, op, x_h, ogx, w_h, ogw, go_h)
    GO = oracle.to_f64(go_h, dtype)
    wgx, wgw = oracle.to_f64(ogx, dtype), oracle.to_f64(ogw, dtype)
    assert_within(dtype, cout // groups * kernel * kernel, host(dev, gx).reshape(-1), wgx, GO, W,
                  extra=2 * ULP[dtype] * float(np.abs(wgx).max()), what="grad_img")
    # the restatement rounds the filter gradient to the element type after every image, the device once per chunk
    assert_within(dtype, batch * h * w_, host(dev, gw).reshape(-1), wgw, GO, X,
                  extra=(batch + 2) * ULP[dtype] * float(np.abs(wgw).max()), what="grad_filters")


# 3 x 3 filters at unit stride with padding 1, input channels in chunks of 32, output channels in blocks of 64, an even
# width and at least 128 pixels: the forward product runs on the kernel that keeps a band of the image in LDS and has no
# patch matrix in any form (conv3x3.hip).  Shapes: one and several channel chunks / output blocks, pixel blocks that end
# in the middle of a row or of the image (one partial block; 196, 200 and 280 pixels), H * W off the 8-pixel grid (the
# 8-byte store form), bands of 3 to 24 rows, an odd height, a width of 112 (four units of the band per thread).
BAND_CONFIGS = [(2, 32, 64, 16, 16), (1, 64, 64, 14, 14), (3, 96, 128, 20, 14), (2, 64, 64, 56, 56), (2, 128, 192, 28, 28),
                (1, 32, 64, 9, 112), (2, 64, 64, 31, 12), (1, 64, 64, 112, 112), (5, 32, 64, 8, 16), (2, 32, 64, 50, 4),
                (1, 32, 64, 6, 224), (1, 32, 64, 3, 254)]   # (the last two: rows so wide that a thread owns five or six units of a band)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("cfg", BAND_CONFIGS, ids=lambda c: "x".join(map(str, c)))
def test_conv2d_3x3_forward_from_a_band_in_lds(cfg, dtype):
    dev, g = device(), rng(504)
    batch, cin, cout, h, w_ = cfg
    announce("conv2d 3x3 band kernel", cfg, dtype)
    op = Conv2DOp.make(batch, cin, cout, h, w_, 3, 1, 1, 1, 1)
    x = upload(dev, g.standard_normal((batch, cin, h, w_)), dtype)
    w = upload(dev, g.standard_normal((cout, cin, 3, 3)) / np.sqrt(cin * 9), dtype)
    y = dev.conv2d_forward(x, w, stride=1, padding=1)
    assert y.shape == (batch, cout, h, w_)
    x_h, w_h = dev.to_host(x).reshape(-1), dev.to_host(w).reshape(-1)
    want = oracle.to_f64(conv2d_forward(dtype, op, x_h, w_h), dtype)
    assert_within(dtype, cin * 9, host(dev, y).reshape(-1), want, oracle.to_f64(x_h, dtype), oracle.to_f64(w_h, dtype),
                  extra=ULP[dtype] * float(np.abs(want).max()), what="out")
    # the same call again gives the same bits (nothing in the kernel depends on timing)
    y2 = dev.conv2d_forward(x, w, stride=1, padding=1)
    np.testing.assert_array_equal(dev.to_host(y), dev.to_host(y2))


def test_conv2d_3x3_band_kernel_zero_padding_is_exact():
    """An image of ones against filters of ones: every output is the number of taps inside the image times the channel
    count -- 4 C in the corners, 6 C on the edges, 9 C inside -- exactly (small integers), whichever rows and columns a
    pixel block starts and ends on."""
    dev = device()
    batch, cin, cout, h, w_ = 2, 64, 64, 23, 18
    announce("conv2d 3x3 band kernel, ones", batch, cin, cout, h, w_)
    x = upload(dev, np.ones((batch, cin, h, w_)), "f16")
    w = upload(dev, np.ones((cout, cin, 3, 3)), "f16")
    got = host(dev, dev.conv2d_forward(x, w, stride=1, padding=1))
    ny = 3 - (np.arange(h) == 0) - (np.arange(h) == h - 1)
    nx = 3 - (np.arange(w_) == 0) - (np.arange(w_) == w_ - 1)
    want = (ny[:, None] * nx[None, :] * cin).astype(np.float64)
    np.testing.assert_array_equal(got, np.broadcast_to(want, got.shape))


# Backward of the same family with whole blocks of 64 input and output channels and rows of at most 64 pixels: neither
# gradient goes through a patch matrix (image gradient: the band kernel with the filters turned; filter gradient:
# conv3x3_wgrad.hip).  Shapes: several channel blocks on either side, bands that end below the image (H not a multiple of
# the rows per band), a grad_out band of exactly 256 records (62-pixel rows), one row per image, more work items than
# workgroups and fewer.
WGRAD_CONFIGS = [(2, 128, 64, 20, 14), (3, 64, 128, 9, 30), (1, 64, 64, 5, 62), (2, 64, 64, 1, 40), (70, 64, 64, 8, 8),
                 (2, 128, 128, 33, 12), (1, 64, 64, 6, 112), (2, 64, 64, 5, 84)]   # (the last two: rows too wide for as many per item as the band holds)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])   # (f32: channel-major bands, one value per lane and MFMA)
@pytest.mark.parametrize("cfg", WGRAD_CONFIGS, ids=lambda c: "x".join(map(str, c)))
def test_conv2d_3x3_backward_without_patch_matrix(cfg, dtype):
    dev, g = device(), rng(505)
    batch, cin, cout, h, w_ = cfg
    announce("conv2d 3x3 backward, no patch matrix", cfg, dtype)
    op = Conv2DOp.make(batch, cin, cout, h, w_, 3, 1, 1, 1, 1)
    x = upload(dev, g.standard_normal((batch, cin, h, w_)), dtype)
    w = upload(dev, g.standard_normal((cout, cin, 3, 3)) / np.sqrt(cin * 9), dtype)
    go = upload(dev, g.standard_normal((batch, cout, h, w_)), dtype)
    gx0, gw0 = upload(dev, g.standard_normal(x.shape), dtype), upload(dev, g.standard_normal(w.shape), dtype)
    outs = []
    for _ in range(2):   # twice: the same bits (the shares of the filter gradient are added in a fixed order)
        gx, gw = dev.tensor(dev.to_host(gx0), dtype), dev.tensor(dev.to_host(gw0), dtype)
        dev.conv2d_backward(x, gx, w, gw, go, stride=1, padding=1)
        outs.append((dev.to_host(gx), dev.to_host(gw)))
    np.testing.assert_array_equal(outs[0][0], outs[1][0])
    np.testing.assert_array_equal(outs[0][1], outs[1][1])
    x_h, w_h, go_h = dev.to_host(x).reshape(-1), dev.to_host(w).reshape(-1), dev.to_host(go).reshape(-1)
    ogx, ogw = dev.to_host(gx0).reshape(-1).copy(), dev.to_host(gw0).reshape(-1).copy()
    conv2d_backward(dtype, op, x_h, ogx, w_h, ogw, go_h)
    X, W, GO = oracle.to_f64(x_h, dtype), oracle.to_f64(w_h, dtype), oracle.to_f64(go_h, dtype)
    wgx, wgw = oracle.to_f64(ogx, dtype), oracle.to_f64(ogw, dtype)
    assert_within(dtype, cout * 9, oracle.to_f64(outs[0][0], dtype).reshape(-1), wgx, GO, W,
                  extra=2 * ULP[dtype] * float(np.abs(wgx).max()), what="grad_img")
    # the restatement rounds the filter gradient to the element type after every image, the device once
    assert_within(dtype, batch * h * w_, oracle.to_f64(outs[0][1], dtype).reshape(-1), wgw, GO, X,
                  extra=(batch + 2) * ULP[dtype] * float(np.abs(wgw).max()), what="grad_filters")


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_conv2d_3x3_filter_gradient_counts_pixels_exactly(dtype):
    """Images and output gradients of ones: the gradient of filter tap (ky, kx) is batch x the number of pixels whose
    neighbour at that tap lies inside the image -- (H - |ky - 1|) (W - |kx - 1|) -- exactly, for every channel pair."""
    dev = device()
    batch, cin, cout, h, w_ = 3, 64, 64, 11, 10
    announce("conv2d 3x3 filter gradient, ones", batch, cin, cout, h, w_, dtype)
    x = upload(dev, np.ones((batch, cin, h, w_)), dtype)
    w = upload(dev, np.zeros((cout, cin, 3, 3)), dtype)
    go = upload(dev, np.ones((batch, cout, h, w_)), dtype)
    gx, gw = dev.zeros(dtype, x.shape), dev.zeros(dtype, w.shape)
    dev.conv2d_backward(x, gx, w, gw, go, stride=1, padding=1)
    got = host(dev, gw)
    want = np.array([[batch * (h - abs(ky - 1)) * (w_ - abs(kx - 1)) for kx in range(3)] for ky in range(3)], dtype=np.float64)
    np.testing.assert_array_equal(got, np.broadcast_to(want, got.shape))
    np.testing.assert_array_equal(host(dev, gx), 0.0)   # zero filters: no image gradient


# one shape per form of the backward pass: band + filter-gradient kernels, band + patch matrix, folded small images,
# strided (cells of 2 x 2 and the per-pixel gather), few input channels, depthwise, 1 x 1, the general form with padded rows
DEFERRED_CONFIGS = [(2, 64, 64, 12, 14, 3, 1, 1, 1, 1), (1, 32, 64, 6, 224, 3, 1, 1, 1, 1), (5, 32, 32, 7, 7, 3, 1, 1, 1, 1),
                    (2, 16, 32, 48, 48, 3, 2, 1, 1, 1), (2, 4, 8, 23, 19, 3, 5, 1, 1, 1), (2, 3, 64, 32, 32, 3, 1, 1, 1, 1),
                    (2, 8, 8, 12, 14, 3, 1, 1, 1, 8), (2, 6, 6, 9, 10, 3, 2, 1, 1, 6), (4, 64, 128, 8, 8, 1, 1, 0, 1, 1), (2, 8, 16, 12, 20, 5, 1, 0, 1, 1),
                    (1, 5, 3, 7, 6, 2, 1, 3, 1, 1)]


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("cfg", DEFERRED_CONFIGS, ids=lambda c: "x".join(map(str, c)))
def test_conv2d_backward_into_gradients_declared_zero(cfg, dtype):
    """Gradient buffers whose zero fill is deferred: the image gradient is stored instead of added (or cleared first, where a
    form adds into a padded copy), the same bits as with buffers cleared beforehand; nothing stays pending afterwards."""
    dev, g = device(), rng(507)
    batch, cin, cout, h, w_, kernel, stride, padding, dilation, groups = cfg
    announce("conv2d backward, deferred zeros", cfg, dtype)
    kw = dict(stride=stride, padding=padding, dilation=dilation, groups=groups)
    x = upload(dev, g.standard_normal((batch, cin, h, w_)), dtype)
    w = upload(dev, g.standard_normal((cout, cin // groups, kernel, kernel)) / np.sqrt(cin // groups * kernel * kernel), dtype)
    go = upload(dev, g.standard_normal(dev.conv2d_forward(x, w, **kw).shape), dtype)
    gx0, gw0 = dev.zeros(dtype, x.shape), dev.zeros(dtype, w.shape)
    dev.conv2d_backward(x, gx0, w, gw0, go, **kw)
    gx1, gw1 = dev.zeros_many([x, w], deferred=True)
    dev.conv2d_backward(x, gx1, w, gw1, go, **kw)
    np.testing.assert_array_equal(dev.to_host(gx1), dev.to_host(gx0))
    np.testing.assert_array_equal(dev.to_host(gw1), dev.to_host(gw0))
    # a second call accumulates: twice the gradient, within a rounding of the element type
    dev.conv2d_backward(x, gx1, w, gw1, go, **kw)
    once, twice = host(dev, gx0), host(dev, gx1)
    assert np.abs(twice - 2 * once).max() <= 4 * ULP.get(dtype, 2.0 ** -23) * (np.abs(once).max() + 1.0)


def test_conv2d_unbatched_equals_batch_of_one():
    dev, g = device(), rng(502)
    announce("conv2d unbatched")
    x3 = upload(dev, g.standard_normal((3, 12, 12)), "f32")
    w = upload(dev, g.standard_normal((4, 3, 3, 3)), "f32")
    y3 = dev.conv2d_forward(x3, w, padding=1)
    x4 = dev.tensor(dev.to_host(x3).reshape(1, 3, 12, 12), "f32")
    y4 = dev.conv2d_forward(x4, w, padding=1)
    assert y3.shape == (4, 12, 12) and y4.shape == (1, 4, 12, 12)
    np.testing.assert_array_equal(host(dev, y3), host(dev, y4)[0])


def test_conv2d_shape_checks():
    dev = device()
    x = dev.zeros("f32", (1, 4, 8, 8))
    with pytest.raises(AssertionError, match="left: 4\n right: 6"):
        dev.conv2d_forward(x, dev.zeros("f32", (2, 3, 3, 3)), groups=2)
    with pytest.raises(ValueError, match="must be contiguous"):
        dev.conv2d_forward(x.permute(0, 1, 3, 2), dev.zeros("f32", (2, 4, 3, 3)))


def test_conv2d_batch_larger_than_one_patch_chunk():
    """A batch whose unfolded patches exceed the per-launch patch budget is processed in several chunks; every
    chunk boundary must be seamless (outputs of all images, gradients summed over all of them)."""
    dev, g = device(), rng(503)
    dtype, (batch, c, h, w_) = "f16", (80, 64, 112, 112)
    announce("conv2d chunked batch", batch, c, h, w_)
    cout = 64  # forward patches 14.4 MB per image, backward patches the same: both exceed the budget at batch 80
    op = Conv2DOp.make(batch, c, cout, h, w_, 3, 1, 1, 1, 1)
    x = upload(dev, g.standard_normal((batch, c, h, w_)).astype(np.float32), dtype)
    w = upload(dev, g.standard_normal((cout, c, 3, 3)) / 24.0, dtype)
    y = dev.conv2d_forward(x, w, padding=1)
    go = upload(dev, g.standard_normal(y.shape).astype(np.float32), dtype)
    gx, gw = dev.zeros_like_storage(x), dev.zeros_like_storage(w)
    dev.conv2d_backward(x, gx, w, gw, go, padding=1)
    x_h, w_h, go_h = (dev.to_host(t).reshape(-1) for t in (x, w, go))
    y_h, gx_h = dev.to_host(y).reshape(batch, -1), dev.to_host(gx).reshape(batch, -1)
    op1 = Conv2DOp.make(1, c, cout, h, w_, 3, 1, 1, 1, 1)
    per_x, per_y = c * h * w_, cout * h * w_
    W = oracle.to_f64(w_h, dtype)
    gw_sum = np.zeros(w_h.size)
    for b in range(batch):
        xb, gob = x_h[b * per_x:(b + 1) * per_x], go_h[b * per_y:(b + 1) * per_y]
        ogx, ogw = np.zeros(per_x, np.float16), np.zeros(w_h.size, np.float32)
        if b in (0, 36, 37, 73, 74, 79):  # around the chunk boundaries
            want = oracle.to_f64(conv2d_forward(dtype, op1, xb, w_h), dtype)
            assert_within(dtype, c * 9, oracle.to_f64(y_h[b], dtype), want, oracle.to_f64(xb, dtype), W, extra=ULP[dtype] * 8, what=f"out[{b}]")
            conv2d_backward(dtype, op1, xb, ogx, w_h, np.zeros_like(w_h), gob)
            assert_within(dtype, cout * 9, oracle.to_f64(gx_h[b], dtype), oracle.to_f64(ogx, dtype), oracle.to_f64(gob, dtype), W, extra=ULP[dtype] * 8, what=f"grad_img[{b}]")
        # filter gradient in float32 per image (exact enough), summed in float64
        conv2d_backward("f32", op1, oracle.to_f64(xb, dtype).astype(np.float32), np.zeros(per_x, np.float32),
                        W.astype(np.float32), ogw, oracle.to_f64(gob, dtype).astype(np.float32))
        gw_sum += ogw
    got = oracle.to_f64(dev.to_host(gw).reshape(-1), dtype)
    tol = 2e-3 * np.sqrt(batch * h * w_) * 5.0 * 5.0
    assert float(np.abs(got - gw_sum).max()) <= tol + 4 * ULP[dtype] * float(np.abs(gw_sum).max())
