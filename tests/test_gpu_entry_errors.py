"""Error behaviour of the entry points around the matmuls, through the C ABI on a live context: bad arguments
come back as negative codes (never a launch), empty problems are accepted and do nothing."""
import ctypes

import numpy as np
import pytest

from gpu_util import announce, device

pytestmark = pytest.mark.gpu

I64, VP, F32, F64 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_double
INVALID, UNSUPPORTED, ALIASED = -1, -2, -4


def arr(values):
    return (ctypes.c_int64 * len(values))(*values)


def test_bias_and_softmax_argument_checks():
    dev = device()
    lib, ctx = dev.lib, dev.ctx
    announce("bias / softmax / scalar-mul argument checks")
    buf = dev.zeros("f32", (64,))
    p = VP(buf.ptr)
    assert lib.dfdx_rocm_bias_forward(ctx, 0, I64(-1), I64(4), p, p, p) == INVALID
    assert lib.dfdx_rocm_bias_forward(ctx, 0, I64(4), I64(4), VP(), p, p) == INVALID
    assert lib.dfdx_rocm_bias_forward(ctx, 3, I64(2), I64(2), p, p, p) == 0                # f64 is served (Linear needs it)
    assert lib.dfdx_rocm_bias_forward(ctx, 9, I64(4), I64(4), p, p, p) == UNSUPPORTED      # no such element type
    assert lib.dfdx_rocm_bias_forward(ctx, 0, I64(0), I64(4), VP(), VP(), VP()) == 0        # empty: nothing to do
    assert lib.dfdx_rocm_bias_backward(ctx, 0, I64(4), I64(1 << 31), p, p) == INVALID
    assert lib.dfdx_rocm_bias_backward(ctx, 0, I64(4), I64(0), VP(), VP()) == 0
    assert lib.dfdx_rocm_softmax_forward(ctx, 0, I64(2), I64(-3), p, F32(1.0), p) == INVALID
    assert lib.dfdx_rocm_softmax_forward(ctx, 9, I64(2), I64(3), p, F32(1.0), p) == UNSUPPORTED
    assert lib.dfdx_rocm_softmax_backward(ctx, 0, I64(2), I64(3), p, F32(1.0), p, VP()) == INVALID
    assert lib.dfdx_rocm_softmax_forward(ctx, 0, I64(0), I64(3), VP(), F32(1.0), VP()) == 0
    assert lib.dfdx_rocm_scalar_mul_forward(ctx, 0, I64(-1), p, F64(2.0), p) == INVALID
    assert lib.dfdx_rocm_scalar_mul_backward(ctx, 0, I64(4), F64(2.0), VP(), p) == INVALID
    assert lib.dfdx_rocm_scalar_mul_forward(ctx, 0, I64(0), VP(), F64(2.0), VP()) == 0
    dev.synchronize()
    assert np.all(dev.to_host(buf) == 0)


def test_reshape_argument_checks():
    dev = device()
    lib, ctx = dev.lib, dev.ctx
    announce("reshape argument checks")
    buf = dev.zeros("f32", (64,))
    p = VP(buf.ptr)
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 7, arr([1] * 7), arr([1] * 7), p, p) == INVALID   # rank <= 6
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 2, arr([2, -3]), arr([3, 1]), p, p) == INVALID
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 2, arr([2, 3]), arr([3, -1]), p, p) == INVALID
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 2, arr([2, 3]), arr([3, 1]), VP(), p) == INVALID
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 2, arr([0, 3]), arr([3, 1]), VP(), VP()) == 0
    assert lib.dfdx_rocm_reshape_backward(ctx, 0, 2, arr([2, 3]), arr([0, 1]), p, p) == 0   # a broadcast axis is summed over
    assert lib.dfdx_rocm_reshape_forward(ctx, 0, 0, None, None, p, p) == 0                        # rank 0: one element
    dev.synchronize()


def test_conv2d_argument_checks():
    from dfdx_amd.rocm import Conv2DOp
    dev = device()
    lib, ctx = dev.lib, dev.ctx
    announce("conv2d argument checks")
    buf = dev.zeros("f32", (4096,))
    p = VP(buf.ptr)
    good = Conv2DOp(3, 1, 1, 1, 1, 1, 2, 2, 8, 8, 8, 8)
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, ctypes.byref(good), p, p, VP()) == INVALID
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, None, p, p, p) == INVALID
    bad_out = Conv2DOp(3, 1, 1, 1, 1, 1, 2, 2, 8, 7, 8, 8)          # h_out does not follow from h_in
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, ctypes.byref(bad_out), p, p, p) == INVALID
    bad_groups = Conv2DOp(3, 1, 1, 1, 3, 1, 2, 2, 8, 8, 8, 8)        # channels not divisible by groups
    assert lib.dfdx_rocm_conv2d_backward(ctx, 0, ctypes.byref(bad_groups), p, p, p, p, p) == INVALID
    zero_stride = Conv2DOp(3, 0, 1, 1, 1, 1, 2, 2, 8, 8, 8, 8)
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, ctypes.byref(zero_stride), p, p, p) == INVALID
    too_big_kernel = Conv2DOp(9, 1, 0, 1, 1, 1, 2, 2, 8, 0, 8, 0)
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, ctypes.byref(too_big_kernel), p, p, p) == INVALID
    assert lib.dfdx_rocm_conv2d_forward(ctx, 3, ctypes.byref(good), p, p, p) == UNSUPPORTED
    empty = Conv2DOp(3, 1, 1, 1, 1, 0, 2, 2, 8, 8, 8, 8)
    assert lib.dfdx_rocm_conv2d_forward(ctx, 0, ctypes.byref(empty), VP(), VP(), VP()) == 0
    dev.synchronize()
    assert np.all(dev.to_host(buf) == 0)


def test_linear_backward_without_bias_gradient():
    """grad_bias may be NULL (a Linear without a trainable bias): the two products still run."""
    dev = device()
    announce("linear backward, no grad_bias")
    x, w, go = dev.zeros("f32", (4, 8)), dev.zeros("f32", (3, 8)), dev.zeros("f32", (4, 3))
    gx, gw = dev.zeros("f32", (4, 8)), dev.zeros("f32", (3, 8))
    dev.linear_backward(x, gx, w, gw, None, go)
    dev.synchronize()


def test_layer_norm_relu_add_argument_checks():
    dev = device()
    lib, ctx = dev.lib, dev.ctx
    announce("layer norm / relu / add argument checks")
    buf = dev.zeros("f32", (64,))
    p = VP(buf.ptr)
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 0, I64(-1), I64(4), p, p, p, F64(1e-5), p) == INVALID
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 0, I64(2), I64(1 << 24), p, p, p, F64(1e-5), p) == INVALID
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 0, I64(2), I64(4), p, VP(), p, F64(1e-5), p) == INVALID
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 3, I64(2), I64(4), p, p, p, F64(1e-5), p) == 0             # f64 is served
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 9, I64(2), I64(4), p, p, p, F64(1e-5), p) == UNSUPPORTED   # no such element type
    assert lib.dfdx_rocm_layer_norm_forward(ctx, 0, I64(0), I64(4), VP(), VP(), VP(), F64(1e-5), VP()) == 0
    assert lib.dfdx_rocm_layer_norm_backward(ctx, 0, I64(2), I64(4), p, p, F64(1e-5), p, p, VP(), p) == INVALID
    assert lib.dfdx_rocm_layer_norm_backward(ctx, 0, I64(2), I64(0), VP(), VP(), F64(1e-5), VP(), VP(), VP(), VP()) == 0
    assert lib.dfdx_rocm_relu_forward(ctx, 0, I64(-1), p, p) == INVALID
    assert lib.dfdx_rocm_relu_forward(ctx, 0, I64(4), VP(), p) == INVALID
    assert lib.dfdx_rocm_relu_forward(ctx, 3, I64(4), p, p) == 0
    assert lib.dfdx_rocm_relu_forward(ctx, 9, I64(4), p, p) == UNSUPPORTED
    assert lib.dfdx_rocm_relu_backward(ctx, 0, I64(4), p, p, VP()) == INVALID
    assert lib.dfdx_rocm_relu_forward(ctx, 0, I64(0), VP(), VP()) == 0
    assert lib.dfdx_rocm_add_forward(ctx, 0, I64(4), p, VP(), p) == INVALID
    assert lib.dfdx_rocm_add_backward(ctx, 0, I64(4), p, VP(), p) == INVALID
    assert lib.dfdx_rocm_add_backward(ctx, 0, I64(4), VP(), VP(), p) == INVALID
    assert lib.dfdx_rocm_add_forward(ctx, 0, I64(0), VP(), VP(), VP()) == 0
    dev.synchronize()
    assert np.all(dev.to_host(buf) == 0)
