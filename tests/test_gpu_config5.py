"""Config 5: a transformer encoder block (d_model 1024, 16 heads, d_ff 4096, seq 512, batch 16; bf16 weights
~N(0, 0.02), inputs ~N(0, 1), f32 accumulate), full forward + backward with EVERY Linear and attention matmul
dispatched to the Rocm kernels through the kernel-trait entry points.

Each of those GEMM calls is checked, on its actual inputs, against the CPU oracle's driver for the same
trait call, to the stated tolerance (2e-3*sqrt(K)*max|a|*max|b| for bf16/f16).  The glue between the
GEMMs (bias, softmax, LayerNorm, ReLU, residuals) runs on the host -- the "Cpu-equivalent path".  A small
block is additionally run end to end on both backends and the final outputs / gradients compared."""
import numpy as np
import pytest

import oracle
from encoder_ref import OracleBackend, View, encoder_block, init_params, val
from helpers import rng, tolerance
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

ULP = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}


class RocmBackend:
    """Kernel-trait calls on the GPU; optionally every call is replayed on the oracle and compared."""

    def __init__(self, dev, dtype, check=False):
        self.dev, self.dtype, self.check, self.calls = dev, dtype, check, []
        self.oracle = OracleBackend(dtype)

    def _up(self, v):
        return self.dev.tensor(v.storage, self.dtype, v.shape, v.strides)

    def _compare(self, what, got, want, k, a, b, roundings=1):
        g, w = oracle.to_f64(got, self.dtype), oracle.to_f64(want, self.dtype)
        amax, bmax = float(np.abs(val(a, self.dtype)).max()), float(np.abs(val(b, self.dtype)).max())
        tol = tolerance(self.dtype, k, amax, bmax) + 2 * roundings * ULP[self.dtype] * float(np.abs(w).max())
        err = float(np.abs(g - w).max())
        assert np.all(np.isfinite(g)), what
        assert err <= tol, f"{what}: max|err| {err:.3e} > tol {tol:.3e} (K={k})"
        self.calls.append((what, err, tol))

    def forward(self, lhs, rhs):
        announce("config5 forward", lhs.shape, lhs.strides, rhs.shape, rhs.strides)
        out = self.dev.to_host(self.dev.forward(self._up(lhs), self._up(rhs)))
        if self.check:
            self._compare(f"fwd {lhs.shape}x{rhs.shape}", out, self.oracle.forward(lhs, rhs), lhs.shape[-1], lhs.storage, rhs.storage)
        return out

    def backward(self, lhs, grad_lhs, rhs, grad_rhs, grad_out):
        announce("config5 backward", lhs.shape, lhs.strides, rhs.shape, rhs.strides)
        dl, dr = self._up(lhs), self._up(rhs)
        dgl = self.dev.tensor(grad_lhs, self.dtype, lhs.shape, lhs.strides)
        dgr = self.dev.tensor(grad_rhs, self.dtype, rhs.shape, rhs.strides)
        dgo = self.dev.tensor(grad_out, self.dtype)
        self.dev.backward(dl, dgl, dr, dgr, dgo)
        gl, gr = self.dev.to_host(dgl), self.dev.to_host(dgr)
        if self.check:
            wl, wr = grad_lhs.copy(), grad_rhs.copy()
            self.oracle.backward(lhs, wl, rhs, wr, grad_out)
            m, n = lhs.shape[-2], rhs.shape[-1]
            shared = len(rhs.shape) == 2 and len(lhs.shape) == 3      # broadcast rhs: one accumulator for all batches
            batches = lhs.shape[0] if shared else 1
            self._compare(f"grad_lhs {lhs.shape}x{rhs.shape}", gl, wl, n, grad_out, rhs.storage)
            self._compare(f"grad_rhs {lhs.shape}x{rhs.shape}", gr, wr, m * batches, lhs.storage, grad_out, roundings=batches)
        grad_lhs[:] = gl
        grad_rhs[:] = gr


def test_small_encoder_block_matches_the_oracle_path_end_to_end():
    dev, g = device(), rng(5005)
    dtype, (B, S, d, H, ff) = "bf16", (2, 64, 128, 4, 256)
    p = init_params(g, d, ff, dtype)
    x = g.standard_normal((B * S, d)).astype(np.float32)
    gout = g.standard_normal((B * S, d)).astype(np.float32) / (B * S)
    out_o, grads_o, dx_o = encoder_block(OracleBackend(dtype), dtype, p, x, B, S, d, H, ff, gout)
    be = RocmBackend(dev, dtype, check=True)
    out_g, grads_g, dx_g = encoder_block(be, dtype, p, x, B, S, d, H, ff, gout)
    assert len(be.calls) == 6 + 2 + 2 * (6 + 2)          # 6 Linear + 2 attention matmuls, forward; two grads each backward
    # layer-normed output: O(1) values stored in bf16; a flipped rounding upstream moves a result by ~1 ulp
    assert np.abs(out_g - out_o).max() <= 16 * ULP[dtype] * np.abs(out_o).max()
    assert np.abs(dx_g - dx_o).max() <= 16 * ULP[dtype] * np.abs(dx_o).max() + 1e-12
    for name in grads_o:
        go, gg = val(grads_o[name], dtype), val(grads_g[name], dtype)
        assert np.abs(gg - go).max() <= 16 * ULP[dtype] * np.abs(go).max() + 1e-12, name


def test_config5_encoder_block_bf16_full_size():
    dev, g = device(), rng(5006)
    dtype, (B, S, d, H, ff) = "bf16", (16, 512, 1024, 16, 4096)
    p = init_params(g, d, ff, dtype)
    x = g.standard_normal((B * S, d)).astype(np.float32)
    gout = g.standard_normal((B * S, d)).astype(np.float32) / (B * S)
    be = RocmBackend(dev, dtype, check=True)
    out, grads, dx = encoder_block(be, dtype, p, x, B, S, d, H, ff, gout)
    assert len(be.calls) == 24
    worst = max(be.calls, key=lambda c: c[1] / c[2])
    print("config5 worst GEMM vs oracle:", worst)
    # the block ends in a LayerNorm with gamma = 1, beta = 0: rows have mean 0 and variance 1 (to bf16 accuracy)
    assert np.all(np.isfinite(out)) and np.all(np.isfinite(dx))
    assert np.abs(out.mean(axis=-1)).max() < 2e-2 and np.abs(out.var(axis=-1) - 1).max() < 5e-2
    # d(loss)/d(beta2) = column sums of gout; the weight gradients are non-trivial
    np.testing.assert_allclose(val(grads["be2"], dtype), gout.sum(axis=0), atol=2 ** -7 * np.abs(gout.sum(axis=0)).max())
    for name in ("wq", "wk", "wv", "wo", "w1", "w2"):
        assert np.abs(val(grads[name], dtype)).max() > 0
