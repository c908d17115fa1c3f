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


def _device_block(dev, dtype, p, d, H, ff):
    from dfdx_amd.encoder import EncoderBlock
    shapes = {"wq": (d, d), "wk": (d, d), "wv": (d, d), "wo": (d, d), "w1": (ff, d), "w2": (d, ff)}
    params = {n: dev.tensor(v, dtype, shapes.get(n, (v.size,))) for n, v in p.items()}
    return EncoderBlock(dev, dtype, d, H, ff, params)


def test_small_encoder_block_entirely_on_the_device():
    """The same block with EVERY op on the device (dfdx_amd/encoder.py: Linear with fused bias, the attention
    matmuls, softmax with the scale folded in, the copying reshape, residual adds, LayerNorm, ReLU and all their
    backward ops), against the host-glue + CPU-oracle path.  The device ops evaluate each formula in f32 and round
    once where the host path rounds after every numpy op, so results agree to a few ulp of the largest value."""
    dev, g = device(), rng(5005)
    dtype, (B, S, d, H, ff) = "bf16", (2, 64, 128, 4, 256)
    p = init_params(g, d, ff, dtype)
    for name in ("g1", "g2", "be1", "be2"):                       # non-trivial LayerNorm parameters
        p[name] = oracle.to_storage((val(p[name], dtype) + 0.1 * g.standard_normal(d)).astype(np.float32), dtype)
    x = g.standard_normal((B * S, d)).astype(np.float32)
    gout = g.standard_normal((B * S, d)).astype(np.float32) / (B * S)
    out_o, grads_o, dx_o = encoder_block(OracleBackend(dtype), dtype, p, x, B, S, d, H, ff, gout)
    announce("config5 on-device block", (B, S, d, H, ff))
    blk = _device_block(dev, dtype, p, d, H, ff)
    xd = dev.tensor(oracle.to_storage(x.reshape(-1), dtype), dtype, (B, S, d))
    out_v, saved = blk.forward(xd)
    grads_v, gx_v = blk.backward(saved, dev.tensor(oracle.to_storage(gout.reshape(-1), dtype), dtype, (B, S, d)))
    out_g = val(dev.to_host(out_v), dtype).reshape(B * S, d)
    assert np.abs(out_g - out_o).max() <= 16 * ULP[dtype] * np.abs(out_o).max()
    dx_g = val(dev.to_host(gx_v), dtype).reshape(B * S, d)
    assert np.abs(dx_g - dx_o).max() <= 24 * ULP[dtype] * np.abs(dx_o).max() + 1e-12
    for name in grads_o:
        go, gg = val(grads_o[name], dtype), val(dev.to_host(grads_v[name]), dtype)
        if name == "bk":   # a bias on the keys shifts every score of a row alike: its gradient is 0 up to rounding noise
            assert max(np.abs(go).max(), np.abs(gg).max()) <= 1e-2 * np.abs(val(grads_o["bq"], dtype)).max()
            continue
        # A pre-activation that rounds to the other side of 0 flips one ReLU derivative (the fused Linear bias rounds
        # once, the host path twice): about 0.3 % of the entries of the gradient behind the ReLU are then off by
        # their whole value, which is a few percent of its norm; everything else differs by rounding only.
        assert np.abs(gg - go).max() <= 48 * ULP[dtype] * np.abs(go).max() + 1e-12, name
        assert np.linalg.norm(gg - go) <= 6e-2 * np.linalg.norm(go) + 1e-12, name


def test_config5_encoder_block_on_the_device_full_size():
    """Full-size config 5 with every op on the device: invariants of the output and of the gradients that have
    closed forms (the host path at this size is covered GEMM by GEMM above)."""
    dev, g = device(), rng(5007)
    dtype, (B, S, d, H, ff) = "bf16", (16, 512, 1024, 16, 4096)
    p = init_params(g, d, ff, dtype)
    blk = _device_block(dev, dtype, p, d, H, ff)
    x = g.standard_normal((B * S, d)).astype(np.float32)
    gout = g.standard_normal((B * S, d)).astype(np.float32) / (B * S)
    announce("config5 on-device block, full size")
    out_v, saved = blk.forward(dev.tensor(oracle.to_storage(x.reshape(-1), dtype), dtype, (B, S, d)))
    gout_st = oracle.to_storage(gout.reshape(-1), dtype)
    grads, gx = blk.backward(saved, dev.tensor(gout_st, dtype, (B, S, d)))
    out = val(dev.to_host(out_v), dtype).reshape(B * S, d)
    assert np.all(np.isfinite(out)) and np.all(np.isfinite(val(dev.to_host(gx), dtype)))
    assert np.abs(out.mean(axis=-1)).max() < 2e-2 and np.abs(out.var(axis=-1) - 1).max() < 5e-2
    gsum = val(gout_st, dtype).reshape(B * S, d).sum(axis=0)
    np.testing.assert_allclose(val(dev.to_host(grads["be2"]), dtype), gsum, atol=2 ** -7 * np.abs(gsum).max())
    probs = val(dev.to_host(saved["probs"]), dtype).reshape(-1, S)
    assert np.abs(probs.sum(axis=-1) - 1).max() < 2e-2
    for name in ("wq", "wk", "wv", "wo", "w1", "w2", "g1", "b1"):
        assert np.abs(val(dev.to_host(grads[name]), dtype)).max() > 0, name
