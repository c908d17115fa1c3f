"""Host-side restatement of the callers of the matmul path: Linear, MultiHeadAttention and the
transformer encoder block, forward and backward, with every matrix product delegated to a `backend`.

Only the GEMMs are the product under test; everything else here is the "Cpu-equivalent glue" the
benchmark configurations name, restated from the reference in numpy (float32 math, results rounded to
the storage dtype after every op, as a dfdx tensor of that dtype would be):

  Linear            dfdx/src/nn/layers/linear.rs:82-89       y = x . W^T (zero-copy permuted weight view) + bias
  Bias1D            dfdx/src/nn/layers/bias1d.rs:62-78       broadcast add; db = sum over rows
  MultiHeadAttention dfdx/src/nn/layers/multi_head_attention.rs:105-146
  softmax           dfdx-core/src/tensor_ops/softmax.rs:70-83   exp(x - max) / sum
  LayerNorm1D       dfdx/src/nn/layers/layer_norm1d.rs:87-91 over normalize.rs:35-49 (population variance, eps 1e-5)
  ReLU              dfdx-core/src/tensor_ops/relu/cpu_kernel.rs:7-16
  ResidualAdd       dfdx/src/nn/layers/residual_add.rs:42-45
  EncoderBlock      dfdx/src/nn/layers/transformer.rs:24-48  (ResidualAdd<MHA>, LN, ResidualAdd<(Linear, ReLU, Linear)>, LN)

A backend implements
    forward(lhs, rhs) -> out                      (flat storage array of the output dtype)
    backward(lhs, grad_lhs, rhs, grad_rhs, grad_out)   (accumulates into the flat grad storages)
where lhs / rhs are (storage, shape, strides) views exactly as the kernel traits receive them.
"""
from __future__ import annotations

import numpy as np

import oracle
from helpers import row_major_strides


def wt(dtype: str):
    """The numpy type the glue computes in: float32, or float64 for f64 tensors."""
    return np.float64 if dtype == "f64" else np.float32


def rt(x32: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 values to the storage dtype and back (what storing into a tensor of that dtype does)."""
    if dtype == "f64":
        return np.asarray(x32, dtype=np.float64)
    if dtype == "f32":
        return x32.astype(np.float32)
    if dtype == "f16":
        return x32.astype(np.float16).astype(np.float32)
    return oracle.bf16_to_f32(oracle.f32_to_bf16(np.ascontiguousarray(x32, dtype=np.float32)))


def st(x32: np.ndarray, dtype: str) -> np.ndarray:
    """float32 values -> flat storage array."""
    return oracle.to_storage(np.ascontiguousarray(x32, dtype=wt(dtype)).reshape(-1), dtype)


def val(storage: np.ndarray, dtype: str) -> np.ndarray:
    return oracle.to_f64(storage, dtype).astype(wt(dtype))


class View:
    def __init__(self, storage, shape, strides=None):
        self.storage, self.shape = storage, tuple(shape)
        self.strides = tuple(row_major_strides(shape)) if strides is None else tuple(strides)

    def permute(self, *axes):
        return View(self.storage, [self.shape[a] for a in axes], [self.strides[a] for a in axes])


class OracleBackend:
    """dfdx's Cpu kernels, restated (oracle/)."""

    def __init__(self, dtype):
        self.dtype = dtype

    def _fns(self, lhs, rhs):
        L, R = len(lhs.shape), len(rhs.shape)
        if L == 2 and R == 2:
            return oracle.matmat_forward, oracle.matmat_backward, lhs.shape + rhs.shape[-1:]
        if L == 3 and R == 2:
            return oracle.matmat_br_forward, oracle.matmat_br_backward, lhs.shape + rhs.shape[-1:]
        if L == 3 and R == 3:
            return oracle.matmat_batch3_forward, oracle.matmat_batch3_backward, lhs.shape + rhs.shape[-1:]
        return oracle.matmat_batch4_forward, oracle.matmat_batch4_backward, lhs.shape + rhs.shape[-1:]

    def forward(self, lhs, rhs):
        fwd, _, dims = self._fns(lhs, rhs)
        return fwd(self.dtype, *dims, lhs.storage, lhs.strides, rhs.storage, rhs.strides)

    def backward(self, lhs, grad_lhs, rhs, grad_rhs, grad_out):
        _, bwd, dims = self._fns(lhs, rhs)
        bwd(self.dtype, *dims, lhs.storage, lhs.strides, grad_lhs, rhs.storage, rhs.strides, grad_rhs, grad_out)


def linear_fwd(be, dtype, x: View, w: np.ndarray, b: np.ndarray, o: int, i: int):
    """x (..., I) -> (..., O).  Returns flat storage of y."""
    y = val(be.forward(x, View(w, (i, o), (1, i))), dtype).reshape(-1, o)
    return st(rt(y + val(b, dtype)[None, :], dtype), dtype)


def linear_bwd(be, dtype, x: View, gx, w, gw, gb, gy_storage, o: int, i: int):
    be.backward(x, gx, View(w, (i, o), (1, i)), gw, gy_storage)
    g = val(gy_storage, dtype).reshape(-1, o)
    gb[:] = st(rt(val(gb, dtype) + rt(g.sum(axis=0, dtype=g.dtype), dtype), dtype), dtype)


def softmax_fwd(x, dtype):
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return rt(e / e.sum(axis=-1, keepdims=True, dtype=e.dtype), dtype)


def softmax_bwd(p, gp):
    return p * (gp - (gp * p).sum(axis=-1, keepdims=True, dtype=p.dtype))


def layernorm_fwd(x, gamma, beta, dtype, eps=1e-5):
    mean = x.mean(axis=-1, keepdims=True, dtype=x.dtype)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True, dtype=x.dtype)
    inv = 1.0 / np.sqrt(var + x.dtype.type(eps))
    xhat = (x - mean) * inv
    return rt(xhat * gamma + beta, dtype), (xhat, inv)


def layernorm_bwd(gy, gamma, cache):
    xhat, inv = cache
    g = gy * gamma
    n = xhat.shape[-1]
    t = xhat.dtype
    gx = inv * (g - g.mean(axis=-1, keepdims=True, dtype=t) - xhat * (g * xhat).mean(axis=-1, keepdims=True, dtype=t))
    return gx, (gy * xhat).reshape(-1, n).sum(axis=0, dtype=t), gy.reshape(-1, n).sum(axis=0, dtype=t)


PARAMS = ("wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "g1", "be1", "w1", "b1", "w2", "b2", "g2", "be2")


def init_params(g: np.random.Generator, d: int, ff: int, dtype: str, std: float = 0.02):
    p = {}
    for name, shape in (("wq", (d, d)), ("wk", (d, d)), ("wv", (d, d)), ("wo", (d, d)), ("w1", (ff, d)), ("w2", (d, ff))):
        p[name] = st(g.standard_normal(shape).astype(np.float32) * std, dtype)
    for name, n in (("bq", d), ("bk", d), ("bv", d), ("bo", d), ("b1", ff), ("b2", d)):
        p[name] = st(g.standard_normal(n).astype(np.float32) * std, dtype)
    for name in ("g1", "g2"):
        p[name] = st(np.ones(d, np.float32), dtype)
    for name in ("be1", "be2"):
        p[name] = st(np.zeros(d, np.float32), dtype)
    return p


def encoder_block(be, dtype, p, x32, B, S, d, H, ff, gout):
    """Forward + backward of one encoder block; `gout` (T, d) is d(loss)/d(out), e.g. R / T for the loss
    sum(out * R) / T.  (mean(out) itself is identically 0 after the final LayerNorm with beta = 0, and its
    gradient vanishes, so a random projection is used instead.)  Returns (out, grads dict, dx)."""
    D = d // H
    T = B * S
    z = lambda n: np.zeros(n, oracle.NP_DTYPES[dtype])
    x = st(x32, dtype)
    xv = View(x, (B, S, d))
    # ---- MultiHeadAttention (multi_head_attention.rs:123-145)
    q = linear_fwd(be, dtype, xv, p["wq"], p["bq"], d, d)
    k = linear_fwd(be, dtype, xv, p["wk"], p["bk"], d, d)
    v = linear_fwd(be, dtype, xv, p["wv"], p["bv"], d, d)
    qv = View(q, (B, S, H, D)).permute(0, 2, 1, 3)   # (B,H,S,D), head-interleaved strides
    kv = View(k, (B, S, H, D)).permute(0, 2, 3, 1)   # (B,H,D,S)
    vv = View(v, (B, S, H, D)).permute(0, 2, 1, 3)
    scores = be.forward(qv, kv)                                           # (B,H,S,S)
    scaled = rt(val(scores, dtype).reshape(B, H, S, S) * wt(dtype)(1.0 / np.sqrt(D)), dtype)
    probs = softmax_fwd(scaled, dtype)
    pst = st(probs, dtype)
    tokens = be.forward(View(pst, (B, H, S, S)), vv)                      # (B,H,S,D) contiguous
    tok = np.ascontiguousarray(val(tokens, dtype).reshape(B, H, S, D).transpose(0, 2, 1, 3)).reshape(T, d)  # permute + reshape copy
    tokst = st(tok, dtype)
    attn = linear_fwd(be, dtype, View(tokst, (B, S, d)), p["wo"], p["bo"], d, d)
    h1 = rt(val(attn, dtype).reshape(T, d) + val(x, dtype).reshape(T, d), dtype)                # ResidualAdd
    n1, c1 = layernorm_fwd(h1, val(p["g1"], dtype), val(p["be1"], dtype), dtype)
    n1st = st(n1, dtype)
    # ---- feed forward
    f1 = linear_fwd(be, dtype, View(n1st, (B, S, d)), p["w1"], p["b1"], ff, d)
    r1 = np.maximum(val(f1, dtype), 0).reshape(T, ff)
    r1st = st(r1, dtype)
    f2 = linear_fwd(be, dtype, View(r1st, (B, S, ff)), p["w2"], p["b2"], d, ff)
    h2 = rt(val(f2, dtype).reshape(T, d) + n1, dtype)
    out, c2 = layernorm_fwd(h2, val(p["g2"], dtype), val(p["be2"], dtype), dtype)

    # ---- backward
    grads = {name: z(p[name].size) for name in PARAMS}
    gh2, gg2, gbe2 = layernorm_bwd(rt(gout, dtype), val(p["g2"], dtype), c2)
    grads["g2"], grads["be2"] = st(rt(gg2, dtype), dtype), st(rt(gbe2, dtype), dtype)
    gh2 = rt(gh2, dtype)
    gf2 = st(gh2, dtype)                                      # into the FF branch
    gr1 = z(T * ff)
    linear_bwd(be, dtype, View(r1st, (B, S, ff)), gr1, p["w2"], grads["w2"], grads["b2"], gf2, d, ff)
    gf1 = st(rt(val(gr1, dtype).reshape(T, ff) * (r1 > 0), dtype), dtype)
    gn1 = z(T * d)
    linear_bwd(be, dtype, View(n1st, (B, S, d)), gn1, p["w1"], grads["w1"], grads["b1"], gf1, ff, d)
    gn1_tot = rt(val(gn1, dtype).reshape(T, d) + gh2, dtype)  # residual: both uses of n1
    gh1, gg1, gbe1 = layernorm_bwd(gn1_tot, val(p["g1"], dtype), c1)
    grads["g1"], grads["be1"] = st(rt(gg1, dtype), dtype), st(rt(gbe1, dtype), dtype)
    gh1 = rt(gh1, dtype)
    gattn = st(gh1, dtype)
    gtok = z(T * d)
    linear_bwd(be, dtype, View(tokst, (B, S, d)), gtok, p["wo"], grads["wo"], grads["bo"], gattn, d, d)
    gtokens = st(np.ascontiguousarray(val(gtok, dtype).reshape(B, S, H, D).transpose(0, 2, 1, 3)), dtype)  # reshape/permute backward
    gp, gv = z(B * H * S * S), z(T * d)
    be.backward(View(pst, (B, H, S, S)), gp, vv, gv, gtokens)
    gscaled = rt(softmax_bwd(probs, val(gp, dtype).reshape(B, H, S, S)), dtype)
    gscores = st(rt(gscaled * wt(dtype)(1.0 / np.sqrt(D)), dtype), dtype)
    gq, gk = z(T * d), z(T * d)
    be.backward(qv, gq, kv, gk, gscores)
    gx = z(T * d)                                             # x feeds three Linears: three accumulations into one buffer
    linear_bwd(be, dtype, xv, gx, p["wq"], grads["wq"], grads["bq"], gq, d, d)
    linear_bwd(be, dtype, xv, gx, p["wk"], grads["wk"], grads["bk"], gk, d, d)
    linear_bwd(be, dtype, xv, gx, p["wv"], grads["wv"], grads["bv"], gv, d, d)
    dx = rt(val(gx, dtype).reshape(T, d) + gh1, dtype)        # plus the residual path
    return out, grads, dx
