"""Host-side mirror of dfdx's ``TransformerEncoderBlock`` on the Rocm device: every op is one call into the C ABI.

    TransformerEncoderBlock   dfdx/src/nn/layers/transformer.rs:24-48
        = ResidualAdd<MultiHeadAttention>, LayerNorm1D, ResidualAdd<(Linear, ReLU, Linear)>, LayerNorm1D
    MultiHeadAttention        dfdx/src/nn/layers/multi_head_attention.rs:105-146
    Linear / LayerNorm1D / ResidualAdd   linear.rs:82-89, layer_norm1d.rs:87-91, residual_add.rs:38-45

The forward keeps what the reference's tape would keep (the inputs of every op); the backward walks the ops in
reverse; every gradient buffer starts as zeros and is accumulated into, as with
``Gradients::get_or_alloc_mut`` (dfdx-core/src/tensor/gradients.rs:53-58) -- here all of a pass's buffers are carved
from one allocation and declared zero without a fill (``dfdx_rocm_zero_deferred``): the first op that accumulates
into a whole buffer stores 0 + value, so the step pays neither the fill nor the read of the zeros; a buffer whose
first use is anything else is filled then.  ``deferred_zeros=False`` restores the single eager fill.  The
multiplication by 1/sqrt(head dim) between q.k^T and the softmax (multi_head_attention.rs:133-134) is folded into the
softmax kernel.
"""
from __future__ import annotations

import math
from typing import Dict, Tuple

import numpy as np

from .rocm import Rocm, View

PARAMS = ("wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "g1", "be1", "w1", "b1", "w2", "b2", "g2", "be2")


class EncoderBlock:
    """Parameters are device ``View``s: w* are (out, in) row-major Linear weights, b* biases, g*/be* the LayerNorm
    gamma / beta."""

    def __init__(self, dev: Rocm, dtype: str, d_model: int, heads: int, d_ff: int, params: Dict[str, View],
                 deferred_zeros: bool = True):
        assert d_model % heads == 0, f"left: {d_model % heads}\n right: 0"
        missing = [n for n in PARAMS if n not in params]
        assert not missing, f"missing parameters: {missing}"
        self.dev, self.dtype, self.d, self.h, self.ff, self.p = dev, dtype, d_model, heads, d_ff, params
        self.deferred_zeros = deferred_zeros

    def forward(self, x: View) -> Tuple[View, dict]:
        """x: (batch, seq, d_model) contiguous.  Returns the block's output and the tensors the backward needs."""
        dev, p = self.dev, self.p
        B, S, d = x.shape
        assert d == self.d, f"left: {d}\n right: {self.d}"
        H, D = self.h, self.d // self.h
        q = dev.linear_forward(x, p["wq"], p["bq"])
        k = dev.linear_forward(x, p["wk"], p["bk"])
        v = dev.linear_forward(x, p["wv"], p["bv"])
        heads = lambda t: View(t.storage, t.dtype, (B, S, H, D), (S * d, d, D, 1), t.offset)
        qv = heads(q).permute(0, 2, 1, 3)          # (B, H, S, D), head-interleaved strides
        kv = heads(k).permute(0, 2, 3, 1)          # (B, H, D, S)
        vv = heads(v).permute(0, 2, 1, 3)
        scores = dev.forward(qv, kv)               # (B, H, S, S)
        scale = 1.0 / math.sqrt(D)
        # The softmax entry takes its scale as a C float.  An f64 block whose 1/sqrt(head dim) has no exact float value
        # multiplies by the double scalar in an op of its own, as the reference does (multi_head_attention.rs:133-134).
        folded = self.dtype != "f64" or float(np.float32(scale)) == scale
        if not folded:
            scores = dev.scalar_mul_forward(scores, scale)
        probs = dev.softmax_forward(scores, scale if folded else 1.0)
        tokens = dev.forward(probs, vv)            # (B, H, S, D)
        tok = dev.reshape_forward(tokens.permute(0, 2, 1, 3), (B, S, d))
        attn = dev.linear_forward(tok, p["wo"], p["bo"])
        h1 = dev.add_forward(attn, x)
        n1 = dev.layer_norm_forward(h1, p["g1"], p["be1"])
        f1 = dev.linear_forward(n1, p["w1"], p["b1"])
        r1 = dev.relu_forward(f1)
        f2 = dev.linear_forward(r1, p["w2"], p["b2"])
        h2 = dev.add_forward(f2, n1)
        out = dev.layer_norm_forward(h2, p["g2"], p["be2"])
        saved = dict(x=x, qv=qv, kv=kv, vv=vv, probs=probs, tokens=tokens, tok=tok, h1=h1, n1=n1, f1=f1, r1=r1, h2=h2,
                     scale=scale, folded=folded)
        return out, saved

    def backward(self, saved: dict, grad_out: View) -> Tuple[Dict[str, View], View]:
        """grad_out: d(loss)/d(out), contiguous like the output.  Returns ({parameter: gradient}, d(loss)/d(x))."""
        dev, p, s = self.dev, self.p, saved
        x, n1, tok, tokens, probs = s["x"], s["n1"], s["tok"], s["tokens"], s["probs"]
        qv, kv, vv = s["qv"], s["kv"], s["vv"]
        # every gradient buffer of the pass: one allocation, pieces aligned to 256 B, zero by declaration (or one fill)
        acts = dict(gh2=s["h2"], gf2=s["h2"], gn1=n1, gr1=s["r1"], gf1=s["f1"], gh1=s["h1"], gattn=s["h1"], gx=x, gtok=tok,
                    gtokens=tokens, gp=probs, gscores=probs, gq=x, gk=x, gv=x)   # gq, gk, gv: laid out like the q, k, v storages
        if not s["folded"]:
            acts["gscaled"] = probs   # gradient of the scaled scores, between the softmax and the scalar multiply
        bufs = dev.zeros_many([p[n] for n in PARAMS] + list(acts.values()), deferred=self.deferred_zeros)
        grads = dict(zip(PARAMS, bufs[:len(PARAMS)]))
        g = dict(zip(acts, bufs[len(PARAMS):]))
        gh2, gf2, gn1, gr1, gf1, gh1, gattn, gx = (g[k] for k in ("gh2", "gf2", "gn1", "gr1", "gf1", "gh1", "gattn", "gx"))
        gtok, gtokens, gp, gscores, gq, gk, gv = (g[k] for k in ("gtok", "gtokens", "gp", "gscores", "gq", "gk", "gv"))
        try:
            dev.layer_norm_backward(s["h2"], p["g2"], gh2, grads["g2"], grads["be2"], grad_out)
            dev.add_backward(gf2, gn1, gh2)            # h2 = f2 + n1
            dev.linear_backward(s["r1"], gr1, p["w2"], grads["w2"], grads["b2"], gf2)
            dev.relu_backward(s["f1"], gf1, gr1)
            dev.linear_backward(n1, gn1, p["w1"], grads["w1"], grads["b1"], gf1)
            dev.layer_norm_backward(s["h1"], p["g1"], gh1, grads["g1"], grads["be1"], gn1)
            dev.add_backward(gattn, gx, gh1)           # h1 = attn + x
            dev.linear_backward(tok, gtok, p["wo"], grads["wo"], grads["bo"], gattn)
            dev.reshape_backward(tokens.permute(0, 2, 1, 3), gtokens, gtok)
            dev.backward(probs, gp, vv, gv, gtokens)
            if s["folded"]:
                dev.softmax_backward(probs, gscores, gp, s["scale"])
            else:
                dev.softmax_backward(probs, g["gscaled"], gp, 1.0)
                dev.scalar_mul_backward(s["scale"], gscores, g["gscaled"])
            dev.backward(qv, gq, kv, gk, gscores)
            for w, b, gg in (("wq", "bq", gq), ("wk", "bk", gk), ("wv", "bv", gv)):   # x feeds three Linears: one buffer
                dev.linear_backward(x, gx, p[w], grads[w], grads[b], gg)
            dev.settle_zeros()   # nothing is left pending in this block; a gradient no op touched would be filled here
        except BaseException:
            # an op refused or raised in mid-pass: no declaration may outlive the pass unsettled, whoever still holds
            # a View of the arena (the caller sees the exception, not zeros it could rely on)
            if bufs and bufs[0].owner is not None:
                bufs[0].owner.forget()
            raise
        return grads, gx
