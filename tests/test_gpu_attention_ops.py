"""GPU parity of the ops that sit between attention's GEMMs (multi_head_attention.rs:105-146): scalar multiply,
softmax over the last axis, and the copying reshape of a permuted tensor -- against the reference's literals and
the numpy restatement -- and the attention-shaped chain of config 4 with every op on the device."""
import json
import os

import numpy as np
import pytest

import oracle
from oracle import nn_ops
from helpers import assert_within, logical, rng, row_major_strides
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
GLUE = json.load(open(os.path.join(GOLD, "attention_glue_literals.json")))
EPS = {"f32": 2.0 ** -24, "f16": 2.0 ** -11, "bf16": 2.0 ** -8}  # half an ulp at 1.0


def host(dev, view):
    return logical(oracle.to_f64(dev.to_host(view), view.dtype), view.shape, view.strides, view.offset)


def upload(dev, values, dtype):
    values = np.asarray(values, dtype=np.float64)
    return dev.tensor(oracle.to_storage(values.reshape(-1), dtype).reshape(values.shape), dtype)


# ------------------------------------------------------------------ literals --
@pytest.mark.parametrize("case", GLUE["softmax"], ids=lambda c: c["name"])
def test_softmax_literals(case):
    dev = device()
    announce("softmax literal", case["name"])
    x = upload(dev, case["x"], "f32")
    p = dev.softmax_forward(x)
    np.testing.assert_allclose(host(dev, p), case["out"], rtol=0, atol=1e-6)
    mask = np.asarray(case["mask"])
    gx = dev.zeros("f32", x.shape)
    dev.softmax_backward(p, gx, upload(dev, mask / mask.size, "f32"))
    np.testing.assert_allclose(host(dev, gx), case["grad_x"], rtol=0, atol=1e-6)


@pytest.mark.parametrize("case", GLUE["reshape"], ids=lambda c: c["name"])
def test_reshape_literals(case):
    from dfdx_amd.rocm import RocmError, View
    dev = device()
    announce("reshape literal", case["name"])
    st = upload(dev, case["storage"], "f32")
    x = View(st.storage, "f32", tuple(case["shape"]), tuple(case["strides"]))
    out = dev.reshape_forward(x, (len(case["out"]),))
    np.testing.assert_allclose(host(dev, out), case["out"], rtol=0, atol=1e-7)
    gi = dev.zeros_like_storage(x)
    go = upload(dev, np.exp(host(dev, out)) / len(case["out"]), "f32")
    if "grad_storage" in case:
        dev.reshape_backward(x, gi, go)
        np.testing.assert_allclose(oracle.to_f64(dev.to_host(gi), "f32"), case["grad_storage"], rtol=0, atol=1e-6)
    else:  # broadcast view (the reference's test holds no gradient literal for it): elements that share an address are
        # summed, which is what reshape_to/cpu_kernel.rs:28-32 does one element after the other
        dev.reshape_backward(x, gi, go)
        want = nn_ops.reshape_backward(case["shape"], case["strides"], np.zeros(len(case["storage"])), host(dev, go), "f32")
        np.testing.assert_allclose(oracle.to_f64(dev.to_host(gi), "f32"), want, rtol=0, atol=1e-6)


@pytest.mark.parametrize("case", GLUE["scalar_mul"], ids=lambda c: c["name"])
def test_scalar_mul_literals(case):
    dev = device()
    announce("scalar mul literal", case["name"])
    x = upload(dev, case["x"], "f32")
    out = dev.scalar_mul_forward(x, case["scalar"])
    np.testing.assert_allclose(host(dev, out), case["out"], rtol=0, atol=1e-7)
    gx = dev.zeros_like_storage(x)
    dev.scalar_mul_backward(case["scalar"], gx, upload(dev, np.exp(host(dev, out)), "f32"))
    np.testing.assert_allclose(host(dev, gx), case["grad_x"], rtol=0, atol=1e-6)


# ---------------------------------------------------------------- scalar mul --
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("n", [1, 7, 64, 1000, 4099, 1 << 20])
def test_scalar_mul_seeded(n, dtype):
    dev, g = device(), rng(401)
    announce("scalar mul", n, dtype)
    x, go, gi0 = (upload(dev, g.standard_normal(n), dtype) for _ in range(3))
    s = 0.3
    out = dev.scalar_mul_forward(x, s)
    np.testing.assert_array_equal(host(dev, out), nn_ops.scalar_mul_forward(host(dev, x), s, dtype))
    gi = dev.tensor(dev.to_host(gi0), dtype)
    dev.scalar_mul_backward(s, gi, go)
    # reference: product and add each round to the element type; here one rounding -> at most one ulp apart
    want = nn_ops.scalar_mul_backward(s, host(dev, gi0), host(dev, go), dtype)
    np.testing.assert_allclose(host(dev, gi), want, rtol=0, atol=4 * EPS[dtype] * float(np.abs(want).max()))


# ------------------------------------------------------------------- softmax --
SOFTMAX_SHAPES = [(1, 1), (3, 5), (7, 64), (5, 1000), (4, 1024), (3, 4096), (2, 5000), (2, 1001), (2, 1500), (1031, 72),
                  (40000, 64),
                  # long rows, a workgroup each: 4 / 8 / 16 vectors per thread in registers, then the three-pass form (a row of logits)
                  (5, 5120), (3, 8200), (2, 16384), (2, 30000), (3, 50257), (2, 70000)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_softmax_seeded(shape, dtype):
    """Forward against the formula evaluated exactly and rounded once (what an f32 row pass targets) and against
    the reference's op-by-op composition; backward, accumulated into a non-zero grad buffer, likewise."""
    dev, g = device(), rng(402)
    rows, cols = shape
    announce("softmax", shape, dtype)
    scale = 0.125
    x = upload(dev, g.standard_normal((rows, cols)) * 6, dtype)
    x64 = host(dev, x)
    p = dev.softmax_forward(x, scale)
    got = host(dev, p)
    once = nn_ops.softmax_forward(x64 * scale, dtype, faithful=False)
    np.testing.assert_allclose(got, once, rtol=0, atol=2 * EPS[dtype] * float(once.max()) + 1e-7)
    assert np.all(np.abs(got.sum(axis=-1) - 1.0) <= cols * EPS[dtype] + 1e-5)
    if cols <= 64 and rows <= 2048:
        # The composition rounds t - max, exp and every step of the running sum to the element type; on short rows
        # that drift is bounded by cols half-ulps.  (On long rows a 16-bit running sum stalls and the composition
        # itself leaves the exact softmax, so it is no yardstick there.)
        faithful = nn_ops.softmax_forward(nn_ops.scalar_mul_forward(x64, scale, dtype), dtype, faithful=True)
        np.testing.assert_allclose(got, faithful, rtol=0, atol=(8 + cols) * EPS[dtype] * float(once.max()) + 1e-6)
    go = upload(dev, g.standard_normal((rows, cols)), dtype)
    gx0 = upload(dev, g.standard_normal((rows, cols)), dtype)
    gx = dev.tensor(dev.to_host(gx0).reshape(rows, cols), dtype)
    dev.softmax_backward(p, gx, go, scale)
    go64, gx064 = host(dev, go), host(dev, gx0)
    want = gx064 + scale * got * (go64 - (go64 * got).sum(axis=-1, keepdims=True))
    np.testing.assert_allclose(host(dev, gx), want, rtol=0, atol=2 * EPS[dtype] * float(np.abs(want).max()) + 1e-6)


def test_softmax_large_logits_do_not_overflow():
    dev = device()
    announce("softmax large logits")
    x = upload(dev, [[1e4, 1e4 - 1.0, -1e4], [88.0, 89.0, 90.0]], "f32")
    got = host(dev, dev.softmax_forward(x))
    want = nn_ops.softmax_forward(host(dev, x), "f32", faithful=False)
    assert np.all(np.isfinite(got))
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-6)


def test_softmax_in_place():
    from dfdx_amd.rocm import View
    import ctypes
    dev, g = device(), rng(403)
    announce("softmax in place")
    x = upload(dev, g.standard_normal((33, 520)), "f16")
    want = host(dev, dev.softmax_forward(x))
    rc = dev.lib.dfdx_rocm_softmax_forward(dev.ctx, 1, ctypes.c_int64(33), ctypes.c_int64(520), ctypes.c_void_p(x.ptr),
                                           ctypes.c_float(1.0), ctypes.c_void_p(x.ptr))
    assert rc == 0
    np.testing.assert_array_equal(host(dev, x), want)


# ------------------------------------------------------------------- reshape --
def _perm_view(dev, g, shape, axes, dtype):
    from dfdx_amd.rocm import View
    st = upload(dev, g.standard_normal(shape), dtype)
    return st.permute(*axes)


RESHAPE_CASES = [
    ((2, 3, 4, 8), (0, 2, 1, 3)),        # head permute, rows of 8 contiguous
    ((2, 4, 16, 64), (0, 2, 1, 3)),      # 16-byte path
    ((5, 7), (1, 0)),                    # plain transpose: element-wise path
    ((3, 5, 7), (2, 0, 1)),
    ((2, 3, 2, 3, 2, 8), (5, 4, 3, 2, 1, 0)),
    ((2, 3, 2, 3, 2, 8), (1, 0, 3, 2, 4, 5)),
    ((4, 6, 10, 24), (0, 2, 1, 3)),      # inner run not a multiple of 16 bytes for f16? 24*2 = 48: it is; strides are
    ((3, 4, 5, 12), (0, 2, 1, 3)),
    ((8, 16, 1024, 64), (0, 2, 1, 3)),   # config 4: tokens (B,H,S,D) -> (B,S,H,D)
    ((70, 130), (1, 0)),                 # a transposed matrix: 64 x 64 tiles through LDS, ragged edges on both axes
    ((3, 40, 100), (0, 2, 1)),           # the same under a batch axis
    ((2, 3, 64, 48), (0, 1, 3, 2)),      # heads x (dim, seq)
    ((33, 20, 17), (2, 1, 0)),           # the storage-contiguous axis becomes the outermost one
    ((1000, 300), (1, 0)),
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,axes", RESHAPE_CASES, ids=lambda v: "x".join(map(str, v)))
def test_reshape_seeded(shape, axes, dtype):
    """Copies and scatter-adds move values without arithmetic (forward) or with one add (backward): bit-exact."""
    dev, g = device(), rng(404)
    if dtype != "f16" and np.prod(shape) > 1 << 20:
        pytest.skip("large case once")
    announce("reshape", shape, axes, dtype)
    v = _perm_view(dev, g, shape, axes, dtype)
    n = int(np.prod(shape))
    out = dev.reshape_forward(v, (n,))
    st64 = oracle.to_f64(dev.to_host(v), dtype)
    np.testing.assert_array_equal(host(dev, out), nn_ops.reshape_forward(st64, v.shape, v.strides))
    go = upload(dev, g.standard_normal(n), dtype)
    gi0 = upload(dev, g.standard_normal(n), dtype)
    gi = dev.tensor(dev.to_host(gi0), dtype)
    dev.reshape_backward(v, gi, go)
    want = nn_ops.reshape_backward(v.shape, v.strides, host(dev, gi0), host(dev, go), dtype)
    np.testing.assert_array_equal(oracle.to_f64(dev.to_host(gi), dtype), want)


def test_reshape_contiguous_is_free():
    dev, g = device(), rng(405)
    x = upload(dev, g.standard_normal((4, 6)), "f32")
    y = dev.reshape_forward(x, (2, 12))
    assert y.storage.data_ptr() == x.storage.data_ptr() and y.strides == (12, 1)
    with pytest.raises(AssertionError, match="left: 24\n right: 25"):
        dev.reshape_forward(x, (5, 5))


# ------------------------------------------------- config 4, every op on the device --
def test_config4_attention_chain_on_device():
    """Q,K,V [8,16,1024,64] f16: scores = Q.K^T -> softmax(scores / 8) -> out = P.V -> tokens (B,S,H*D) by the
    copying reshape; backward through all of it with dTokens ~ N(0,1).  Nothing leaves the device between the ops;
    each op's result is checked against the restatement applied to that op's own (device-produced) inputs on
    sampled heads."""
    dev, g = device(), rng(4104)
    dtype, (B, H, S, D) = "f16", (8, 16, 1024, 64)
    scale = 1.0 / np.sqrt(D)
    q, k, v = (upload(dev, g.standard_normal((B, H, S, D)).astype(np.float32), dtype) for _ in range(3))
    d_tok = upload(dev, g.standard_normal((B, S, H * D)).astype(np.float32), dtype)
    kt = k.permute(0, 1, 3, 2)
    announce("config4 chain forward")
    scores = dev.forward(q, kt)
    p = dev.softmax_forward(scores, scale)
    out = dev.forward(p, v)
    tokens = dev.reshape_forward(out.permute(0, 2, 1, 3), (B, S, H * D))
    announce("config4 chain backward")
    g_out = dev.zeros_like_storage(out)
    dev.reshape_backward(out.permute(0, 2, 1, 3), g_out, d_tok)
    gp, gv = dev.zeros_like_storage(p), dev.zeros_like_storage(v)
    dev.backward(p, gp, v, gv, g_out)
    gs = dev.zeros_like_storage(scores)
    dev.softmax_backward(p, gs, gp, scale)
    gq, gk = dev.zeros_like_storage(q), dev.zeros_like_storage(kt)
    dev.backward(q, gq, kt, gk, gs)
    dev.synchronize()
    announce("config4 chain checks")
    sample = [(0, 0), (5, 9), (7, 15)]
    f = lambda t: oracle.to_f64(dev.to_host(t), dtype)
    Q, K, V = (f(t).reshape(B, H, S, D) for t in (q, k, v))
    SC, P, GP, GS = (f(t).reshape(B, H, S, S) for t in (scores, p, gp, gs))
    O, GO, GQ, GK, GV = (f(t).reshape(B, H, S, D) for t in (out, g_out, gq, gk, gv))
    TOK, DT = f(tokens).reshape(B, S, H, D), f(d_tok).reshape(B, S, H, D)
    np.testing.assert_array_equal(TOK, O.transpose(0, 2, 1, 3))
    np.testing.assert_array_equal(GO, DT.transpose(0, 2, 1, 3))
    e = EPS[dtype]
    for b, h in sample:
        assert_within(dtype, D, SC[b, h], Q[b, h] @ K[b, h].T, Q[b, h], K[b, h], extra=2 * e * 64, what="scores")
        once = nn_ops.softmax_forward(SC[b, h] * scale, dtype, faithful=False)
        np.testing.assert_allclose(P[b, h], once, rtol=0, atol=2 * e * float(once.max()) + 1e-7)
        assert_within(dtype, S, O[b, h], P[b, h] @ V[b, h], P[b, h], V[b, h], extra=2 * e * 4, what="out")
        assert_within(dtype, D, GP[b, h], GO[b, h] @ V[b, h].T, GO[b, h], V[b, h], extra=2 * e * 64, what="dP")
        assert_within(dtype, S, GV[b, h], P[b, h].T @ GO[b, h], P[b, h], GO[b, h], extra=2 * e * 8, what="dV")
        want = scale * P[b, h] * (GP[b, h] - (GP[b, h] * P[b, h]).sum(axis=-1, keepdims=True))
        np.testing.assert_allclose(GS[b, h], want, rtol=0, atol=2 * e * float(np.abs(want).max()) + 1e-6)
        assert_within(dtype, S, GQ[b, h], GS[b, h] @ K[b, h], GS[b, h], K[b, h], extra=2 * e * 16, what="dQ")
        assert_within(dtype, S, GK[b, h], GS[b, h].T @ Q[b, h], GS[b, h], Q[b, h], extra=2 * e * 16, what="dK")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_reshape_backward_through_broadcast_axes(dtype):
    """Views with one or several broadcast axes (stride 0) between real ones: backward sums grad_out over them."""
    from dfdx_amd.rocm import View
    dev, g = device(), rng(5151)
    for shape, strides, nstore in (((4, 6, 5), (5, 0, 1), 20), ((3, 4, 8, 16), (0, 16, 0, 1), 64), ((7, 9), (0, 0), 1),
                                   ((2, 3, 4), (4, 0, 1), 8), ((64, 33, 8), (8, 0, 1), 512)):
        announce("reshape backward, broadcast axes", dtype, shape, strides)
        st = upload(dev, g.standard_normal(nstore), dtype)
        x = View(st.storage, dtype, shape, strides)
        total = int(np.prod(shape))
        go = upload(dev, g.standard_normal(total), dtype)
        gi0 = g.standard_normal(nstore)
        gi = upload(dev, gi0, dtype)
        dev.reshape_backward(x, gi, go)
        want = nn_ops.reshape_backward(shape, strides, oracle.to_f64(dev.to_host(upload(dev, gi0, dtype)), dtype), host(dev, go), dtype)
        exact = oracle.to_f64(dev.to_host(upload(dev, gi0, dtype)), dtype).copy()
        np.add.at(exact, nn_ops._view_indices(shape, strides).reshape(-1), host(dev, go).reshape(-1))
        got = oracle.to_f64(dev.to_host(gi), dtype)
        folded = total // max(1, len(set(nn_ops._view_indices(shape, strides).reshape(-1).tolist())))
        # one rounding of the exact sum; the reference rounds after every add, which the loose bound covers
        np.testing.assert_allclose(got, exact, rtol=0, atol=EPS[dtype] * 2 * np.abs(exact).max() + 1e-6)
        np.testing.assert_allclose(got, want, rtol=0, atol=EPS[dtype] * 2 * folded * np.abs(exact).max() + 1e-6)
        # forward of the same view repeats the stored elements
        out = dev.reshape_forward(x, (total,))
        np.testing.assert_array_equal(host(dev, out), host(dev, x).reshape(-1))
