"""GPU: gradient storage whose zero fill is deferred (`DFDX_ROCM_ZERO_DEFERRED`, `dfdx_rocm_zero_deferred`).

`Gradients::get_or_alloc_mut` (dfdx-core/src/tensor/gradients.rs:53-58) hands every backward op a zero-filled buffer
that the op then accumulates into.  A deferred buffer must be indistinguishable from that through every call of the
library: each case below runs once on buffers filled eagerly and once on buffers that are full of NaN patterns and only
DECLARED zero, and the results must be the same bits.  Poisoning shows a read of the old contents, a fill that was
skipped wrongly, or one that ran where it should not matter."""
import ctypes

import numpy as np
import pytest

import oracle
from gpu_util import announce, device
from helpers import rng

pytestmark = pytest.mark.gpu

ES = {"f32": 4, "f16": 2, "bf16": 2}


def poisoned(dev, dtype, shape, strides=None, numel=None):
    """A view whose storage holds NaN bit patterns and is declared zero without a fill."""
    import torch

    from dfdx_amd.rocm import View, _row_major

    n = int(np.prod(shape, dtype=np.int64)) if numel is None else numel
    raw = torch.full((max(n * ES[dtype], 16),), 0xFF, dtype=torch.uint8, device="cuda")   # 0xFFFF.. is a NaN in every type
    dev.zero_deferred(raw.data_ptr(), n * ES[dtype])
    return View(raw, dtype, tuple(shape), _row_major(tuple(shape)) if strides is None else tuple(strides))


def zeroed(dev, dtype, shape, strides=None, numel=None):
    from dfdx_amd.rocm import View, _row_major

    n = int(np.prod(shape, dtype=np.int64)) if numel is None else numel
    v = dev.zeros(dtype, (n,))
    return View(v.storage, dtype, tuple(shape), _row_major(tuple(shape)) if strides is None else tuple(strides))


def rand(dev, g, dtype, shape, scale=1.0):
    host = (g.standard_normal(int(np.prod(shape))) * scale).astype(np.float32)
    return dev.tensor(oracle.to_storage(host, dtype), dtype, tuple(shape))


def both(dev, fn):
    """fn(make) -> list of gradient views; run with eager and with deferred zeros, compare the storages bit for bit."""
    eager = [dev.to_host(v) for v in fn(zeroed)]
    lazy = [dev.to_host(v) for v in fn(poisoned)]
    assert len(eager) == len(lazy)
    for i, (e, l) in enumerate(zip(eager, lazy)):
        assert np.array_equal(e.view(np.uint8), l.view(np.uint8)), f"gradient {i} differs"
    return eager


def test_alloc_deferred_reads_back_as_zeros():
    from dfdx_amd.rocm import ZERO_DEFERRED

    dev = device()
    announce("alloc deferred")
    for nbytes in (24, 1 << 20):
        ptr = dev.alloc(nbytes, ZERO_DEFERRED)
        host = np.full(nbytes, 0x5A, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_d2h(dev.ctx, host.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes)))
        dev.free(ptr)
        assert not host.any()


def test_synchronize_and_settle_run_the_pending_fills():
    import torch

    dev = device()
    announce("settle / synchronize")
    for settle in (dev.settle_zeros, dev.synchronize):
        raw = torch.full((4096,), 0xFF, dtype=torch.uint8, device="cuda")
        dev.zero_deferred(raw.data_ptr() + 256, 1000)
        settle()
        torch.cuda.synchronize()
        got = raw.cpu().numpy()
        assert np.all(got[:256] == 0xFF) and not got[256:1256].any() and np.all(got[1256:] == 0xFF)


def test_free_drops_the_fill_and_a_cached_buffer_is_not_declared_zero_again():
    from dfdx_amd.rocm import ZERO_DEFERRED

    dev = device()
    announce("free drops a pending fill")
    dev.enable_cache()
    try:
        ptr = dev.alloc(1 << 16, ZERO_DEFERRED)
        dev.free(ptr)
        again = dev.alloc(1 << 16, False)   # the same buffer, not zeroed: nothing may fill it behind the caller's back
        assert again == ptr
        ones = np.full(1 << 16, 7, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_h2d(dev.ctx, ctypes.c_void_p(again), ones.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(1 << 16)))
        dev.synchronize()
        back = np.zeros(1 << 16, np.uint8)
        dev._check(dev.lib.dfdx_rocm_copy_d2h(dev.ctx, back.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(again), ctypes.c_size_t(1 << 16)))
        assert np.all(back == 7)
        dev.free(again)
    finally:
        dev.disable_cache()


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_accumulating_gemm_into_a_whole_deferred_buffer(dtype):
    """MatMat backward: both gradients fresh; then a second backward accumulates on top (no longer fresh)."""
    dev, g = device(), rng(71)
    m, k, n = 96, 160, 72
    a, b, go = rand(dev, g, dtype, (m, k)), rand(dev, g, dtype, (k, n)), rand(dev, g, dtype, (m, n))
    announce("deferred gemm", dtype)

    def run(make):
        ga, gb = make(dev, dtype, (m, k)), make(dev, dtype, (k, n))
        dev.backward(a, ga, b, gb, go)
        dev.backward(a, ga, b, gb, go)
        return [ga, gb]

    ga, gb = both(dev, run)
    assert np.all(np.isfinite(oracle.to_f64(ga, dtype))) and np.abs(oracle.to_f64(gb, dtype)).max() > 0


def test_permuted_and_partial_outputs():
    """A column-major gradient view covers its buffer (stored); a view with a gap in every row does not (filled first,
    the gaps read back as zeros)."""
    dev, g = device(), rng(72)
    dtype, (m, k, n) = "f16", (64, 48, 40)
    a, b = rand(dev, g, dtype, (m, k)), rand(dev, g, dtype, (k, n))
    announce("deferred gemm, permuted / padded C")

    def run(make):
        col_major = make(dev, dtype, (m, n), strides=(1, m))
        padded = make(dev, dtype, (m, n), strides=(n + 8, 1), numel=m * (n + 8))
        for c in (col_major, padded):
            dev.gemm(dev.gemm_desc(dtype, m, k, n, a.ptr, (k, 1), b.ptr, (n, 1), c.ptr, c.strides, accumulate=True))
        return [col_major, padded]

    _, padded = both(dev, run)
    assert not oracle.to_f64(padded, dtype).reshape(m, n + 8)[:, n:].any()


def test_deferred_buffer_as_an_input_operand_is_zeros():
    dev, g = device(), rng(73)
    dtype, (m, k, n) = "f32", (32, 64, 48)
    b = rand(dev, g, dtype, (k, n))
    announce("deferred buffer as operand")
    a = poisoned(dev, dtype, (m, k))
    c = rand(dev, g, dtype, (m, n))
    dev.gemm(dev.gemm_desc(dtype, m, k, n, a.ptr, (k, 1), b.ptr, (n, 1), c.ptr, (n, 1)))
    assert not dev.to_host(c).any() and not dev.to_host(a).any()


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_every_backward_op_treats_a_deferred_gradient_as_zeros(dtype):
    dev, g = device(), rng(74)
    rows, cols = 70, 136
    x, go = rand(dev, g, dtype, (rows, cols)), rand(dev, g, dtype, (rows, cols))
    gamma = rand(dev, g, dtype, (cols,))
    announce("deferred gradients through the backward ops", dtype)

    def run(make):
        out = []
        gb = make(dev, dtype, (cols,))
        dev.bias_backward(go, gb)
        out.append(gb)
        gx = make(dev, dtype, (rows, cols))
        dev.relu_backward(x, gx, go)
        out.append(gx)
        gl, gr = make(dev, dtype, (rows, cols)), make(dev, dtype, (rows, cols))
        dev.add_backward(gl, gr, go)
        dev.add_backward(gl, gl, go)      # t + t: the second add of the pair must see the first
        out += [gl, gr]
        gt = make(dev, dtype, (rows, cols))
        dev.add_backward(gt, gt, go)      # t + t as the first use of a deferred buffer
        out.append(gt)
        gs = make(dev, dtype, (rows, cols))
        dev.scalar_mul_backward(0.37, gs, go)
        out.append(gs)
        p = dev.softmax_forward(x, 0.5)
        gsm = make(dev, dtype, (rows, cols))
        dev.softmax_backward(p, gsm, go, 0.5)
        out.append(gsm)
        gxl, gg, gbeta = make(dev, dtype, (rows, cols)), make(dev, dtype, (cols,)), make(dev, dtype, (cols,))
        dev.layer_norm_backward(x, gamma, gxl, gg, gbeta, go)
        out += [gxl, gg, gbeta]
        # mixed: only one of the two add gradients deferred
        mixed_l, mixed_r = make(dev, dtype, (rows, cols)), zeroed(dev, dtype, (rows, cols))
        dev.add_backward(mixed_l, mixed_r, go)
        out += [mixed_l, mixed_r]
        return out

    res = both(dev, run)
    for r in res:
        assert np.all(np.isfinite(oracle.to_f64(r, dtype)))


def test_reshape_backward_through_a_permuted_view():
    dev, g = device(), rng(75)
    dtype, (B, H, S, D) = "f16", (2, 3, 20, 8)
    announce("deferred reshape backward")
    tokens = rand(dev, g, dtype, (B, H, S, D))
    go = rand(dev, g, dtype, (B, S, H * D))

    def run(make):
        gt = make(dev, dtype, (B, H, S, D))
        dev.reshape_backward(tokens.permute(0, 2, 1, 3), gt, go)
        return [gt]

    both(dev, run)


def test_encoder_block_with_deferred_gradients_matches_the_eager_fill():
    from dfdx_amd.encoder import PARAMS, EncoderBlock

    dev, g = device(), rng(76)
    dtype, (B, S, d, H, ff) = "bf16", (2, 64, 128, 4, 256)
    shapes = {"wq": (d, d), "wk": (d, d), "wv": (d, d), "wo": (d, d), "w1": (ff, d), "w2": (d, ff),
              "bq": (d,), "bk": (d,), "bv": (d,), "bo": (d,), "b1": (ff,), "b2": (d,), "g1": (d,), "g2": (d,), "be1": (d,), "be2": (d,)}
    params = {n: rand(dev, g, dtype, shapes[n], 0.1) for n in PARAMS}
    x, gout = rand(dev, g, dtype, (B, S, d)), rand(dev, g, dtype, (B, S, d), 1.0 / (B * S))
    announce("encoder block, deferred vs eager gradient zeros")
    results = []
    for deferred in (False, True):
        blk = EncoderBlock(dev, dtype, d, H, ff, params, deferred_zeros=deferred)
        _, saved = blk.forward(x)
        grads, gx = blk.backward(saved, gout)
        results.append([dev.to_host(grads[n]) for n in PARAMS] + [dev.to_host(gx)])
    for name, e, l in zip(PARAMS + ("gx",), *results):
        assert np.array_equal(e.view(np.uint8), l.view(np.uint8)), name


def test_forget_zeros_withdraws_declarations_on_caller_owned_storage():
    """Storage the caller owns and has only DECLARED zero may be released before anything consumed the declaration; the
    caller then withdraws it (`dfdx_rocm_forget_zeros`), and no later settle may write into that memory."""
    import torch

    dev = device()
    announce("forget zeros")
    n = 1 << 20
    raw = torch.full((4 * n,), 0x5A, dtype=torch.uint8, device="cuda")
    base = raw.data_ptr()
    dev.zero_deferred(base, n)               # wholly inside the forgotten range: dropped, never filled
    dev.zero_deferred(base + 2 * n, n)       # outside: still promised, filled by the settle below
    dev.zero_deferred(base + n + n // 2, n // 2 + 16)   # reaches past the end of the forgotten range: filled at the forget
    dev.forget_zeros(base, n + n // 2 + 8)
    dev.forget_zeros(base + 3 * n, n)        # nothing declared there: not an error
    dev.forget_zeros(0, 0)
    dev.settle_zeros()
    torch.cuda.synchronize()
    host = raw.cpu().numpy()
    assert (host[:n + n // 2] == 0x5A).all(), "a forgotten declaration was filled after all"
    assert not host[n + n // 2: 2 * n + 16].any(), "a declaration that straddles the range's end must be filled"
    assert not host[2 * n:3 * n].any(), "a declaration outside the range must survive"
    assert (host[3 * n:] == 0x5A).all()


def test_arena_declarations_go_when_the_last_view_goes():
    """`zeros_many(deferred=True)` ties the declarations to the arena: once no View of it is left, the memory returns to
    the allocator, and a later settle must not touch what now belongs to another tensor."""
    import gc

    import torch

    dev = device()
    announce("arena forgets its declarations")
    like = dev.empty("f32", (1 << 18,))
    views = dev.zeros_many([like, like, like], deferred=True)
    ptr, nbytes = views[0].storage.data_ptr(), 3 * (1 << 20)
    keep = views[1]                       # one surviving view keeps the arena and its declarations
    del views
    gc.collect()
    assert dev.to_host(keep)[:16].tolist() == [0.0] * 16          # still zero by declaration -> settled -> zeros
    del keep
    gc.collect()
    torch.cuda.synchronize()
    again = torch.full((nbytes,), 0x33, dtype=torch.uint8, device="cuda")   # the caching allocator hands the block back
    dev.settle_zeros()
    torch.cuda.synchronize()
    assert (again.cpu().numpy() == 0x33).all(), "a stale declaration was filled into memory that has a new owner"
    assert again.data_ptr() == ptr or True   # (whichever block it got: nothing may have been written)


def test_a_refused_product_leaves_the_zero_declaration_of_its_output_in_place():
    """A call that is refused (here: the no-allocation entry with a split whose partial sums exceed its scratch) must
    not consume the declaration of its output: the retry through `dfdx_rocm_gemm` with accumulate = 1 has to give the
    bits of the eagerly filled run, not an accumulation into the poison."""
    from dfdx_amd import RocmError
    from dfdx_amd.rocm import ERR_SCRATCH_TOO_SMALL

    dev, g = device(), rng(77)
    m = n = 1024
    k = 16384
    a, b = rand(dev, g, "f16", (k, m)), rand(dev, g, "f16", (k, n))
    announce("refused product on a deferred output", (m, k, n))

    def run(make):
        c = make(dev, "f16", (m, n))
        desc = dev.gemm_desc("f16", m, k, n, a.ptr, (1, m), b.ptr, (n, 1), c.ptr, (n, 1), accumulate=True, split_k=9)
        with pytest.raises(RocmError) as err:
            dev.gemm_noalloc(desc)
        assert err.value.code == ERR_SCRATCH_TOO_SMALL
        dev.gemm(desc)
        return [c]

    both(dev, run)
