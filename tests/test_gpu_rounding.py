"""GPU: the one rounding every 16-bit result gets, bit for bit, on the values where roundings differ.

The device computes in f32 and rounds once to the element type with the hardware conversions
(`v_cvt_pk_bf16_f32`, `v_cvt_pk_f16_f32`, written as casts); the oracle states the same rounding as integer arithmetic
(`oracle/dfdx_matmul_oracle.c`: `f32_to_bf16`, `f32_to_f16`, round to nearest, ties to even, overflow to infinity,
NaNs quieted -- what `half::f16::from_f32` / `half::bf16::from_f32` do for the reference, dtypes/mod.rs:87-116).  Random
finite data hardly ever lands on a tie, never overflows and never is subnormal, so those classes are crafted here: every
case is an f32 value that the device op forms EXACTLY (a sum of two element-type addends, a product of two element-type
factors) before it rounds, and the stored bits are compared with the oracle's conversion of that same f32 value.
Ops covered: `add_forward` (vector ALU store), `scalar_mul_forward`, a K = 1 product (the rank-1 kernel) and the same
product with the contraction zero-padded to 32 and to 64 (the k-sliced MFMA kernel and the LDS-DMA MFMA tiles).
"""
import numpy as np
import pytest

import oracle
from gpu_util import announce, device

pytestmark = pytest.mark.gpu

MANT = {"bf16": 8, "f16": 11}          # significand bits including the hidden one
EMIN = {"bf16": -126, "f16": -14}      # exponent of the smallest normal
EMAX = {"bf16": 127, "f16": 15}


def elem(dtype, f32_values):
    """f32 values that ARE element-type values -> storage bits (asserting that nothing is lost)."""
    v = np.asarray(f32_values, np.float32)
    st = oracle.to_storage(v, dtype)
    back = oracle.to_f64(st, dtype).astype(np.float32)
    same = (back == v) | (np.isnan(back) & np.isnan(v))
    assert same.all(), f"not {dtype} values: {v[~same][:4]}"
    return st


def bits(st):
    return np.ascontiguousarray(st).view(np.uint16)


def addend_pairs(dtype):
    """(hi, lo) pairs of element-type values whose f32 sum is exact and sits on or next to a rounding boundary."""
    p, emax = MANT[dtype], EMAX[dtype]
    ulp = lambda e: 2.0 ** (e - (p - 1))
    pairs = []
    for e in (0, 5, max(-9, EMIN[dtype] + p + 1), emax - 1):   # (the small addends must stay normal numbers)
        u = ulp(e)
        for hi in (2.0 ** e, 2.0 ** e + u, 2.0 ** e + 2 * u, 2.0 ** (e + 1) - u, 2.0 ** (e + 1) - 2 * u):
            half = u / 2
            tiny = half * 2.0 ** -(p - 1)           # lowest bit an addend with half's exponent carries
            for lo in (half, half + tiny, half - tiny / 2, half / 2, u - tiny):
                for sh, sl in ((1, 1), (-1, -1), (1, -1), (-1, 1)):
                    pairs.append((sh * hi, sl * lo))
    big = (2.0 - 2.0 ** -(p - 1)) * 2.0 ** emax       # largest finite value; its last bit is odd
    half = ulp(emax) / 2
    tiny = half * 2.0 ** -(p - 1)
    for s in (1, -1):
        pairs += [(s * big, s * half), (s * big, s * (half - tiny / 2)), (s * big, s * (half + tiny)), (s * big, s * big),
                  (s * big, s * ulp(emax)), (s * np.inf, 1.0), (s * np.inf, -s * big), (s * 0.0, s * 0.0), (s * 0.0, -s * 0.0)]
    pairs += [(np.inf, -np.inf), (np.nan, 1.0), (1.0, np.nan)]
    return np.array(pairs, np.float32)


def factor_grid(dtype):
    """Element-type factors x[i], s[j] whose f32 products are exact (two p-bit significands, exponents inside f32's
    normal range or its subnormals down to the last bit) and cover ties, near-ties, overflow and subnormal results."""
    p, emin, emax = MANT[dtype], EMIN[dtype], EMAX[dtype]
    one_plus = [1.0, 1.0 + 2.0 ** -(p - 1), 1.5, 2.0 - 2.0 ** -(p - 1), 1.0 + 2.0 ** -(p - 2), 1.25 + 2.0 ** -(p - 1)]
    xs, ss = [], []
    lo1 = -((-emin) // 2)                    # two small exponents for x ...
    s1 = max(emin, emin - lo1 - p + 1)       # ... and for s the ones that put x * s at the bottom of the subnormal range
    for m in one_plus:
        xs += [m, -m, m * 2.0 ** 7, m * 2.0 ** (emax // 2 + 1), m * 2.0 ** lo1, m * 2.0 ** (lo1 - 2)]
    for m in one_plus:
        # results near 1, near the largest finite value and beyond it, and in the subnormal range of the element type
        ss += [m, m * 2.0 ** -(p - 1), m * 2.0 ** (emax // 2), m * 2.0 ** (emax - emax // 2 - 1),
               m * 2.0 ** s1, m * 2.0 ** (s1 + 2), -m * 2.0 ** (s1 + 1)]
    return np.array(xs, np.float32), np.array(ss, np.float32)


def check_bits(dtype, got_st, want_f32, what):
    """Stored bits against the oracle's rounding of `want_f32`; NaNs must be quiet NaNs (their payload is not compared:
    which operand's payload an f32 operation forwards is not part of either contract)."""
    want_st = bits(oracle.to_storage(np.asarray(want_f32, np.float32).reshape(-1), dtype))
    got = bits(got_st).reshape(-1)[: want_st.size]
    nan = np.isnan(np.asarray(want_f32, np.float32).reshape(-1))
    bad = np.flatnonzero((got != want_st) & ~nan)
    assert bad.size == 0, (f"{what} [{dtype}]: {bad.size} of {want_st.size} roundings differ, first at {bad[0]}: "
                           f"value {np.asarray(want_f32, np.float32).reshape(-1)[bad[0]]!r} got {got[bad[0]]:#06x} want {want_st[bad[0]]:#06x}")
    quiet = {"bf16": (0x7f80, 0x0040), "f16": (0x7c00, 0x0200)}[dtype]
    g = got[nan]
    assert ((g & quiet[0]) == quiet[0]).all() and ((g & quiet[1]) != 0).all(), f"{what} [{dtype}]: NaN results must be quiet NaNs, got {g[:4]}"
    return int(np.count_nonzero(~nan))


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_add_rounds_like_the_oracle_on_ties_overflow_and_specials(dtype):
    dev = device()
    pairs = addend_pairs(dtype)
    hi, lo = pairs[:, 0].copy(), pairs[:, 1].copy()
    with np.errstate(invalid="ignore", over="ignore"):
        exact = hi.astype(np.float64) + lo.astype(np.float64)
        want = (hi + lo).astype(np.float32)
    f32_max = float(np.finfo(np.float32).max)
    ok = np.isnan(exact) | (np.abs(exact) > f32_max) | (want.astype(np.float64) == exact)   # (beyond f32: infinity either way)
    assert ok.all(), "a crafted sum is not exact in f32"
    announce("rounding: add_forward", dtype, len(hi), "pairs")
    a, b = dev.tensor(elem(dtype, hi), dtype), dev.tensor(elem(dtype, lo), dtype)
    out = dev.add_forward(a, b)
    n = check_bits(dtype, dev.to_host(out), want, "add_forward")
    # the classes really are in the list: ties, overflow to infinity, a sum that stays the largest finite value
    st = bits(oracle.to_storage(want, dtype))
    inf_bits = {"bf16": 0x7f80, "f16": 0x7c00}[dtype]
    assert np.count_nonzero(((st & 0x7fff) == inf_bits) & np.isfinite(want)) >= 4
    assert n >= 300


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_products_round_like_the_oracle_including_subnormal_results(dtype):
    dev = device()
    xs, ss = factor_grid(dtype)
    with np.errstate(over="ignore", under="ignore"):
        want = np.outer(xs, ss).astype(np.float32)                       # f32 products, exact by construction
        exact = np.outer(xs.astype(np.float64), ss.astype(np.float64))
    f32_max = float(np.finfo(np.float32).max)
    assert ((np.abs(exact) > f32_max) | (want.astype(np.float64) == exact)).all(), "a crafted product is not exact in f32"
    tiny = 2.0 ** EMIN[dtype]
    assert np.count_nonzero((np.abs(want) < tiny) & (want != 0)) >= 20, "no subnormal results in the grid"
    m, n = xs.size, ss.size
    x_st, s_st = elem(dtype, xs), elem(dtype, ss)
    # scalar multiply: one scalar per launch, the whole vector of x
    for j in (0, 1, 3, n - 3, n - 2):
        announce("rounding: scalar_mul_forward", dtype, float(ss[j]))
        out = dev.scalar_mul_forward(dev.tensor(x_st, dtype), float(ss[j]))
        check_bits(dtype, dev.to_host(out), want[:, j], f"scalar_mul_forward by {float(ss[j])!r}")
    # the same products as GEMMs: k = 1 (rank-1 kernel), k = 32 and k = 64 with zero padding (matrix cores)
    for k in (1, 32, 64):
        a = np.zeros((m, k), np.float32)
        b = np.zeros((k, n), np.float32)
        a[:, 0], b[0, :] = xs, ss
        da, db = dev.tensor(elem(dtype, a.reshape(-1)), dtype, (m, k)), dev.tensor(elem(dtype, b.reshape(-1)), dtype, (k, n))
        dc = dev.empty(dtype, (m, n))
        desc = dev.gemm_desc(dtype, m, k, n, da.ptr, (k, 1), db.ptr, (n, 1), dc.ptr, (n, 1))
        announce("rounding: product", dtype, (m, k, n), dev.gemm_plan(desc)[2])
        dev.gemm(desc)
        check_bits(dtype, dev.to_host(dc), want, f"gemm k = {k} ({dev.gemm_plan(desc)[2]})")
    # a larger zero-padded product so that the tiled kernels (not the small-product kernel) store the same values
    reps = 8
    M, N, K = m * reps, n * reps, 128
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    a[:, 0], b[0, :] = np.tile(xs, reps), np.tile(ss, reps)
    Np = (N + 7) // 8 * 8
    bp = np.zeros((K, Np), np.float32)
    bp[:, :N] = b
    da, db = dev.tensor(elem(dtype, a.reshape(-1)), dtype, (M, K)), dev.tensor(elem(dtype, bp.reshape(-1)), dtype, (K, Np))
    dc = dev.empty(dtype, (M, Np))
    from dfdx_amd.rocm import KERNEL_MFMA
    desc = dev.gemm_desc(dtype, M, K, N, da.ptr, (K, 1), db.ptr, (Np, 1), dc.ptr, (Np, 1), kernel=KERNEL_MFMA)
    announce("rounding: tiled product", dtype, (M, K, N), dev.gemm_plan(desc)[2])
    dev.gemm(desc)
    got = bits(dev.to_host(dc)).reshape(M, Np)[:, :N]
    check_bits(dtype, got, np.tile(want, (reps, reps)), f"gemm tiled ({dev.gemm_plan(desc)[2]})")
