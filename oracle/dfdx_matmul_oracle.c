/*
 * CPU oracle for dfdx's matrix-multiplication path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, what dfdx's `Cpu` device computes for
 * `matmul` (reference: dfdx-core/src/tensor_ops/matmul/cpu_kernel.rs).  It is
 * the checker the HIP kernels are compared against and the "port" CPU baseline
 * that the benchmark times.  Nothing in the shipped library links, loads or
 * calls it; only the tests, the smoke check and the benchmark's cpu_baseline
 * leg may.
 *
 * Arithmetic contract (cpu_kernel.rs:38-50, 53-229): one strided GEMM
 *     C[i*crs + j*ccs] = (accum ? C[..] : 0) + sum_k A[i*ars + k*acs] * B[k*brs + j*bcs]
 * The reference forwards this to the third-party `gemm` crate (pinned
 * `gemm = 0.16.14`, dfdx-core/Cargo.toml) as dst := alpha*dst + beta*lhs*rhs
 * with alpha = accum ? 1 : 0, beta = 1 (cpu_kernel.rs:164-185).  That crate is
 * not vendored, so its published contract is restated here: f32 inputs are
 * accumulated in f32; f16 inputs are widened to f32, accumulated in f32 and
 * rounded to f16 (round-to-nearest-even) once when stored; f64 in f64.  bf16
 * is not a dfdx dtype; it follows the f16 rule with bf16 widening/rounding.
 * The unused `naive_gemm` fallback (cpu_kernel.rs:10-36) overwrites instead of
 * summing when accum=false and is deliberately NOT followed.
 *
 * What pins this restatement (tests/test_oracle_*.py): the literals held by
 * the reference's own tests (matmul/mod.rs:368-410, 530-703 and
 * dfdx/src/nn/layers/linear.rs:97-204), an independent float64 BLAS product,
 * exact small-integer products, and the algebraic identities the reference
 * tests assert (mod.rs:413-527).  What is NOT pinned: the summation order
 * inside the gemm crate's micro-kernels (results are compared to a tolerance,
 * never bit-for-bit, as the reference's own tests do), and the crate's
 * intermediate f16 re-rounding between its depth blocks.
 *
 * Per-element summation order here: k ascending, one fused or unfused
 * multiply-add per term (whatever the C compiler emits), in the accumulation
 * type named above.  `acc64 != 0` switches every dtype to double accumulation
 * (the "shadow" result that error bounds are measured against).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2, DT_F64 = 3 };

/* ---------------------------------------------------------------- dtypes -- */

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even, IEEE binary16 */
static inline uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0));
    }
    if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* result is subnormal or zero (|f| < 2^-14) */
        if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        uint32_t e = ax >> 23;
        uint32_t man = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126 - e; /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t e = (ax >> 23) - 127 + 15;
    uint32_t man = ax & 0x7fffffu;
    uint32_t half = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

static inline float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet nan */
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

/* exported for the conversion tests */
void oracle_f16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = f16_to_f32(src[i]);
}
void oracle_f32_to_f16(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = f32_to_f16(src[i]);
}
void oracle_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = bf16_to_f32(src[i]);
}
void oracle_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = f32_to_bf16(src[i]);
}

static size_t dt_size(int dt) {
    switch (dt) {
    case DT_F32: return 4;
    case DT_F16: case DT_BF16: return 2;
    default: return 8;
    }
}

static inline double load_elem(int dt, const void *p, int64_t idx) {
    switch (dt) {
    case DT_F32: return ((const float *)p)[idx];
    case DT_F16: return f16_to_f32(((const uint16_t *)p)[idx]);
    case DT_BF16: return bf16_to_f32(((const uint16_t *)p)[idx]);
    default: return ((const double *)p)[idx];
    }
}

/* ------------------------------------------------------------------ gemm -- */

#define KB 256
#define NB 512

/* Blocked i-k-j product on packed row-major operands; every C element still
 * receives its k terms in ascending order. */
static void packed_gemm_f32(int64_t m, int64_t n, int64_t k, const float *ap, const float *bp, float *acc) {
    for (int64_t j0 = 0; j0 < n; j0 += NB) {
        int64_t jn = (n - j0 < NB) ? n - j0 : NB;
        for (int64_t k0 = 0; k0 < k; k0 += KB) {
            int64_t kn = (k - k0 < KB) ? k - k0 : KB;
#pragma omp parallel for schedule(static)
            for (int64_t i = 0; i < m; i++) {
                float *restrict crow = acc + i * n + j0;
                const float *arow = ap + i * k + k0;
                for (int64_t kk = 0; kk < kn; kk++) {
                    const float a = arow[kk];
                    const float *restrict brow = bp + (k0 + kk) * n + j0;
                    for (int64_t j = 0; j < jn; j++) crow[j] += a * brow[j];
                }
            }
        }
    }
}

static void packed_gemm_f64(int64_t m, int64_t n, int64_t k, const double *ap, const double *bp, double *acc) {
    for (int64_t j0 = 0; j0 < n; j0 += NB) {
        int64_t jn = (n - j0 < NB) ? n - j0 : NB;
        for (int64_t k0 = 0; k0 < k; k0 += KB) {
            int64_t kn = (k - k0 < KB) ? k - k0 : KB;
#pragma omp parallel for schedule(static)
            for (int64_t i = 0; i < m; i++) {
                double *restrict crow = acc + i * n + j0;
                const double *arow = ap + i * k + k0;
                for (int64_t kk = 0; kk < kn; kk++) {
                    const double a = arow[kk];
                    const double *restrict brow = bp + (k0 + kk) * n + j0;
                    for (int64_t j = 0; j < jn; j++) crow[j] += a * brow[j];
                }
            }
        }
    }
}

/*
 * MatMulImpl::matmul (cpu_kernel.rs:38-50; f16 :100-145, f32 :147-187, f64 :189-229).
 * Strides are in elements, as in the reference's `[usize; 2]` arrays:
 * a_strides = [ars, acs] index (i, k); b_strides = [brs, bcs] index (k, j);
 * c_strides = [crs, ccs] index (i, j).  Returns 0, or -1 when out of memory.
 */
int oracle_gemm(int dtype, int64_t m, int64_t k, int64_t n, int accum, int acc64,
                const void *a, int64_t ars, int64_t acs,
                const void *b, int64_t brs, int64_t bcs,
                void *c, int64_t crs, int64_t ccs) {
    if (m <= 0 || n <= 0) return 0;
    const int wide = acc64 || dtype == DT_F64;
    if (wide) {
        double *ap = (double *)malloc(sizeof(double) * (size_t)(m * k + 1));
        double *bp = (double *)malloc(sizeof(double) * (size_t)(k * n + 1));
        double *acc = (double *)calloc((size_t)(m * n), sizeof(double));
        if (!ap || !bp || !acc) { free(ap); free(bp); free(acc); return -1; }
        for (int64_t i = 0; i < m; i++)
            for (int64_t kk = 0; kk < k; kk++) ap[i * k + kk] = load_elem(dtype, a, i * ars + kk * acs);
        for (int64_t kk = 0; kk < k; kk++)
            for (int64_t j = 0; j < n; j++) bp[kk * n + j] = load_elem(dtype, b, kk * brs + j * bcs);
        packed_gemm_f64(m, n, k, ap, bp, acc);
        for (int64_t i = 0; i < m; i++)
            for (int64_t j = 0; j < n; j++) {
                int64_t idx = i * crs + j * ccs;
                double v = acc[i * n + j];
                if (accum) v += load_elem(dtype, c, idx); /* dst := dst + A*B, product formed first */
                switch (dtype) {
                case DT_F32: ((float *)c)[idx] = (float)v; break;
                case DT_F16: ((uint16_t *)c)[idx] = f32_to_f16((float)v); break;
                case DT_BF16: ((uint16_t *)c)[idx] = f32_to_bf16((float)v); break;
                default: ((double *)c)[idx] = v; break;
                }
            }
        free(ap); free(bp); free(acc);
        return 0;
    }
    float *ap = (float *)malloc(sizeof(float) * (size_t)(m * k + 1));
    float *bp = (float *)malloc(sizeof(float) * (size_t)(k * n + 1));
    float *acc = (float *)calloc((size_t)(m * n), sizeof(float));
    if (!ap || !bp || !acc) { free(ap); free(bp); free(acc); return -1; }
    for (int64_t i = 0; i < m; i++)
        for (int64_t kk = 0; kk < k; kk++) ap[i * k + kk] = (float)load_elem(dtype, a, i * ars + kk * acs);
    for (int64_t kk = 0; kk < k; kk++)
        for (int64_t j = 0; j < n; j++) bp[kk * n + j] = (float)load_elem(dtype, b, kk * brs + j * bcs);
    packed_gemm_f32(m, n, k, ap, bp, acc);
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            int64_t idx = i * crs + j * ccs;
            float v = acc[i * n + j];
            if (accum) v += (float)load_elem(dtype, c, idx);
            switch (dtype) {
            case DT_F32: ((float *)c)[idx] = v; break;
            case DT_F16: ((uint16_t *)c)[idx] = f32_to_f16(v); break;
            default: ((uint16_t *)c)[idx] = f32_to_bf16(v); break;
            }
        }
    free(ap); free(bp); free(acc);
    return 0;
}

/* ------------------------------------------------------- kernel drivers --- */
/* Each driver follows the loop structure, offsets and stride swaps of the
 * reference's Cpu impl it cites.  `out` / `grad_out` are contiguous row-major
 * of the output shape (cpu_kernel.rs:242,265,301,327,365,393,431,459); grads
 * are buffers laid out like the operand's physical storage and written through
 * the operand's own strides. */

#define PTR(base, dt, off) ((void *)((char *)(base) + (size_t)(off) * dt_size(dt)))
#define CPTR(base, dt, off) ((const void *)((const char *)(base) + (size_t)(off) * dt_size(dt)))

/* MatMatKernel::forward (cpu_kernel.rs:235-254) */
int oracle_matmat_forward(int dt, int acc64, int64_t m, int64_t k, int64_t n,
                          const void *lhs, const int64_t *ls, const void *rhs, const int64_t *rs, void *out) {
    return oracle_gemm(dt, m, k, n, 0, acc64, lhs, ls[0], ls[1], rhs, rs[0], rs[1], out, n, 1);
}

/* MatMatKernel::backward (cpu_kernel.rs:255-287) */
int oracle_matmat_backward(int dt, int acc64, int64_t m, int64_t k, int64_t n,
                           const void *lhs, const int64_t *ls, void *grad_lhs,
                           const void *rhs, const int64_t *rs, void *grad_rhs, const void *grad_out) {
    int e = oracle_gemm(dt, m, n, k, 1, acc64, grad_out, n, 1, rhs, rs[1], rs[0], grad_lhs, ls[0], ls[1]);
    if (e) return e;
    return oracle_gemm(dt, k, m, n, 1, acc64, lhs, ls[1], ls[0], grad_out, n, 1, grad_rhs, rs[0], rs[1]);
}

/* MatMatBrKernel::forward (cpu_kernel.rs:294-316): lhs (B,M,K) strides ls[3], rhs (K,N) strides rs[2] */
int oracle_matmat_br_forward(int dt, int acc64, int64_t batch, int64_t m, int64_t k, int64_t n,
                             const void *lhs, const int64_t *ls, const void *rhs, const int64_t *rs, void *out) {
    for (int64_t i = 0; i < batch; i++) {
        int e = oracle_gemm(dt, m, k, n, 0, acc64, CPTR(lhs, dt, i * ls[0]), ls[1], ls[2], rhs, rs[0], rs[1],
                            PTR(out, dt, i * m * n), n, 1);
        if (e) return e;
    }
    return 0;
}

/* MatMatBrKernel::backward (cpu_kernel.rs:317-351): grad_rhs is one shared accumulator */
int oracle_matmat_br_backward(int dt, int acc64, int64_t batch, int64_t m, int64_t k, int64_t n,
                              const void *lhs, const int64_t *ls, void *grad_lhs,
                              const void *rhs, const int64_t *rs, void *grad_rhs, const void *grad_out) {
    for (int64_t i = 0; i < batch; i++) {
        const void *go = CPTR(grad_out, dt, i * m * n);
        int e = oracle_gemm(dt, m, n, k, 1, acc64, go, n, 1, rhs, rs[1], rs[0],
                            PTR(grad_lhs, dt, i * ls[0]), ls[1], ls[2]);
        if (e) return e;
        e = oracle_gemm(dt, k, m, n, 1, acc64, CPTR(lhs, dt, i * ls[0]), ls[2], ls[1], go, n, 1,
                        grad_rhs, rs[0], rs[1]);
        if (e) return e;
    }
    return 0;
}

/* MatMatBatch3Kernel::forward (cpu_kernel.rs:358-382) */
int oracle_matmat_batch3_forward(int dt, int acc64, int64_t batch, int64_t m, int64_t k, int64_t n,
                                 const void *lhs, const int64_t *ls, const void *rhs, const int64_t *rs, void *out) {
    for (int64_t i = 0; i < batch; i++) {
        int e = oracle_gemm(dt, m, k, n, 0, acc64, CPTR(lhs, dt, i * ls[0]), ls[1], ls[2],
                            CPTR(rhs, dt, i * rs[0]), rs[1], rs[2], PTR(out, dt, i * m * n), n, 1);
        if (e) return e;
    }
    return 0;
}

/* MatMatBatch3Kernel::backward (cpu_kernel.rs:383-417) */
int oracle_matmat_batch3_backward(int dt, int acc64, int64_t batch, int64_t m, int64_t k, int64_t n,
                                  const void *lhs, const int64_t *ls, void *grad_lhs,
                                  const void *rhs, const int64_t *rs, void *grad_rhs, const void *grad_out) {
    for (int64_t i = 0; i < batch; i++) {
        const void *go = CPTR(grad_out, dt, i * m * n);
        int e = oracle_gemm(dt, m, n, k, 1, acc64, go, n, 1, CPTR(rhs, dt, i * rs[0]), rs[2], rs[1],
                            PTR(grad_lhs, dt, i * ls[0]), ls[1], ls[2]);
        if (e) return e;
        e = oracle_gemm(dt, k, m, n, 1, acc64, CPTR(lhs, dt, i * ls[0]), ls[2], ls[1], go, n, 1,
                        PTR(grad_rhs, dt, i * rs[0]), rs[1], rs[2]);
        if (e) return e;
    }
    return 0;
}

/* MatMatBatch4Kernel::forward (cpu_kernel.rs:424-448) */
int oracle_matmat_batch4_forward(int dt, int acc64, int64_t batch, int64_t seq, int64_t m, int64_t k, int64_t n,
                                 const void *lhs, const int64_t *ls, const void *rhs, const int64_t *rs, void *out) {
    for (int64_t i = 0; i < batch; i++)
        for (int64_t j = 0; j < seq; j++) {
            int e = oracle_gemm(dt, m, k, n, 0, acc64, CPTR(lhs, dt, i * ls[0] + j * ls[1]), ls[2], ls[3],
                                CPTR(rhs, dt, i * rs[0] + j * rs[1]), rs[2], rs[3],
                                PTR(out, dt, (i * seq + j) * m * n), n, 1);
            if (e) return e;
        }
    return 0;
}

/* MatMatBatch4Kernel::backward (cpu_kernel.rs:449-485) */
int oracle_matmat_batch4_backward(int dt, int acc64, int64_t batch, int64_t seq, int64_t m, int64_t k, int64_t n,
                                  const void *lhs, const int64_t *ls, void *grad_lhs,
                                  const void *rhs, const int64_t *rs, void *grad_rhs, const void *grad_out) {
    for (int64_t i = 0; i < batch; i++)
        for (int64_t j = 0; j < seq; j++) {
            const void *go = CPTR(grad_out, dt, (i * seq + j) * m * n);
            int e = oracle_gemm(dt, m, n, k, 1, acc64, go, n, 1, CPTR(rhs, dt, i * rs[0] + j * rs[1]), rs[3], rs[2],
                                PTR(grad_lhs, dt, i * ls[0] + j * ls[1]), ls[2], ls[3]);
            if (e) return e;
            e = oracle_gemm(dt, k, m, n, 1, acc64, CPTR(lhs, dt, i * ls[0] + j * ls[1]), ls[3], ls[2], go, n, 1,
                            PTR(grad_rhs, dt, i * rs[0] + j * rs[1]), rs[2], rs[3]);
            if (e) return e;
        }
    return 0;
}
