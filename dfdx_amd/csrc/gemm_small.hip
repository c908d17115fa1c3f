// Small products in every element type: one 16 x 16 tile of C per workgroup, the contraction cut over its waves.
//
// A product of a few MFLOP (a Linear layer on 64 rows, the reference's own test shapes) is bound by the chain
// launch -> load -> MFMA -> store, not by any rate, and the tiled kernels walk k in steps behind one another (9.7 us for
// f32 64 x 512 x 256 as four k pieces plus the combining launch).  Here every wave of a workgroup takes one slice of k,
// requests ALL the operand values of a pass (four steps) at once -- straight into the registers the MFMA reads, no LDS
// staging, any strides --, the next pass's behind them where the registers allow, runs its MFMA chain on two
// accumulators, and the slices meet in LDS, added in wave order (the result does not depend on timing).  Lane l supplies
// A[row l % 16][k] and B[k][col l % 16] for KL consecutive k per step, k = 4 KL s + KL (l / 16) + c, c < KL: one 16-byte
// load where the operand is stored along k and aligned.  The 16-bit types take KL = 8 and feed the eight values to one
// v_mfma_f32_16x16x32 (with four values and the 16x16x16 instruction the same kernel needed twice the loads:
// 16 x 4096 x 4096 f16 16.7 -> 9.8 us); f32 and f64 take KL = 4 and four v_mfma_*_16x16x4 (whose lane group l / 16 is
// the k index: any bijection between (lane group, instruction) and k serves, as long as A and B share it).
//
// Optional second result: the sums of A's rows over k, from the values the workgroups of tile column 0 hold anyway
// (Linear's bias gradient out of the weight-gradient launch).
#include "gemm_internal.h"
#include <algorithm>

namespace dfdx_rocm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short i16x8 __attribute__((ext_vector_type(8)));

struct SmallParams {
    const void *a, *b;
    void *c;
    const void *bias;
    int m, n, k, tiles_n;
    int64_t a_rs, a_cs, b_rs, b_cs, ldc;
    int accumulate, bias_mode;
    int a_vec, b_vec;  // the operand is stored along k and every 4-k group of a row is one aligned vector
    int slice;         // k per wave, a multiple of the step (16 k; 32 for the 16-bit types)
    void *ksum;        // may be null: ksum[i] (+)= sum_k A[i][k]
    int ksum_accumulate;
};

// Per element type: the accumulator type, four k-values of one row as the MFMA wants them, the MFMA step, and which row
// of the 16 x 16 tile register r of lane l holds.
template <typename T> struct Small;
template <> struct Small<float> {
    typedef float acc_t;
    typedef f32x4 acc4;
    typedef f32x4 pack;
    static constexpr int KL = 4;  // k values a lane supplies per step
    static __device__ __forceinline__ pack zero() { return pack{0.f, 0.f, 0.f, 0.f}; }
    static __device__ __forceinline__ pack vec(const float *p) { return *(const f32x4 *)p; }
    static __device__ __forceinline__ void set(pack &v, int c, const float *p) { v[c] = *p; }
    static __device__ __forceinline__ acc4 mma(pack a, pack b, acc4 acc) {
#pragma unroll
        for (int c = 0; c < 4; c++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], b[c], acc, 0, 0, 0);
        return acc;
    }
    static __device__ __forceinline__ float sum_pack(pack v) { return (v[0] + v[1]) + (v[2] + v[3]); }
    static __device__ __forceinline__ int out_row(int r, int q) { return 4 * q + r; }
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Small<double> {
    typedef double acc_t;
    typedef f64x4 acc4;
    typedef f64x4 pack;
    static constexpr int KL = 4;
    static __device__ __forceinline__ pack zero() { return pack{0.0, 0.0, 0.0, 0.0}; }
    static __device__ __forceinline__ pack vec(const double *p) {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
        const f64x2 lo = *(const f64x2 *)p, hi = *(const f64x2 *)(p + 2);
        return pack{lo[0], lo[1], hi[0], hi[1]};
    }
    static __device__ __forceinline__ void set(pack &v, int c, const double *p) { v[c] = *p; }
    static __device__ __forceinline__ acc4 mma(pack a, pack b, acc4 acc) {
#pragma unroll
        for (int c = 0; c < 4; c++) acc = __builtin_amdgcn_mfma_f64_16x16x4f64(a[c], b[c], acc, 0, 0, 0);
        return acc;
    }
    static __device__ __forceinline__ double sum_pack(pack v) { return (v[0] + v[1]) + (v[2] + v[3]); }
    static __device__ __forceinline__ int out_row(int r, int q) { return 4 * r + q; }  // f64: register r is row 4 r + l / 16
    static __device__ __forceinline__ double load(const double *p) { return *p; }
    static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
};
template <> struct Small<_Float16> {  // eight k per lane: one 16-byte load, v_mfma_f32_16x16x32_f16
    typedef float acc_t;
    typedef f32x4 acc4;
    typedef f16x8 pack;
    static constexpr int KL = 8;
    static __device__ __forceinline__ pack zero() { return pack{0, 0, 0, 0, 0, 0, 0, 0}; }
    static __device__ __forceinline__ pack vec(const _Float16 *p) { return *(const f16x8 *)p; }
    static __device__ __forceinline__ void set(pack &v, int c, const _Float16 *p) { v[c] = *p; }
    static __device__ __forceinline__ acc4 mma(pack a, pack b, acc4 acc) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0); }
    static __device__ __forceinline__ float sum_pack(pack v) {
        return (((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3])) + (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
    }
    static __device__ __forceinline__ int out_row(int r, int q) { return 4 * q + r; }
    static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct Small<__bf16> {
    typedef float acc_t;
    typedef f32x4 acc4;
    typedef i16x8 pack;
    static constexpr int KL = 8;
    static __device__ __forceinline__ float widen(short b) { return __uint_as_float((uint32_t)(uint16_t)b << 16); }
    static __device__ __forceinline__ pack zero() { return pack{0, 0, 0, 0, 0, 0, 0, 0}; }
    static __device__ __forceinline__ pack vec(const __bf16 *p) { return *(const i16x8 *)p; }
    static __device__ __forceinline__ void set(pack &v, int c, const __bf16 *p) { v[c] = *(const short *)p; }
    static __device__ __forceinline__ acc4 mma(pack a, pack b, acc4 acc) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float sum_pack(pack v) {
        return ((widen(v[0]) + widen(v[1])) + (widen(v[2]) + widen(v[3]))) + ((widen(v[4]) + widen(v[5])) + (widen(v[6]) + widen(v[7])));
    }
    static __device__ __forceinline__ int out_row(int r, int q) { return 4 * q + r; }
    static __device__ __forceinline__ float load(const __bf16 *p) { return widen(*(const short *)p); }
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }
};

// LONG: slices of more than one pass.  The one-pass form is kept as short as it can be: at 4 - 5 us a launch, the
// instructions a longer kernel has to fetch and jump over show (0.3 - 0.6 us on a 64-row Linear layer's gradients).
template <typename T, int WAVES, bool LONG> __global__ __launch_bounds__(WAVES * 64) void gemm_small_kernel(const SmallParams p) {
    typedef Small<T> S;
    typedef typename S::acc_t A;
    typedef typename S::acc4 A4;
    typedef typename S::pack Pack;
    constexpr int KL = S::KL, STEP = 4 * KL, PASS = 4 * STEP;  // k per lane and step, per step of a wave, per pass
    __shared__ A part[WAVES][256];
    __shared__ A part_rows[WAVES][16];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int r16 = lane % 16, q = lane / 16;
    const int tm = blockIdx.x / p.tiles_n, tn = blockIdx.x % p.tiles_n;
    const int row = tm * 16 + r16, col = tn * 16 + r16;
    const bool row_ok = row < p.m, col_ok = col < p.n;
    const T *ap = (const T *)p.a + (int64_t)(row_ok ? row : 0) * p.a_rs;
    const T *bp = (const T *)p.b + (int64_t)(col_ok ? col : 0) * p.b_cs;
    const int k0 = wave * p.slice, k1 = min(p.k, k0 + p.slice);
    // Four k values of a pass that the slice's end may cut.  One-pass form in f32 and f64: a branch per value.  Otherwise
    // every lane loads from an address inside the slice and the values beyond the end (or of a row / column beyond m / n)
    // are replaced by zeros afterwards, so that all the loads of the pass are in flight together (16-bit values come one
    // 2-byte load each, which the branches would space out: 0.3 - 0.7 us on the same gradients).
    constexpr bool BRANCHY = !LONG && sizeof(T) >= 4;
    auto fetch = [&](const T *base, int64_t kstride, bool ok, bool vec, int kk) -> Pack {
        Pack v = S::zero();
        if constexpr (BRANCHY) {  // (this order of the tests and no test per step measured best of the forms tried)
            if (!ok || kk >= k1) return v;
            if (vec && kk + KL - 1 < k1) return S::vec(base + kk);
#pragma unroll
            for (int c = 0; c < KL; c++)
                if (kk + c < k1) S::set(v, c, base + (int64_t)(kk + c) * kstride);
        } else {
            if (vec && kk + KL - 1 < k1) return ok ? S::vec(base + kk) : v;
            const Pack z = S::zero();
#pragma unroll
            for (int c = 0; c < KL; c++) {
                S::set(v, c, base + (int64_t)max(0, min(kk + c, k1 - 1)) * kstride);
                if (!ok || kk + c >= k1) v[c] = z[c];
            }
        }
        return v;
    };
    A4 acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
    const bool sums = p.ksum && tn == 0;
    A rsum = 0;  // of A[row r16][this lane's k values]
    // Passes of four steps of 16 k (8 loads per lane each); LONG: the loads of the next pass in flight behind the MFMAs
    // of this one (not f64).
    Pack av[4], bv[4];
    // A pass that lies inside the slice is loaded without a test per value: the rows and columns beyond m and n read
    // row / column 0 (their results are never stored), and the branches on the layout are the same for the whole launch.
    auto whole = [&](const T *base, int64_t kstride, bool vec, int kk) -> Pack {
        if (vec) return S::vec(base + kk);
        Pack v = S::zero();
#pragma unroll
        for (int c = 0; c < KL; c++) S::set(v, c, base + (int64_t)(kk + c) * kstride);
        return v;
    };
    auto load_pass = [&](Pack *a, Pack *b, int kb) {
        if (LONG && kb + PASS <= k1) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                a[u] = whole(ap, p.a_cs, p.a_vec, kb + STEP * u + KL * q);
                b[u] = whole(bp, p.b_rs, p.b_vec, kb + STEP * u + KL * q);
            }
        } else {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (BRANCHY || kb + STEP * u < k1) {  // the same in every lane: steps past the end are not loaded at all
                    a[u] = fetch(ap, p.a_cs, row_ok, p.a_vec, kb + STEP * u + KL * q);
                    b[u] = fetch(bp, p.b_rs, col_ok, p.b_vec, kb + STEP * u + KL * q);
                } else {
                    a[u] = S::zero();
                    b[u] = S::zero();
                }
            }
        }
    };
    auto use_pass = [&](const Pack *a, const Pack *b) {
        if (sums) {
#pragma unroll
            for (int u = 0; u < 4; u++) rsum += S::sum_pack(a[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (u % 2 == 0) acc0 = S::mma(a[u], b[u], acc0);
            else acc1 = S::mma(a[u], b[u], acc1);
        }
    };
    if constexpr (!LONG) {
        load_pass(av, bv, k0);
        use_pass(av, bv);
    } else if constexpr (sizeof(T) < 8) {
        Pack an[4], bn[4];
        load_pass(av, bv, k0);
        for (int kb = k0; kb < k1; kb += 2 * PASS) {  // k0, k1 and kb are the same in every lane of a wave
            if (kb + PASS < k1) load_pass(an, bn, kb + PASS);
            use_pass(av, bv);
            if (kb + PASS < k1) {
                if (kb + 2 * PASS < k1) load_pass(av, bv, kb + 2 * PASS);
                use_pass(an, bn);
            }
        }
    } else {  // f64: two passes of operands would halve the waves a compute unit holds
        for (int kb = k0; kb < k1; kb += PASS) {
            load_pass(av, bv, kb);
            use_pass(av, bv);
        }
    }
    A4 sum = acc0 + acc1;
    if (sums) {  // uniform over the workgroup
        rsum += __shfl_xor(rsum, 16, 64);
        rsum += __shfl_xor(rsum, 32, 64);
        if (lane < 16) part_rows[wave][lane] = rsum;
    }
    if constexpr (WAVES > 1) {
#pragma unroll
        for (int r = 0; r < 4; r++) part[wave][r * 64 + lane] = sum[r];
        __syncthreads();
        if (wave != 0) return;
        sum = A4{part[0][lane], part[0][64 + lane], part[0][128 + lane], part[0][192 + lane]};
#pragma unroll
        for (int w = 1; w < WAVES; w++)
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] += part[w][r * 64 + lane];
    }
    if (sums && lane < 16 && row_ok) {  // slices in wave order, then the old value unless the gradient is fresh
        A v = part_rows[0][lane];
#pragma unroll
        for (int w = 1; w < WAVES; w++) v += part_rows[w][lane];
        T *dst = (T *)p.ksum + row;
        S::store(dst, (p.ksum_accumulate ? S::load(dst) : A(0)) + v);
    }
    if (!col_ok) return;
    const A cb = p.bias_mode == BIAS_PER_COL ? S::load((const T *)p.bias + col) : A(0);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int orow = tm * 16 + S::out_row(r, q);
        if (orow >= p.m) continue;
        T *dst = (T *)p.c + (int64_t)orow * p.ldc + col;
        A v = sum[r] + cb;
        if (p.bias_mode == BIAS_PER_ROW) v += S::load((const T *)p.bias + orow);
        if (p.accumulate) v += S::load(dst);
        S::store(dst, v);
    }
}

inline size_t elem_size(int dt) { return dt == DT_F64 ? 8 : dt == DT_F32 ? 4 : 2; }
// waves per workgroup: slices of at least 32 k; sixteen once each of them has two passes to overlap (not f64, whose two
// passes of operands fill the 128 registers a lane of such a workgroup may have)
inline int small_waves(int dtype, int64_t k) {
    return (k >= 2048 && dtype != DT_F64) ? 16 : k >= 256 ? 8 : k >= 128 ? 4 : k >= 64 ? 2 : 1;
}

template <typename T, bool LONG> hipError_t launch_form(const SmallParams &p, int waves, dim3 grid, hipStream_t stream) {
    switch (waves) {
    case 16:
        if constexpr (sizeof(T) < 8) gemm_small_kernel<T, 16, LONG><<<grid, 1024, 0, stream>>>(p);
        else return hipErrorInvalidValue;
        break;
    case 8: gemm_small_kernel<T, 8, LONG><<<grid, 512, 0, stream>>>(p); break;
    case 4: gemm_small_kernel<T, 4, LONG><<<grid, 256, 0, stream>>>(p); break;
    case 2: gemm_small_kernel<T, 2, LONG><<<grid, 128, 0, stream>>>(p); break;
    default: gemm_small_kernel<T, 1, LONG><<<grid, 64, 0, stream>>>(p); break;
    }
    return hipGetLastError();
}
template <typename T> hipError_t launch_t(const SmallParams &p, int waves, dim3 grid, hipStream_t stream) {
    return p.slice > 16 * Small<T>::KL ? launch_form<T, true>(p, waves, grid, stream) : launch_form<T, false>(p, waves, grid, stream);
}

}  // namespace

bool small_supported(const GemmProblem &p) {
    if (p.dtype < DT_F32 || p.dtype > DT_F64) return false;
    if (p.m < 1 || p.n < 1 || p.k < 1 || p.k >= (1ll << 30)) return false;
    if (p.c_cs != 1 && p.n != 1) return false;
    if (p.n > 1 && p.m > 1 && p.c_rs < p.n) return false;
    if (p.nb1 * p.nb2 != 1) return false;  // one product per launch
    const uintptr_t mask = elem_size(p.dtype) - 1;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uintptr_t)p.c | (uintptr_t)p.bias) & mask) return false;
    return ((p.m + 15) / 16) * ((p.n + 15) / 16) < (1ll << 20);
}

bool small_ksum_supported(const GemmProblem &p) {
    return p.ksum && p.ksum_of == KSUM_OF_A && small_supported(p) && ((uintptr_t)p.ksum & (elem_size(p.dtype) - 1)) == 0;
}

// Estimated time, fitted to timings on a 256-CU MI355X: the launch; then the longer of (a) the chain of loads of one
// workgroup, which grows with the whole contraction however many waves share it (the 16 rows of a load instruction lie
// a row stride apart), and (b) the bytes all workgroups pull through the caches -- no
// operand value is shared between workgroups, so every tile fetches its 16 rows and 16 columns again (5 - 8 TB/s over
// the whole chip); an operand that is not stored along k costs a 2- or 4-byte load per value on top, and so does C.
double small_time(const GemmProblem &p, int compute_units) {
    const double tiles = (double)((p.m + 15) / 16) * (double)((p.n + 15) / 16);
    const double es = (double)elem_size(p.dtype);
    const bool half = p.dtype == DT_F16 || p.dtype == DT_BF16;
    const int strided = (p.a_cs != 1) + (p.b_rs != 1);  // operands not stored along k
    // per k: 16-byte loads of 16 rows (16-bit types: eight k each, 1.7 ns; f32: four k, 3.4 ns; f64: 6.8 ns)
    const double per_k = p.dtype == DT_F64 ? 6.8e-9 : half ? 1.7e-9 : 3.4e-9;
    const double chain = std::max(0.5e-6, (double)p.k * per_k);
    // an operand that is not stored along k comes one 2- or 4-byte load per value: a fixed cost in the chain, and, where
    // the operand is large, a rate (16 x 4096 x 4096: f16 9.8 us A.B^T against 22.9 us A.B, f32 18.9 against 24.1).  With
    // one row of tiles and only the large operand strided, the gathers of all tiles run beside the chain instead of in
    // it (4 x 2048 x 2048 f16 A.B 6.6 us, 4 x 1024 x 8192 f32 A.B 13.9 us): the longer of the two counts.
    const double strided_values = (p.a_cs != 1 ? (double)p.m * (double)p.k : 0.0) + (p.b_rs != 1 ? (double)p.k * (double)p.n : 0.0);
    const bool one_row = std::min(p.m, p.n) <= 16 && strided == 1;
    const double gather = p.dtype == DT_F64 ? 0.0
                          : (half ? 0.9e-6 : 0.4e-6) * strided + (one_row ? 0.0 : strided_values / (half ? 1.3e12 : 3.3e12));
    const double gather_stream = p.dtype == DT_F64 || !one_row ? 0.0 : strided_values / (half ? 0.87e12 : 0.8e12);
    // one row (or column) of tiles: the 16 rows of the small operand are the same for every tile and stay in the caches,
    // what streams is the large operand, once -- at the rate of HBM when it is larger than the caches hold
    const double rows_per_tile = std::min(p.m, p.n) <= 16 ? 16.0 : 32.0;
    const double streamed = tiles * rows_per_tile * es * (double)p.k;
    const double unique = ((double)p.m + (double)p.n) * (double)p.k * es;
    const double bandwidth = (unique > 64e6 ? 4.5e12 : p.dtype == DT_F64 ? 8e12 : 7.5e12) * std::max(1, compute_units) / 256.0;
    // C leaves in pieces of 16 elements of a row: 1.5 - 2.5 TB/s (a rank-1 update of 4096^2 through this kernel: 22 - 34 us)
    const double c_bytes = (double)p.m * (double)p.n * es * (p.accumulate ? 2.0 : 1.0);
    const double c_rate = (p.dtype == DT_F16 || p.dtype == DT_BF16 ? 1.5e12 : 2.2e12) * std::max(1, compute_units) / 256.0;
    return 2.1e-6 + gather + std::max(std::max(chain, streamed / bandwidth), gather_stream) + c_bytes / c_rate;
}

hipError_t launch_small(const GemmProblem &g, hipStream_t stream) {
    if (!small_supported(g) || g.splits > 1) return hipErrorInvalidValue;
    const size_t es = elem_size(g.dtype);
    const int kl = es == 2 ? 8 : 4;  // k values per lane and step: 16 bytes (f64: 32 bytes as two halves)
    const uintptr_t vmask = 15;
    SmallParams p;
    p.a = g.a; p.b = g.b; p.c = g.c; p.bias = g.bias;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.tiles_n = (int)((g.n + 15) / 16);
    p.a_rs = g.a_rs; p.a_cs = g.a_cs; p.b_rs = g.b_rs; p.b_cs = g.b_cs;
    p.ldc = g.m == 1 ? g.n : g.c_rs;
    p.accumulate = g.accumulate; p.bias_mode = g.bias ? g.bias_mode : BIAS_NONE;
    const int64_t vq = (int64_t)((vmask + 1) / es);  // row stride must keep the vectors aligned
    p.a_vec = g.a_cs == 1 && (g.m == 1 || g.a_rs % vq == 0) && ((uintptr_t)g.a & vmask) == 0;
    p.b_vec = g.b_rs == 1 && (g.n == 1 || g.b_cs % vq == 0) && ((uintptr_t)g.b & vmask) == 0;
    p.ksum = (g.ksum && g.ksum_of == KSUM_OF_A) ? g.ksum : nullptr;
    p.ksum_accumulate = g.ksum_accumulate;
    const int waves = small_waves(g.dtype, g.k);
    const int step = 4 * kl;
    p.slice = (int)(((g.k + waves - 1) / waves + step - 1) / step * step);
    const dim3 grid((unsigned)(((g.m + 15) / 16) * p.tiles_n));
    switch (g.dtype) {
    case DT_F32: return launch_t<float>(p, waves, grid, stream);
    case DT_F16: return launch_t<_Float16>(p, waves, grid, stream);
    case DT_BF16: return launch_t<__bf16>(p, waves, grid, stream);
    case DT_F64: return launch_t<double>(p, waves, grid, stream);
    default: return hipErrorInvalidValue;
    }
}


namespace {

// ---- thin contractions (k <= 32) with large outputs: the matrix cores as a row-streaming kernel ----
//
// A product such as 4096 x 16 x 4096 writes 2 K bytes of C per byte it reads: what bounds it is how C leaves the chip.
// The tiled kernels pad k to their step and reach 2 - 3 TB/s on it.  Here a wave keeps the fragments of 64 columns of B
// in registers (four 16-column tiles, every k of the product) and walks down the rows of A sixteen at a time: one 16-byte
// load per lane is a whole 16 x k piece of a row-major A, four (f32: sixteen) MFMAs make a 16 x 64 strip of C, and the
// strip goes through a wave-private LDS tile so that it leaves as whole rows -- eight (f32: sixteen) lanes with 16 bytes
// each per row, never the 32-byte row pieces of the accumulator layout.  The MFMA's operands are swapped (B's columns as
// its rows), which leaves four consecutive columns of one row of C in a lane: the LDS tile is written 16 bytes at a time.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));  // element-aligned: global memory takes such 16-byte accesses

struct ThinParams {
    const void *a, *b;
    void *c;
    const void *bias;
    int m, n, k;
    int64_t a_rs, a_cs, b_rs, b_cs, ldc;
    int accumulate, bias_mode;
    int a_vec, b_vec;      // stored along k, every k group of a row / column one aligned 16-byte vector
    int rows_per_block;    // a multiple of 16
    int nb2;               // batches: blockIdx.z = i1 * nb2 + i2
    int64_t a_b1, a_b2, b_b1, b_b2, c_b1, c_b2;
};

template <typename T, int STEPS, bool ALIGNED> __global__ __launch_bounds__(256) void gemm_thin_kernel(const ThinParams p) {
    typedef Small<T> S;
    typedef typename S::pack Pack;
    constexpr int KL = S::KL, STEP = 4 * KL;
    constexpr int PIECE = 16 / (int)sizeof(T);  // elements of C a lane stores at once
    constexpr int PPR = 64 / PIECE;             // such pieces per row of the strip
    constexpr int RPI = 64 / PPR;               // rows of the strip one store instruction covers
    constexpr int H = 16 / RPI;                 // store instructions per strip
    constexpr int LDW = 68;                     // floats per row of the LDS tile (64 + 4: the rows start four banks apart)
    __shared__ float tile[4][16 * LDW];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, r16 = lane % 16, q = lane / 16;
    const int n0 = blockIdx.x * 256 + wave * 64;
    if (n0 >= p.n) return;  // (no workgroup barrier below: a wave may leave alone)
    const int m_begin = blockIdx.y * p.rows_per_block, m_end = min(p.m, m_begin + p.rows_per_block);
    const int i1 = blockIdx.z / p.nb2, i2 = blockIdx.z % p.nb2;
    const T *a_mat = (const T *)p.a + i1 * p.a_b1 + i2 * p.a_b2;
    const T *b_mat = (const T *)p.b + i1 * p.b_b1 + i2 * p.b_b2;
    T *c_mat = (T *)p.c + i1 * p.c_b1 + i2 * p.c_b2;
    // The k values of step s that lane group q supplies.  16-bit types: the eight consecutive ones 32 s + 8 q + c, one
    // 16-byte load where the operand is stored along k (a group that the end of k cuts: every load from an address inside
    // the operand, zeros put in afterwards; a group beyond k: nothing loaded).  f32: the c-th 16x16x4 MFMA of a step takes
    // k = 8 (c / 2) + 2 (c % 2) + {0, 4, 1, 5}[q] -- the order in which the tiled f32 kernels contract (their 32x32x2
    // MFMAs take the pairs (0, 4), (1, 5), (2, 6), (3, 7) of every eight k), so that a product gives the same bits
    // whether it comes here as one tall matrix or goes to them as a batch.
    auto fetch = [&](const T *base, int64_t kstride, bool ok, bool vec, int s) -> Pack {
        Pack v = S::zero();
        const Pack z = S::zero();
        if constexpr (sizeof(T) == 4) {
            // loaded as k = 16 s + 4 q + j (one vector where the operand is stored along k), then the wave's halves
            // trade the odd and even values: two v_permlane32_swap put every value where the order above wants it
            const int kk = STEP * s + 4 * q;
            Pack x = S::zero();
            if (ok && kk < p.k) {
                if (vec && kk + 4 <= p.k) {
                    x = S::vec(base + kk);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        S::set(x, j, base + (int64_t)min(kk + j, p.k - 1) * kstride);
                        if (kk + j >= p.k) x[j] = 0.0f;
                    }
                }
            }
            const auto r01 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x[0]), __float_as_uint(x[1]), false, false);
            const auto r23 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x[2]), __float_as_uint(x[3]), false, false);
            v[0] = __uint_as_float(r01[0]); v[1] = __uint_as_float(r23[0]);
            v[2] = __uint_as_float(r01[1]); v[3] = __uint_as_float(r23[1]);
        } else {
            const int kk = STEP * s + KL * q;
            if (!ok || kk >= p.k) return v;
            if (vec && kk + KL <= p.k) return S::vec(base + kk);
#pragma unroll
            for (int c = 0; c < KL; c++) {
                S::set(v, c, base + (int64_t)min(kk + c, p.k - 1) * kstride);
                if (kk + c >= p.k) v[c] = z[c];
            }
        }
        return v;
    };
    Pack bf[STEPS][4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int col = n0 + 16 * t + r16;
        const bool ok = col < p.n;
        const T *base = b_mat + (int64_t)(ok ? col : 0) * p.b_cs;
#pragma unroll
        for (int s = 0; s < STEPS; s++) bf[s][t] = fetch(base, p.b_rs, ok, p.b_vec, s);
    }
    auto rows_of_a = [&](int m0, Pack (&af)[STEPS]) {
        const T *base = a_mat + (int64_t)min(m0 + r16, p.m - 1) * p.a_rs;
#pragma unroll
        for (int s = 0; s < STEPS; s++) af[s] = fetch(base, p.a_cs, true, p.a_vec, s);
    };
    const int pc = lane % PPR, prow = lane / PPR;
    const int col = n0 + PIECE * pc;
    // ALIGNED: every row of C starts on a 16-byte boundary and n is a whole number of pieces (the form without the tests
    // below is 0.3 - 0.8 us faster on a 4096 x 16 x 4096 product).  Otherwise the pieces move as unaligned 16-byte
    // accesses; the last piece of a row, where n cuts it, element by element.
    const bool piece_ok = col < p.n, whole = ALIGNED || col + PIECE <= p.n;
    float cb[PIECE];
#pragma unroll
    for (int i = 0; i < PIECE; i++) cb[i] = (p.bias_mode == BIAS_PER_COL && col + i < p.n) ? S::load((const T *)p.bias + col + i) : 0.0f;
    float *mine = tile[wave];
    Pack next[STEPS];
    rows_of_a(m_begin, next);
    for (int m0 = m_begin; m0 < m_end; m0 += 16) {
        Pack cur[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; s++) cur[s] = next[s];
        if (m0 + 16 < m_end) rows_of_a(m0 + 16, next);
        u32x4 old[H];
#pragma unroll
        for (int h = 0; h < H; h++) old[h] = u32x4{0u, 0u, 0u, 0u};
        if (p.accumulate) {
#pragma unroll
            for (int h = 0; h < H; h++) {
                const int row = m0 + prow + RPI * h;
                if (row < m_end && piece_ok) {
                    const T *src = c_mat + (int64_t)row * p.ldc + col;
                    if (whole) {
                        if constexpr (ALIGNED) old[h] = *(const u32x4 *)src;
                        else old[h] = *(const u32x4_unaligned *)src;
                    } else {
                        T was[PIECE];
#pragma unroll
                        for (int i = 0; i < PIECE; i++) was[i] = src[col + i < p.n ? i : 0];
                        __builtin_memcpy(&old[h], was, 16);
                    }
                }
            }
        }
        f32x4 acc[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < STEPS; s++) acc[t] = S::mma(bf[s][t], cur[s], acc[t]);
        }
        // register r of lane (r16, q), tile t = C[m0 + r16][n0 + 16 t + 4 q + r]
#pragma unroll
        for (int t = 0; t < 4; t++) *(f32x4 *)&mine[r16 * LDW + 16 * t + 4 * q] = acc[t];
        // the lanes of a wave run its LDS instructions in order: no wait, but the compiler must keep the order too
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int h = 0; h < H; h++) {
            const int row_l = prow + RPI * h, row = m0 + row_l;
            float v[PIECE];
#pragma unroll
            for (int i = 0; i < PIECE; i += 4) {
                const f32x4 x = *(const f32x4 *)&mine[row_l * LDW + PIECE * pc + i];
                v[i] = x[0]; v[i + 1] = x[1]; v[i + 2] = x[2]; v[i + 3] = x[3];
            }
            if (row < m_end && piece_ok) {
                const float rb = p.bias_mode == BIAS_PER_ROW ? S::load((const T *)p.bias + row) : 0.0f;
                T was[PIECE], out[PIECE];
                __builtin_memcpy(was, &old[h], 16);
#pragma unroll
                for (int i = 0; i < PIECE; i++) {
                    float x = v[i] + cb[i];
                    if (p.bias_mode == BIAS_PER_ROW) x += rb;
                    if (p.accumulate) x += S::load(&was[i]);
                    S::store(&out[i], x);
                }
                u32x4 raw;
                __builtin_memcpy(&raw, out, 16);
                T *dst = c_mat + (int64_t)row * p.ldc + col;
                if (whole) {
                    // non-temporal where aligned: C is megabytes written once, whole lines per wave instruction, and is
                    // not kept in the caches on its way out (f32 65536 x 8 x 256 17.1 -> 16.3 us, 4096 x 16 x 4096 18.0 ->
                    // 17.2 us, f16 12.0 -> 11.5 us, launch after launch on one buffer set)
                    if constexpr (ALIGNED) __builtin_nontemporal_store(raw, (u32x4 *)dst);
                    else *(u32x4_unaligned *)dst = raw;
                } else {
#pragma unroll
                    for (int i = 0; i < PIECE; i++)
                        if (col + i < p.n) dst[i] = out[i];
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <typename T, bool ALIGNED> hipError_t launch_thin_a(const ThinParams &p, dim3 grid, hipStream_t stream) {
    if (p.k <= 4 * Small<T>::KL) gemm_thin_kernel<T, 1, ALIGNED><<<grid, 256, 0, stream>>>(p);
    else gemm_thin_kernel<T, 2, ALIGNED><<<grid, 256, 0, stream>>>(p);
    return hipGetLastError();
}
template <typename T> hipError_t launch_thin_t(const ThinParams &p, bool aligned, dim3 grid, hipStream_t stream) {
    return aligned ? launch_thin_a<T, true>(p, grid, stream) : launch_thin_a<T, false>(p, grid, stream);
}

// rows per workgroup: as many as leave a thousand workgroups (the fragments of B are loaded once per workgroup)
inline int thin_rows_per_block(const GemmProblem &g) {
    const int64_t blocks_n = (g.n + 255) / 256 * g.nb1 * g.nb2;
    int rows = 256;
    while (rows > 16 && blocks_n * ((g.m + rows - 1) / rows) < 1024) rows /= 2;
    return rows;
}

}  // namespace

// k <= 32 and a large row-major output (rows off the 16-byte grid move as unaligned pieces); batches as grid.z.  (The
// 16-bit types at k = 33 .. 64, two MFMA steps, were measured on the attention-score products, 128 x (1024 x 64 x 1024):
// 89 us against 73 us of the LDS-DMA tiles -- every workgroup fetches its own fragments of B, and at that k the
// operands are no longer small next to C.)
bool thin_mfma_supported(const GemmProblem &g) {
    if (g.dtype != DT_F32 && g.dtype != DT_F16 && g.dtype != DT_BF16) return false;
    const int64_t es = (int64_t)elem_size(g.dtype), nb = g.nb1 * g.nb2;
    const int64_t step = es == 2 ? 32 : 16;
    if (g.k < 1 || g.k > (es == 2 ? step : 2 * step) || g.m < 64 || g.n < 64 || g.reduce || nb < 1 || nb > 65535) return false;
    if (g.m >= (1ll << 30) || g.n >= (1ll << 30)) return false;
    if (g.c_cs != 1 || g.c_rs < g.n) return false;
    // below these sizes of C the small-product and the tiled kernels are as fast or faster (past one MFMA step a strip
    // takes two rounds of MFMAs and only pays on outputs that leave the last-level cache)
    const int64_t bytes = nb * g.m * g.n * es;
    if (g.k > step && g.n < 1024) return false;  // (f32 16 x 16 x (512 x 32 x 512): 107 us against 92 us of the tiles)
    if (bytes < (g.k > step ? (64ll << 20) : es == 2 ? (1ll << 20) : (4ll << 20))) return false;
    const int rows = thin_rows_per_block(g);
    if ((g.m + rows - 1) / rows > 65535) return false;  // row blocks are grid.y
    const uintptr_t mask = (uintptr_t)es - 1;
    return (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c | (uintptr_t)g.bias) & mask) == 0;
}

hipError_t launch_thin_mfma(const GemmProblem &g, hipStream_t stream) {
    if (!thin_mfma_supported(g)) return hipErrorInvalidValue;
    const int64_t vq = 16 / (int64_t)elem_size(g.dtype);
    ThinParams p;
    p.a = g.a; p.b = g.b; p.c = g.c; p.bias = g.bias;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.a_rs = g.a_rs; p.a_cs = g.a_cs; p.b_rs = g.b_rs; p.b_cs = g.b_cs; p.ldc = g.c_rs;
    p.accumulate = g.accumulate; p.bias_mode = g.bias ? g.bias_mode : BIAS_NONE;
    p.a_vec = g.a_cs == 1 && g.a_rs % vq == 0 && g.a_b1 % vq == 0 && g.a_b2 % vq == 0 && ((uintptr_t)g.a & 15) == 0;
    p.b_vec = g.b_rs == 1 && g.b_cs % vq == 0 && g.b_b1 % vq == 0 && g.b_b2 % vq == 0 && ((uintptr_t)g.b & 15) == 0;
    p.rows_per_block = thin_rows_per_block(g);
    p.nb2 = (int)g.nb2;
    p.a_b1 = g.a_b1; p.a_b2 = g.a_b2; p.b_b1 = g.b_b1; p.b_b2 = g.b_b2; p.c_b1 = g.c_b1; p.c_b2 = g.c_b2;
    const dim3 grid((unsigned)((g.n + 255) / 256), (unsigned)((g.m + p.rows_per_block - 1) / p.rows_per_block),
                    (unsigned)(g.nb1 * g.nb2));
    const bool aligned = ((uintptr_t)g.c & 15) == 0 && g.c_rs % vq == 0 && g.n % vq == 0 && (g.nb1 * g.nb2 == 1 || (g.c_b1 % vq == 0 && g.c_b2 % vq == 0));
    switch (g.dtype) {
    case DT_F32: return launch_thin_t<float>(p, aligned, grid, stream);
    case DT_F16: return launch_thin_t<_Float16>(p, aligned, grid, stream);
    case DT_BF16: return launch_thin_t<__bf16>(p, aligned, grid, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace dfdx_rocm
