// f64 GEMM on the matrix cores: v_mfma_f64_16x16x4_f64, f64 accumulate -- the fourth element type of the reference's
// matmul (`MatMulImpl<f64>`, dfdx-core/src/tensor_ops/matmul/cpu_kernel.rs:189-229), which the reference's whole test
// suite also runs in.
//
// One instruction multiplies a 16x4 by a 4x16 tile and takes 64 cycles on a SIMD (78.6 TFLOP/s over the chip): with 16
// accumulator tiles per wave a k step of 4 is 1024 cycles of matrix-core time against eight 8-byte LDS reads, so the
// kernel is bound by the matrix cores as soon as the operands are in LDS at all.  The structure is therefore the plain
// one: a workgroup of four waves owns a BM x BN tile of C, both operand tiles (BK = 16) are staged global -> registers
// -> LDS with one buffer computing while the other is filled, every global access is one bounds-checked 8-byte element
// (any strides, any alignment, any extent; the axis with the unit stride decides which thread mapping coalesces), LDS
// holds both operands k-contiguous with an odd row pitch.
//
// Lane l of a wave supplies A[row l % 16][k = l / 16] and B[k = l / 16][col l % 16] and receives, in register r of a
// tile, C[row 4 * r + l / 16][col l % 16].
#include "gemm_internal.h"
#include <algorithm>

namespace dfdx_rocm {
namespace {

typedef double f64x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 16;
constexpr int LDS_ROW = BK + 1;  // doubles; odd: the 16 rows a fragment read touches fall on different banks

struct Params {
    const double *a, *b;
    double *c;
    const double *bias;
    int m, n, k;
    int64_t a_rs, a_ks, b_cs, b_ks;  // element strides: A[i][k] = a[i * a_rs + k * a_ks], B[k][j] = b[j * b_cs + k * b_ks]
    int64_t ldc;
    int64_t a_b1, a_b2, b_b1, b_b2, c_b1, c_b2;
    int nb2, kbatches;
    int tiles_m, tiles_n, tiles_per_batch, total_blocks;
    int accumulate, bias_mode;
};

// One operand tile ROWS x BK: NT threads, ROWS * BK / NT elements each.  KC: the operand is k-contiguous in memory
// (a wave reads 4 rows x 128 B), else row-contiguous (a wave reads 64 consecutive rows of one k: 512 B).
template <int ROWS, int NT, bool KC> struct Loader {
    static constexpr int N = ROWS * BK / NT;
    static_assert(N >= 1 && NT % BK == 0 && (KC || NT % ROWS == 0 || ROWS % NT == 0), "tile does not divide over the threads");
    double regs[N];
    __device__ __forceinline__ static void where(int i, int tid, int *row, int *k) {
        if constexpr (KC) {
            *k = tid % BK;
            *row = tid / BK + (NT / BK) * i;
        } else {
            *row = tid % ROWS;
            *k = tid / ROWS + (NT / ROWS) * i;
        }
    }
    // `g` = element (row 0 of the tile, k = 0 of the k tile); rows_left / k_left bound the tile.
    __device__ __forceinline__ void load(const double *g, int64_t row_stride, int64_t k_stride, int rows_left, int k_left, int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            int row, k;
            where(i, tid, &row, &k);
            regs[i] = (row < rows_left && k < k_left) ? g[row * row_stride + k * k_stride] : 0.0;
        }
    }
    __device__ __forceinline__ void store(double *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < N; i++) {
            int row, k;
            where(i, tid, &row, &k);
            lds[row * LDS_ROW + k] = regs[i];
        }
    }
};

// Two waves per SIMD keep the matrix core issuing (a lone wave reaches 3/4 of the rate of two, measured on MFMA-only
// loops): the 128 x 128 tile runs 8 waves, the 64 x 64 tile 4 waves with several workgroups per compute unit.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_mfma64_kernel(const Params p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 16, TN = WTN / 16;
    static_assert(WTM % 16 == 0 && WTN % 16 == 0, "bad tile");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    double(*As)[BM * LDS_ROW] = (double(*)[BM * LDS_ROW])smem;                                      // [2][BM][LDS_ROW]
    double(*Bs)[BN * LDS_ROW] = (double(*)[BN * LDS_ROW])(smem + 2 * BM * LDS_ROW * sizeof(double)); // [2][BN][LDS_ROW]

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    const int l16 = lane % 16, lq = lane / 16;

    const int work = xcd_remap(blockIdx.x, p.total_blocks);
    const int batch = work / p.tiles_per_batch, tile = work % p.tiles_per_batch;
    const int bm0 = (tile % p.tiles_m) * BM, bn0 = (tile / p.tiles_m) * BN;
    const int ktiles = (p.k + BK - 1) / BK;
    const int iters = ktiles * p.kbatches;

    auto a_tile = [&](int it) -> const double * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch, kt = p.kbatches > 1 ? it % ktiles : it;
        return p.a + (int64_t)(kb / p.nb2) * p.a_b1 + (int64_t)(kb % p.nb2) * p.a_b2 + (int64_t)bm0 * p.a_rs + (int64_t)kt * BK * p.a_ks;
    };
    auto b_tile = [&](int it) -> const double * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch, kt = p.kbatches > 1 ? it % ktiles : it;
        return p.b + (int64_t)(kb / p.nb2) * p.b_b1 + (int64_t)(kb % p.nb2) * p.b_b2 + (int64_t)bn0 * p.b_cs + (int64_t)kt * BK * p.b_ks;
    };
    auto k_left = [&](int it) -> int { return p.k - (p.kbatches > 1 ? it % ktiles : it) * BK; };

    Loader<BM, NT, A_KC> la;
    Loader<BN, NT, B_KC> lb;
    f64x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

    if (iters > 0) {
        la.load(a_tile(0), p.a_rs, p.a_ks, p.m - bm0, k_left(0), tid);
        lb.load(b_tile(0), p.b_cs, p.b_ks, p.n - bn0, k_left(0), tid);
        la.store(As[0], tid);
        lb.store(Bs[0], tid);
    }
    __syncthreads();
    for (int it = 0; it < iters; it++) {
        const int cur = it & 1;
        const bool more = it + 1 < iters;
        if (more) {  // the next tile travels to registers while this one is multiplied
            la.load(a_tile(it + 1), p.a_rs, p.a_ks, p.m - bm0, k_left(it + 1), tid);
            lb.load(b_tile(it + 1), p.b_cs, p.b_ks, p.n - bn0, k_left(it + 1), tid);
        }
        const double *af = As[cur] + (wm0 + l16) * LDS_ROW + lq;
        const double *bf = Bs[cur] + (wn0 + l16) * LDS_ROW + lq;
#pragma unroll
        for (int ks = 0; ks < BK / 4; ks++) {
            double a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = af[i * 16 * LDS_ROW + ks * 4];
#pragma unroll
            for (int j = 0; j < TN; j++) b[j] = bf[j * 16 * LDS_ROW + ks * 4];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            la.store(As[cur ^ 1], tid);
            lb.store(Bs[cur ^ 1], tid);
        }
        __syncthreads();
    }

    // ---- epilogue: register r of tile (i, j) is C[wm0 + 16 i + 4 r + lq][wn0 + 16 j + l16] ----
    const int cb = p.kbatches > 1 ? 0 : batch;
    double *cbase = p.c + (int64_t)(cb / p.nb2) * p.c_b1 + (int64_t)(cb % p.nb2) * p.c_b2;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = bm0 + wm0 + i * 16 + 4 * r + lq;
            if (row >= p.m) continue;
            double *crow = cbase + (int64_t)row * p.ldc;
            const double rbias = p.bias_mode == BIAS_PER_ROW ? p.bias[row] : 0.0;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int col = bn0 + wn0 + j * 16 + l16;
                if (col >= p.n) continue;
                double v = acc[i][j][r] + rbias;
                if (p.bias_mode == BIAS_PER_COL) v += p.bias[col];
                if (p.accumulate) v += crow[col];
                crow[col] = v;
            }
        }
}

struct Variant {
    const char *name;
    int bm, bn;
};
constexpr Variant kVariants[] = {{"128x128x16_w2x4", 128, 128}, {"64x64x16_w2x2", 64, 64}};
constexpr int kNumVariants = 2;

template <int BM, int BN, int WM, int WN> hipError_t launch_layout(const Params &p, bool a_kc, bool b_kc, hipStream_t stream) {
    dim3 grid((unsigned)p.total_blocks), block(WM * WN * 64);
    constexpr size_t lds = (size_t)2 * (BM + BN) * LDS_ROW * sizeof(double);  // 69.6 KB for 128 x 128: above the static limit
#define DFDX_LAUNCH(AKC, BKC)                                                                                  \
    do {                                                                                                       \
        auto kern = gemm_mfma64_kernel<BM, BN, WM, WN, AKC, BKC>;                                              \
        static PerDevice configured_on;                                                                        \
        std::atomic<int> &configured = configured_on.here();                                                   \
        if (!configured.load(std::memory_order_acquire)) {                                                     \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                               (int)lds);                                                      \
            if (e != hipSuccess) return e;                                                                     \
            configured.store(1, std::memory_order_release);                                                    \
        }                                                                                                      \
        kern<<<grid, block, lds, stream>>>(p);                                                                 \
    } while (0)
    if (a_kc && b_kc) DFDX_LAUNCH(true, true);
    else if (a_kc) DFDX_LAUNCH(true, false);
    else if (b_kc) DFDX_LAUNCH(false, true);
    else DFDX_LAUNCH(false, false);
#undef DFDX_LAUNCH
    return hipGetLastError();
}

}  // namespace

// The last id is the small-product kernel (gemm_small.hip).
int mfma64_small_variant() { return kNumVariants + 1; }
int mfma64_variant_count() { return mfma64_small_variant(); }
const char *mfma64_variant_name(int v) {
    if (v == mfma64_small_variant()) return "small_16x16_ksliced";
    return (v >= 1 && v <= kNumVariants) ? kVariants[v - 1].name : "?";
}

// Row-major C (unit column stride); the operands may have any non-negative strides (every access is one element; the
// unit-stride axis only decides which access pattern coalesces).
bool mfma64_supported(const GemmProblem &p, int variant) {
    if (variant == mfma64_small_variant()) return p.dtype == DT_F64 && small_supported(p);
    if (p.dtype != DT_F64 || variant < 1 || variant > kNumVariants) return false;
    if (p.m < 1 || p.n < 1 || p.k < 1 || p.m >= (1 << 30) || p.n >= (1 << 30) || p.k >= (1 << 30)) return false;
    if (p.c_cs != 1 && p.n != 1) return false;
    if (p.n > 1 && p.m > 1 && p.c_rs < p.n) return false;
    if (p.a_rs < 0 || p.a_cs < 0 || p.b_rs < 0 || p.b_cs < 0) return false;
    if (p.nb1 * p.nb2 > 1 && (p.a_b1 < 0 || p.a_b2 < 0 || p.b_b1 < 0 || p.b_b2 < 0)) return false;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uintptr_t)p.c | (uintptr_t)p.bias) & 7u) return false;
    const Variant &v = kVariants[variant - 1];
    const int64_t tiles = ((p.m + v.bm - 1) / v.bm) * ((p.n + v.bn - 1) / v.bn);
    if (tiles * (p.reduce ? 1 : p.nb1 * p.nb2) >= (1ll << 31) || p.nb1 * p.nb2 >= (1ll << 31)) return false;
    if (p.k * (p.reduce ? p.nb1 * p.nb2 : 1) >= (1ll << 31)) return false;
    return true;
}

// The large tile once its workgroups fill half the chip, the small one below that.
int mfma64_pick_variant(const GemmProblem &p, int compute_units) {
    if (!mfma64_supported(p, 1)) return 0;
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t big = ((p.m + 127) / 128) * ((p.n + 127) / 128) * nbatch;
    return big * 2 >= compute_units ? 1 : 2;
}

// Estimated seconds of a tiled variant, for the comparison with the small-product kernel: a k tile of 16 takes a lone
// workgroup 1.25 us (64 x 64 tiles measure 9 / 14 / 24 / 44 / 84 us for k = 64 ... 1024), or its flops at the compute
// unit's share of 50 TFLOP/s once that is more.
double mfma64_time(const GemmProblem &p, int variant, int compute_units) {
    if (variant < 1 || variant > kNumVariants) return 1e300;
    const Variant &t = kVariants[variant - 1];
    const int cus = std::max(1, compute_units);
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const double blocks = (double)((p.m + t.bm - 1) / t.bm) * (double)((p.n + t.bn - 1) / t.bn) * (double)nbatch;
    const double steps = (double)((p.k + 15) / 16) * (double)(p.reduce ? p.nb1 * p.nb2 : 1);
    const double step = std::max(1.25e-6, 2.0 * t.bm * t.bn * 16 / (50e12 / 256));
    return 4e-6 + std::max(1.0, blocks / cus) * steps * step;
}

hipError_t launch_mfma64(const GemmProblem &g, int variant, hipStream_t stream) {
    if (!mfma64_supported(g, variant)) return hipErrorInvalidValue;
    if (variant == mfma64_small_variant()) return launch_small(g, stream);
    const Variant &v = kVariants[variant - 1];
    Params p;
    p.a = (const double *)g.a; p.b = (const double *)g.b; p.c = (double *)g.c; p.bias = (const double *)g.bias;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.a_rs = g.a_rs; p.a_ks = g.a_cs; p.b_cs = g.b_cs; p.b_ks = g.b_rs;
    p.ldc = g.m == 1 ? g.n : g.c_rs;
    p.a_b1 = g.a_b1; p.a_b2 = g.a_b2; p.b_b1 = g.b_b1; p.b_b2 = g.b_b2; p.c_b1 = g.c_b1; p.c_b2 = g.c_b2;
    p.nb2 = (int)g.nb2;
    const int nbatch = (int)(g.nb1 * g.nb2);
    p.kbatches = g.reduce ? nbatch : 1;
    p.tiles_m = (int)((g.m + v.bm - 1) / v.bm);
    p.tiles_n = (int)((g.n + v.bn - 1) / v.bn);
    p.tiles_per_batch = p.tiles_m * p.tiles_n;
    p.total_blocks = p.tiles_per_batch * (g.reduce ? 1 : nbatch);
    p.accumulate = g.accumulate;
    p.bias_mode = g.bias ? g.bias_mode : BIAS_NONE;
    // which operand axis has the unit stride decides the global access pattern only
    const bool a_kc = g.a_cs == 1 || g.k == 1, b_kc = g.b_rs == 1 || g.k == 1;
    return variant == 1 ? launch_layout<128, 128, 2, 4>(p, a_kc, b_kc, stream) : launch_layout<64, 64, 2, 2>(p, a_kc, b_kc, stream);
}

}  // namespace dfdx_rocm
