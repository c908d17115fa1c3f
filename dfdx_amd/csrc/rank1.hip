// Rank-1 updates and thin contractions: the products with a contraction of one to eight,
// C = (accumulate ? C : 0) + bias + sum_k a[:, k] (x) b[k, :].
//
// dfdx reaches k = 1 as vec (x) vec (an outer product is the (M,1).(1,N) product, dfdx-core/src/tensor_ops/matmul/mod.rs:139-144)
// and, far larger, as the weight gradient of every vec.mat / mat.vec product: grad_rhs += lhs^T . grad_out with one row on
// each side (cpu_kernel.rs:276-286 with m = 1); k = 2 .. 8 as a Linear layer on a handful of input features and as the
// input gradient of a layer with a handful of outputs (grad_x = grad_y . W with W of 10 rows).  There is next to nothing to
// contract: the launch streams C once (twice when it accumulates) and is bound by HBM, so it is an elementwise kernel and
// not a tile of a matrix-core kernel, whose 16 x 16 or 256 x 256 tiles write C in short row pieces (1.5 - 3 TB/s at 4096^2
// against the 5 - 6 TB/s of whole rows).  A thread owns 16 bytes of columns, keeps its pieces of b's rows (and of a
// per-column bias) in registers and walks rows; the threads of a workgroup lie along a row as far as it reaches (4 KiB of
// C per row and workgroup when it is wide enough), the rest of them on further rows.  k = 1: product, bias and old value
// are added in f32 (f64 for f64) and rounded apart, like the matrix-core kernels and the CPU path; k > 1: the sum over k
// ascending by fused multiply-adds (beyond eight -- four for the 16-bit types -- the vector ALUs, not HBM, would bound the
// launch: the tiled kernels stay).
#include "elem.h"
#include "gemm_internal.h"
#include <algorithm>

#pragma clang fp contract(off)  // nothing is fused but what is written as a fused multiply-add below

namespace dfdx_rocm {
namespace {

struct Rank1Params {
    const void *a, *b, *bias;
    void *c;
    int m, n, k;
    int64_t a_stride, b_stride, ldc;  // along the rows of a, the columns of b, the rows of C
    int64_t a_k_stride, b_k_stride;
    int accumulate, bias_mode;
    int tx_log2;  // threads of a workgroup along a row: 2^tx_log2 <= 256
    int rows_per_block;
};

// 16 bytes of a row of C as the computing type and back.  ALIGNED: the address is a multiple of 16; otherwise it is only
// element-aligned (an odd leading dimension or extent) and the access is one unaligned 16-byte load or store, which
// global memory allows.
// STREAM (aligned rows only): the non-temporal forms, for an accumulation into 256 MiB of C or more -- read once, written
// once, too large to be found in the last-level cache by anybody (a weight gradient W += x (x) y on 16384^2: f32 414 ->
// 372 us, f16 197 -> 188 us; on a 4096^2 that is updated launch after launch the cached forms are faster, 10.1 against 11.5 us).
template <typename T, bool ALIGNED, bool STREAM = false>
__device__ __forceinline__ void load_row_piece(const T *p, typename Acc<T>::type (&v)[Elem<T>::VEC]) {
    constexpr int N = Elem<T>::VEC;
    u32x4 raw;
    if constexpr (ALIGNED && STREAM) raw = __builtin_nontemporal_load((const u32x4 *)p);
    else if constexpr (ALIGNED) raw = *(const u32x4 *)p;
    else raw = *(const u32x4_unaligned *)p;
    T tmp[N];
    __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
}
template <typename T, bool ALIGNED, bool STREAM = false>
__device__ __forceinline__ void store_row_piece(T *p, const typename Acc<T>::type (&v)[Elem<T>::VEC]) {
    constexpr int N = Elem<T>::VEC;
    T tmp[N];
#pragma unroll
    for (int i = 0; i < N; i++) Elem<T>::store(&tmp[i], v[i]);
    u32x4 raw;
    __builtin_memcpy(&raw, tmp, 16);
    if constexpr (ALIGNED && STREAM) __builtin_nontemporal_store(raw, (u32x4 *)p);
    else if constexpr (ALIGNED) *(u32x4 *)p = raw;
    else *(u32x4_unaligned *)p = raw;
}

__device__ __forceinline__ float fused(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fused(double a, double b, double c) { return __builtin_fma(a, b, c); }

constexpr int STAGED_A = 4096;  // values of a one workgroup keeps in LDS (k > 1): rows per workgroup x KMAX stays below

// KMAX: 1, or the power of two that holds k.
template <typename T, bool ALIGNED, int KMAX, bool STREAM = false> __global__ __launch_bounds__(256) void rank1_kernel(const Rank1Params p) {
    typedef typename Acc<T>::type A;
    constexpr int N = Elem<T>::VEC;
    const int tx = 1 << p.tx_log2, ty = 256 >> p.tx_log2;
    const int col = ((int)blockIdx.y * tx + (int)(threadIdx.x & (tx - 1))) * N;
    const int have = max(0, min(N, p.n - col));  // below N only at the end of a row whose length is no multiple of N
    // The rows of b over the workgroup's columns: gathered once by all its threads, neighbouring threads on neighbouring
    // addresses whichever way b is stored, and handed out through LDS (a thread that gathered its own 8 x KMAX values
    // would touch a cache line per lane and load where b is stored along k).  Every load goes to an address inside the
    // operand (indices clamped); what lies beyond the end is replaced by zero afterwards: no branch per value.
    A bv[KMAX][N], cb[N];
    const int block_row = (int)blockIdx.x * p.rows_per_block;
    __shared__ A sa[KMAX == 1 ? 1 : STAGED_A];
    if constexpr (KMAX == 1) {
#pragma unroll
        for (int e = 0; e < N; e++) {
            const A v = Elem<T>::load((const T *)p.b + (int64_t)min(col + e, p.n - 1) * p.b_stride);
            bv[0][e] = e < have ? v : A(0);
        }
    } else {
        __shared__ T sh[KMAX][256 * N];
        const int width = tx * N, col_first = (int)blockIdx.y * width;
        const bool along_k = p.b_k_stride == 1;  // the same in every lane: consecutive threads walk k first, or the columns
        for (int idx = threadIdx.x; idx < KMAX * width; idx += 256) {
            const int kk = along_k ? idx % KMAX : idx / width, j = along_k ? idx / KMAX : idx % width;
            const T v = *((const T *)p.b + (int64_t)min(kk, p.k - 1) * p.b_k_stride + (int64_t)min(col_first + j, p.n - 1) * p.b_stride);
            sh[kk][j] = v;
        }
        // ... and a's values for the workgroup's rows, zeros beyond k, so that the row loop below loads nothing but C
        const int rows_here = min(p.rows_per_block, p.m - block_row);
        const bool rows_first = p.a_stride == 1;  // a stored along its rows (the transposed operand of a weight gradient)
        for (int idx = threadIdx.x; idx < KMAX * rows_here; idx += 256) {
            const int kk = rows_first ? idx / rows_here : idx % KMAX, r = rows_first ? idx % rows_here : idx / KMAX;
            const A v = Elem<T>::load((const T *)p.a + (int64_t)(block_row + r) * p.a_stride + (int64_t)min(kk, p.k - 1) * p.a_k_stride);
            sa[r * KMAX + kk] = kk < p.k ? v : A(0);
        }
        __syncthreads();
        const int mine = (int)(threadIdx.x & (tx - 1)) * N;
#pragma unroll
        for (int kk = 0; kk < KMAX; kk++)
#pragma unroll
            for (int e = 0; e < N; e++) bv[kk][e] = (e < have && kk < p.k) ? (A)Elem<T>::load(&sh[kk][mine + e]) : A(0);
    }
#pragma unroll
    for (int e = 0; e < N; e++) cb[e] = A(0);
    if (p.bias_mode == BIAS_PER_COL) {
#pragma unroll
        for (int e = 0; e < N; e++) {
            const A v = Elem<T>::load((const T *)p.bias + min(col + e, p.n - 1));
            cb[e] = e < have ? v : A(0);
        }
    }
    if (have == 0) return;
    const int row0 = block_row + (int)(threadIdx.x >> p.tx_log2);
    const int row_end = min(p.m, ((int)blockIdx.x + 1) * p.rows_per_block);
    for (int row = row0; row < row_end; row += 2 * ty) {  // two rows in flight
        const int row2 = row + ty;
        const bool two = row2 < row_end;
        T *d0 = (T *)p.c + (int64_t)row * p.ldc + col, *d1 = (T *)p.c + (int64_t)row2 * p.ldc + col;
        A a0[KMAX], a1[KMAX];
        const int row2c = two ? row2 : row;
        if constexpr (KMAX == 1) {
            a0[0] = Elem<T>::load((const T *)p.a + (int64_t)row * p.a_stride);
            a1[0] = Elem<T>::load((const T *)p.a + (int64_t)row2c * p.a_stride);
        } else {
#pragma unroll
            for (int kk = 0; kk < KMAX; kk++) {
                a0[kk] = sa[(row - block_row) * KMAX + kk];
                a1[kk] = sa[(row2c - block_row) * KMAX + kk];
            }
        }
        A rb0 = 0, rb1 = 0;
        if (p.bias_mode == BIAS_PER_ROW) {
            rb0 = Elem<T>::load((const T *)p.bias + row);
            if (two) rb1 = Elem<T>::load((const T *)p.bias + row2);
        }
        A o0[N], o1[N];
#pragma unroll
        for (int e = 0; e < N; e++) o0[e] = o1[e] = 0;
        if (p.accumulate) {
            if (have == N) {
                load_row_piece<T, ALIGNED, STREAM>(d0, o0);
                if (two) load_row_piece<T, ALIGNED, STREAM>(d1, o1);
            } else {
#pragma unroll
                for (int e = 0; e < N; e++)
                    if (e < have) {
                        o0[e] = Elem<T>::load(d0 + e);
                        if (two) o1[e] = Elem<T>::load(d1 + e);
                    }
            }
        }
#pragma unroll
        for (int e = 0; e < N; e++) {
            A v0 = a0[0] * bv[0][e], v1 = a1[0] * bv[0][e];
#pragma unroll
            for (int kk = 1; kk < KMAX; kk++) {
                v0 = fused(a0[kk], bv[kk][e], v0);
                v1 = fused(a1[kk], bv[kk][e], v1);
            }
            v0 += cb[e]; v1 += cb[e];
            v0 += rb0; v1 += rb1;
            o0[e] = v0 + o0[e]; o1[e] = v1 + o1[e];
        }
        if (have == N) {
            store_row_piece<T, ALIGNED, STREAM>(d0, o0);
            if (two) store_row_piece<T, ALIGNED, STREAM>(d1, o1);
        } else {
#pragma unroll
            for (int e = 0; e < N; e++)
                if (e < have) {
                    Elem<T>::store(d0 + e, o0[e]);
                    if (two) Elem<T>::store(d1 + e, o1[e]);
                }
        }
    }
}

template <typename T> hipError_t launch_t(const Rank1Params &base, const GemmProblem &g, hipStream_t stream) {
    constexpr int VEC = Elem<T>::VEC;
    Rank1Params p = base;
    const bool aligned = p.ldc % VEC == 0 && ((uintptr_t)g.c & 15u) == 0;  // every row piece starts on a 16-byte boundary
    const int64_t pieces = (g.n + VEC - 1) / VEC;  // threads a row wants
    p.tx_log2 = 0;
    while (p.tx_log2 < 8 && (1ll << p.tx_log2) < pieces) p.tx_log2++;
    const int ty = 256 >> p.tx_log2;
    const int64_t blocks_y = (pieces + (1ll << p.tx_log2) - 1) >> p.tx_log2;
    // rows per thread: two (k = 1) or eight at least, sixteen at most, and about 2048 workgroups in between -- 1024 for the
    // 16-bit types, whose rows are half as many bytes (4096^2: 10.4 -> 9.3 us; not where unaligned rows are read back
    // as well, 4095 x 4097 with beta = 1: 13.0 against 13.7 us)
    const int64_t passes = (g.m + ty - 1) / ty * blocks_y;
    const int least = g.k > 1 ? 8 : 2;  // the b pieces a thread gathers first want more rows to pay for them
    const int64_t groups = (sizeof(T) == 2 && (aligned || !p.accumulate)) ? 1024 : 2048;
    const int per_thread = (int)std::min<int64_t>(16, std::max<int64_t>(least, passes / groups / 2 * 2));
    p.rows_per_block = ty * per_thread;
    if (g.k > 1) {  // the staged values of a: rows x KMAX within STAGED_A, an even number of rows per thread
        const int kmax = g.k == 2 ? 2 : g.k <= 4 ? 4 : 8;
        p.rows_per_block = std::min(p.rows_per_block, std::max(2 * ty, STAGED_A / kmax / (2 * ty) * (2 * ty)));
    }
    const int64_t blocks_x = (g.m + p.rows_per_block - 1) / p.rows_per_block;
    if (blocks_y > 65535 || blocks_x >= (1ll << 31)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks_x, (unsigned)blocks_y);
    const bool streamed = p.accumulate && (double)g.m * (double)g.n * (double)sizeof(T) >= 268435456.0;
#define DFDX_RANK(KMAX)                                                          \
    do {                                                                         \
        if (aligned && streamed) rank1_kernel<T, true, KMAX, true><<<grid, 256, 0, stream>>>(p); \
        else if (aligned) rank1_kernel<T, true, KMAX><<<grid, 256, 0, stream>>>(p); \
        else rank1_kernel<T, false, KMAX><<<grid, 256, 0, stream>>>(p);          \
    } while (0)
    if (g.k == 1) DFDX_RANK(1);
    else if (g.k == 2) DFDX_RANK(2);
    else if (g.k <= 4) DFDX_RANK(4);
    else DFDX_RANK(8);
#undef DFDX_RANK
    return hipGetLastError();
}

}  // namespace

// One product per launch, both extents above one (a row or a column of C is a vector product), C row-major.
bool rank1_supported(const GemmProblem &g) {
    if (g.dtype < DT_F32 || g.dtype > DT_F64) return false;
    // 16-bit elements: 8 columns per thread, and past k = 4 their multiply-adds cost what the stores do (65536 x 8 x 256:
    // 17.9 us here, 16.7 us on the matrix cores)
    const int kmost = (g.dtype == DT_F16 || g.dtype == DT_BF16) ? 4 : 8;
    if (g.k < 1 || g.k > kmost || g.m < 2 || g.n < 2 || g.reduce || g.nb1 * g.nb2 != 1) return false;
    if (g.c_cs != 1 || g.c_rs < g.n) return false;
    if (g.m >= (1ll << 30) || g.n >= (1ll << 30)) return false;  // 32-bit row and column indices with room for a block past the end
    const int vec = (int)(16 / dtype_size(g.dtype));
    if (((g.n + vec - 1) / vec + 255) / 256 > 65535) return false;  // column blocks are grid.y
    const uintptr_t mask = dtype_size(g.dtype) - 1;
    return (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c | (uintptr_t)g.bias) & mask) == 0;
}

hipError_t launch_rank1(const GemmProblem &g, hipStream_t stream) {
    if (!rank1_supported(g)) return hipErrorInvalidValue;
    Rank1Params p;
    p.a = g.a; p.b = g.b; p.c = g.c; p.bias = g.bias;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.a_stride = g.a_rs; p.b_stride = g.b_cs; p.ldc = g.c_rs;
    p.a_k_stride = g.a_cs; p.b_k_stride = g.b_rs;
    p.accumulate = g.accumulate;
    p.bias_mode = g.bias ? g.bias_mode : BIAS_NONE;
    p.tx_log2 = 0; p.rows_per_block = 0;
    switch (g.dtype) {
    case DT_F32: return launch_t<float>(p, g, stream);
    case DT_F16: return launch_t<_Float16>(p, g, stream);
    case DT_BF16: return launch_t<__bf16>(p, g, stream);
    case DT_F64: return launch_t<double>(p, g, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace dfdx_rocm
