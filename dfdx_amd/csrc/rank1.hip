// Rank-1 updates: the products with a contraction of one, C = (accumulate ? C : 0) + bias + a (x) b.
//
// dfdx reaches them as vec (x) vec (an outer product is the (M,1).(1,N) product, dfdx-core/src/tensor_ops/matmul/mod.rs:139-144)
// and, far larger, as the weight gradient of every vec.mat / mat.vec product: grad_rhs += lhs^T . grad_out with one row on
// each side (cpu_kernel.rs:276-286 with m = 1).  There is nothing to contract: the launch streams C once (twice when it
// accumulates) and is bound by HBM, so it is an elementwise kernel and not a tile of a matrix-core kernel, whose 16 x 16 or
// 256 x 256 tiles write C in short row pieces (1.5 - 3 TB/s at 4096^2 against the 5 - 6 TB/s of whole rows).  A thread
// owns 16 bytes of columns, keeps its piece of b (and of a per-column bias) in registers and walks rows; the threads of a
// workgroup lie along a row as far as it reaches (4 KiB of C per row and workgroup when it is wide enough), the rest of
// them on further rows.  Product, bias and old value are added in f32 (f64 for f64) and rounded once.
#include "elem.h"
#include "gemm_internal.h"
#include <algorithm>

#pragma clang fp contract(off)  // product and sums are rounded apart, as the matrix-core kernels and the CPU path do

namespace dfdx_rocm {
namespace {

struct Rank1Params {
    const void *a, *b, *bias;
    void *c;
    int m, n;
    int64_t a_stride, b_stride, ldc;
    int accumulate, bias_mode;
    int tx_log2;  // threads of a workgroup along a row: 2^tx_log2 <= 256
    int rows_per_block;
};

// 16 bytes of a row of C as the computing type and back.  ALIGNED: the address is a multiple of 16; otherwise it is only
// element-aligned (an odd leading dimension or extent) and the access is one unaligned 16-byte load or store, which
// global memory allows.
template <typename T, bool ALIGNED> __device__ __forceinline__ void load_row_piece(const T *p, typename Acc<T>::type (&v)[Elem<T>::VEC]) {
    constexpr int N = Elem<T>::VEC;
    u32x4 raw;
    if constexpr (ALIGNED) raw = *(const u32x4 *)p;
    else raw = *(const u32x4_unaligned *)p;
    T tmp[N];
    __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
}
template <typename T, bool ALIGNED> __device__ __forceinline__ void store_row_piece(T *p, const typename Acc<T>::type (&v)[Elem<T>::VEC]) {
    constexpr int N = Elem<T>::VEC;
    T tmp[N];
#pragma unroll
    for (int i = 0; i < N; i++) Elem<T>::store(&tmp[i], v[i]);
    u32x4 raw;
    __builtin_memcpy(&raw, tmp, 16);
    if constexpr (ALIGNED) *(u32x4 *)p = raw;
    else *(u32x4_unaligned *)p = raw;
}

template <typename T, bool ALIGNED> __global__ __launch_bounds__(256) void rank1_kernel(const Rank1Params p) {
    typedef typename Acc<T>::type A;
    constexpr int N = Elem<T>::VEC;
    const int tx = 1 << p.tx_log2, ty = 256 >> p.tx_log2;
    const int col = ((int)blockIdx.y * tx + (int)(threadIdx.x & (tx - 1))) * N;
    if (col >= p.n) return;
    const int have = min(N, p.n - col);  // below N only in the last piece of a row whose length is no multiple of N
    A bv[N], cb[N];
#pragma unroll
    for (int e = 0; e < N; e++) {
        bv[e] = e < have ? (A)Elem<T>::load((const T *)p.b + (int64_t)(col + e) * p.b_stride) : A(0);
        cb[e] = (e < have && p.bias_mode == BIAS_PER_COL) ? (A)Elem<T>::load((const T *)p.bias + col + e) : A(0);
    }
    const int row0 = (int)blockIdx.x * p.rows_per_block + (int)(threadIdx.x >> p.tx_log2);
    const int row_end = min(p.m, ((int)blockIdx.x + 1) * p.rows_per_block);
    for (int row = row0; row < row_end; row += 2 * ty) {  // two rows in flight
        const int row2 = row + ty;
        const bool two = row2 < row_end;
        T *d0 = (T *)p.c + (int64_t)row * p.ldc + col, *d1 = (T *)p.c + (int64_t)row2 * p.ldc + col;
        const A a0 = Elem<T>::load((const T *)p.a + (int64_t)row * p.a_stride);
        const A a1 = two ? (A)Elem<T>::load((const T *)p.a + (int64_t)row2 * p.a_stride) : A(0);
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
                load_row_piece<T, ALIGNED>(d0, o0);
                if (two) load_row_piece<T, ALIGNED>(d1, o1);
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
            A v0 = a0 * bv[e], v1 = a1 * bv[e];
            v0 += cb[e]; v1 += cb[e];
            v0 += rb0; v1 += rb1;
            o0[e] = v0 + o0[e]; o1[e] = v1 + o1[e];
        }
        if (have == N) {
            store_row_piece<T, ALIGNED>(d0, o0);
            if (two) store_row_piece<T, ALIGNED>(d1, o1);
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
    // rows per thread: two at least (both in flight), sixteen at most, and about 2048 workgroups in between
    const int64_t passes = (g.m + ty - 1) / ty * blocks_y;
    const int per_thread = (int)std::min<int64_t>(16, std::max<int64_t>(2, passes / 2048 / 2 * 2));
    p.rows_per_block = ty * per_thread;
    const int64_t blocks_x = (g.m + p.rows_per_block - 1) / p.rows_per_block;
    if (blocks_y > 65535 || blocks_x >= (1ll << 31)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks_x, (unsigned)blocks_y);
    if (aligned) rank1_kernel<T, true><<<grid, 256, 0, stream>>>(p);
    else rank1_kernel<T, false><<<grid, 256, 0, stream>>>(p);
    return hipGetLastError();
}

}  // namespace

// One product per launch, both extents above one (a row or a column of C is a vector product), C row-major.
bool rank1_supported(const GemmProblem &g) {
    if (g.k != 1 || g.m < 2 || g.n < 2 || g.reduce || g.nb1 * g.nb2 != 1) return false;
    if (g.dtype < DT_F32 || g.dtype > DT_F64) return false;
    if (g.c_cs != 1 || g.c_rs < g.n) return false;
    if (g.m >= (1ll << 31) || g.n >= (1ll << 31)) return false;
    const int vec = (int)(16 / dtype_size(g.dtype));
    if (((g.n + vec - 1) / vec + 255) / 256 > 65535) return false;  // column blocks are grid.y
    const uintptr_t mask = dtype_size(g.dtype) - 1;
    return (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c | (uintptr_t)g.bias) & mask) == 0;
}

hipError_t launch_rank1(const GemmProblem &g, hipStream_t stream) {
    if (!rank1_supported(g)) return hipErrorInvalidValue;
    Rank1Params p;
    p.a = g.a; p.b = g.b; p.c = g.c; p.bias = g.bias;
    p.m = (int)g.m; p.n = (int)g.n;
    p.a_stride = g.a_rs; p.b_stride = g.b_cs; p.ldc = g.c_rs;
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
