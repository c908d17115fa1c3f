// Generic strided GEMM: the correctness workhorse.  Any dtype, any stride pattern
// (doubly strided, broadcast inputs), any size incl. M/N/K = 1 and K = 0; batch
// offsets in 64 bit.  LDS-tiled 64x64x16, 256 threads, 4x4 outputs per thread,
// k summed in ascending order in f32 (f64 for f64 storage).
#include "gemm_internal.h"
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

namespace dfdx_rocm {
namespace {

template <typename T> struct Conv;
template <> struct Conv<float> {
    using Acc = float;
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Conv<double> {
    using Acc = double;
    static __device__ __forceinline__ double load(const double *p) { return *p; }
    static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
};
template <> struct Conv<_Float16> {
    using Acc = float;
    static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }  // RNE
};
template <> struct Conv<__bf16> {
    using Acc = float;
    static __device__ __forceinline__ float load(const __bf16 *p) {
        return __uint_as_float((uint32_t)(*(const uint16_t *)p) << 16);
    }
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }  // RNE, quiet NaNs (v_cvt_pk_bf16_f32)
};

constexpr int GT = 64;  // tile edge
constexpr int GK = 16;  // k step

template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmProblem p, int tiles_n, int tiles_per_batch) {
    using Acc = typename Conv<T>::Acc;
    __shared__ Acc as[GK][GT + 1];
    __shared__ Acc bs[GK][GT + 1];

    const int tid = threadIdx.x;
    const int64_t pid = blockIdx.x;
    const int64_t batch = pid / tiles_per_batch;
    const int tile = (int)(pid % tiles_per_batch);
    const int64_t row0 = (int64_t)(tile / tiles_n) * GT;
    const int64_t col0 = (int64_t)(tile % tiles_n) * GT;
    const int tx = tid % 16, ty = tid / 16;

    Acc acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (Acc)0;

    const int64_t nbatch = p.nb1 * p.nb2;
    const int64_t b_begin = p.reduce ? 0 : batch;
    const int64_t b_end = p.reduce ? nbatch : batch + 1;
    for (int64_t bi = b_begin; bi < b_end; bi++) {
        const int64_t b1 = bi / p.nb2, b2 = bi % p.nb2;
        const T *ap = (const T *)p.a + b1 * p.a_b1 + b2 * p.a_b2;
        const T *bp = (const T *)p.b + b1 * p.b_b1 + b2 * p.b_b2;
        for (int64_t k0 = 0; k0 < p.k; k0 += GK) {
            // A tile: 64 rows x 16 k ; B tile: 16 k x 64 cols ; 1024 elements each, 4 per thread
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int idx = e * 256 + tid;
                {   // A: consecutive threads walk k fastest when a_cs is the small stride, rows otherwise
                    const int kk = (p.a_cs <= p.a_rs) ? idx % GK : idx / GT;
                    const int r = (p.a_cs <= p.a_rs) ? idx / GK : idx % GT;
                    const int64_t gi = row0 + r, gk = k0 + kk;
                    as[kk][r] = (gi < p.m && gk < p.k) ? Conv<T>::load(ap + gi * p.a_rs + gk * p.a_cs) : (Acc)0;
                }
                {
                    const int kk = (p.b_rs <= p.b_cs) ? idx % GK : idx / GT;
                    const int c = (p.b_rs <= p.b_cs) ? idx / GK : idx % GT;
                    const int64_t gj = col0 + c, gk = k0 + kk;
                    bs[kk][c] = (gj < p.n && gk < p.k) ? Conv<T>::load(bp + gk * p.b_rs + gj * p.b_cs) : (Acc)0;
                }
            }
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < GK; kk++) {
                Acc av[4], bv[4];
#pragma unroll
                for (int i = 0; i < 4; i++) av[i] = as[kk][ty + 16 * i];
#pragma unroll
                for (int j = 0; j < 4; j++) bv[j] = bs[kk][tx + 16 * j];
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[i][j] += av[i] * bv[j];
            }
            __syncthreads();
        }
    }

    const int64_t cb1 = p.reduce ? 0 : batch / p.nb2, cb2 = p.reduce ? 0 : batch % p.nb2;
    T *cp = (T *)p.c + cb1 * p.c_b1 + cb2 * p.c_b2;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int64_t gi = row0 + ty + 16 * i;
        if (gi >= p.m) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t gj = col0 + tx + 16 * j;
            if (gj >= p.n) continue;
            Acc v = acc[i][j];
            if (p.bias_mode == BIAS_PER_COL) v += Conv<T>::load((const T *)p.bias + gj);
            else if (p.bias_mode == BIAS_PER_ROW) v += Conv<T>::load((const T *)p.bias + gi);
            T *dst = cp + gi * p.c_rs + gj * p.c_cs;
            if (p.accumulate) v += Conv<T>::load(dst);
            Conv<T>::store(dst, v);
        }
    }
}

}  // namespace

hipError_t launch_generic(const GemmProblem &p, hipStream_t stream) {
    if (p.m <= 0 || p.n <= 0) return hipSuccess;
    const int64_t tiles_m = (p.m + GT - 1) / GT, tiles_n = (p.n + GT - 1) / GT;
    const int64_t tiles = tiles_m * tiles_n;
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t blocks = tiles * nbatch;
    if (tiles > 0x7fffffff || blocks > 0x7fffffff) return hipErrorInvalidValue;
    dim3 grid((unsigned)blocks), block(256);
    switch (p.dtype) {
    case DT_F32: gemm_generic_kernel<float><<<grid, block, 0, stream>>>(p, (int)tiles_n, (int)tiles); break;
    case DT_F16: gemm_generic_kernel<_Float16><<<grid, block, 0, stream>>>(p, (int)tiles_n, (int)tiles); break;
    case DT_BF16: gemm_generic_kernel<__bf16><<<grid, block, 0, stream>>>(p, (int)tiles_n, (int)tiles); break;
    case DT_F64: gemm_generic_kernel<double><<<grid, block, 0, stream>>>(p, (int)tiles_n, (int)tiles); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace dfdx_rocm
