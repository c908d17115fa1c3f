// Combines split-k partial sums: C = (accumulate ? C : 0) + bias + sum over splits of the f32 partial tiles,
// splits added in ascending order (deterministic), one rounding to the storage type on store.
#include "gemm_internal.h"

namespace dfdx_rocm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Cvt;
template <> struct Cvt<float> {
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Cvt<_Float16> {
    static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct Cvt<__bf16> {
    static __device__ __forceinline__ float load(const __bf16 *p) { return __uint_as_float((uint32_t)(*(const uint16_t *)p) << 16); }
    static __device__ __forceinline__ void store(__bf16 *p, float v) {
        uint32_t x = __float_as_uint(v);
        uint16_t r = ((x & 0x7fffffffu) > 0x7f800000u) ? (uint16_t)((x >> 16) | 0x40u)
                                                       : (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
        *(uint16_t *)p = r;
    }
};

// one thread: 4 consecutive columns of one row
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *ws, int splits, int64_t ws_ld, int64_t ws_split_stride,
                                                            T *c, int64_t c_rs, int m, int n, int accumulate, int bias_mode,
                                                            const T *bias) {
    const int col = (blockIdx.x * 64 + threadIdx.x % 64) * 4;
    const int row = blockIdx.y * 4 + threadIdx.x / 64;
    if (row >= m || col >= n) return;
    const float *src = ws + (int64_t)row * ws_ld + col;
    f32x4 v = *(const f32x4 *)src;
    for (int s = 1; s < splits; s++) v += *(const f32x4 *)(src + s * ws_split_stride);
    T *dst = c + (int64_t)row * c_rs + col;
    const float rb = (bias_mode == BIAS_PER_ROW) ? Cvt<T>::load(bias + row) : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        if (col + e >= n) break;
        float x = v[e] + rb;
        if (bias_mode == BIAS_PER_COL) x += Cvt<T>::load(bias + col + e);
        if (accumulate) x += Cvt<T>::load(dst + e);
        Cvt<T>::store(dst + e, x);
    }
}

}  // namespace

// C of `p` must have unit column stride and no batch (the planner only splits such problems).
hipError_t launch_splitk_reduce(const GemmProblem &p, int64_t ws_ld, int64_t ws_split_stride, hipStream_t stream) {
    dim3 grid((unsigned)((p.n + 255) / 256), (unsigned)((p.m + 3) / 4)), block(256);
    const int64_t c_rs = p.m == 1 ? p.n : p.c_rs;
    const int bias_mode = p.bias ? p.bias_mode : BIAS_NONE;
    switch (p.dtype) {
    case DT_F32:
        splitk_reduce_kernel<float><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (float *)p.c, c_rs,
                                                                 (int)p.m, (int)p.n, p.accumulate, bias_mode, (const float *)p.bias);
        break;
    case DT_F16:
        splitk_reduce_kernel<_Float16><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (_Float16 *)p.c,
                                                                    c_rs, (int)p.m, (int)p.n, p.accumulate, bias_mode,
                                                                    (const _Float16 *)p.bias);
        break;
    case DT_BF16:
        splitk_reduce_kernel<__bf16><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (__bf16 *)p.c, c_rs,
                                                                  (int)p.m, (int)p.n, p.accumulate, bias_mode, (const __bf16 *)p.bias);
        break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace dfdx_rocm
