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
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }  // RNE, quiet NaNs (v_cvt_pk_bf16_f32)
};

// The row sums that ride along with a split product (`ksum`, one value per row of C, `slots` partial sums each, stored
// [slot][row]).  The first `blocks` workgroups of grid row 0 do nothing else: each takes 16 rows; thread t adds the
// slots t / 16, t / 16 + 16, ... of row t % 16 in ascending order, four loads in flight at a time; the 16 partial sums
// of a row are added in a fixed order through LDS, then the old value unless the gradient is fresh.
struct KsumParts {
    const float *ws;   // null = none
    int64_t stride;
    void *out;
    int accumulate, slots, blocks;
};
constexpr int KSUM_ROWS = 16, KSUM_GROUPS = 256 / KSUM_ROWS;
template <typename T> __device__ __forceinline__ void combine_ksum(const KsumParts &ks, int m) {
    __shared__ float part[KSUM_GROUPS][KSUM_ROWS];
    const int r = threadIdx.x % KSUM_ROWS, g = threadIdx.x / KSUM_ROWS;
    const int row = min((int)blockIdx.x * KSUM_ROWS + r, m - 1);  // rows past the end repeat the last one, unused
    const float *src = ks.ws + row;
    float v = 0.0f;
    int s = g;
    for (; s + 3 * KSUM_GROUPS < ks.slots; s += 4 * KSUM_GROUPS) {
        const float a = src[(int64_t)s * ks.stride], b = src[(int64_t)(s + KSUM_GROUPS) * ks.stride];
        const float c = src[(int64_t)(s + 2 * KSUM_GROUPS) * ks.stride], d = src[(int64_t)(s + 3 * KSUM_GROUPS) * ks.stride];
        v = (((v + a) + b) + c) + d;
    }
    for (; s < ks.slots; s += KSUM_GROUPS) v += src[(int64_t)s * ks.stride];
    part[g][r] = v;
    __syncthreads();
    if (g == 0 && (int)blockIdx.x * KSUM_ROWS + r < m) {
#pragma unroll
        for (int q = 1; q < KSUM_GROUPS; q++) v += part[q][r];
        T *dst = (T *)ks.out + row;
        const float old = ks.accumulate ? Cvt<T>::load(dst) : 0.0f;
        Cvt<T>::store(dst, old + v);
    }
}

// one thread: 4 consecutive columns of one row
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *ws, int splits, int64_t ws_ld, int64_t ws_split_stride,
                                                            T *c, int64_t c_rs, int m, int n, int accumulate, int bias_mode,
                                                            const T *bias, int vec4, KsumParts ks) {
    if (ks.ws && (int)blockIdx.x < ks.blocks) {   // uniform over the workgroup
        if (blockIdx.y == 0) combine_ksum<T>(ks, m);
        return;   // the same block index in the other grid rows has no work
    }
    const int col = (blockIdx.y * 64 + threadIdx.x % 64) * 4;   // rows along grid.x: its limit is 2^31, grid.y's 65535
    const int row = ((int)blockIdx.x - (ks.ws ? ks.blocks : 0)) * 4 + threadIdx.x / 64;
    if (row >= m || col >= n) return;
    const float *src = ws + (int64_t)row * ws_ld + col;
    // eight partial sums requested at a time (a tail repeats the last one, unused), added in ascending order: one round
    // trip to memory per eight splits instead of one per split
    f32x4 v;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        f32x4 part[8];
#pragma unroll
        for (int u = 0; u < 8; u++) part[u] = *(const f32x4 *)(src + (int64_t)min(s0 + u, splits - 1) * ws_split_stride);
        if (s0 == 0) v = part[0];
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (s0 + u < splits && s0 + u > 0) v += part[u];
    }
    T *dst = c + (int64_t)row * c_rs + col;
    const float rb = (bias_mode == BIAS_PER_ROW) ? Cvt<T>::load(bias + row) : 0.0f;
    if constexpr (sizeof(T) == 4) {
        if (vec4 && col + 3 < n) {   // f32 rows aligned to 16 B: one load of the old values, one store
            f32x4 x = v + rb;
            if (bias_mode == BIAS_PER_COL) x += *(const f32x4 *)(bias + col);
            if (accumulate) x += *(const f32x4 *)dst;
            *(f32x4 *)dst = x;
            return;
        }
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
        if (col + e >= n) break;
        float x = v[e] + rb;
        if (bias_mode == BIAS_PER_COL) x += Cvt<T>::load(bias + col + e);
        if (accumulate) x += Cvt<T>::load(dst + e);
        Cvt<T>::store(dst + e, x);
    }
}

// 16-bit outputs whose rows are 16 B-aligned: one thread owns 8 consecutive columns of one row -- two 16 B loads per
// split, requested four splits at a time, the old C values (beta = 1) requested before the first partial arrives, one
// 16 B store.  Same order of additions per element as the general kernel: splits ascending, row bias, column bias, old C.
template <typename T> struct Bits16;
template <> struct Bits16<_Float16> {
    static __device__ __forceinline__ float widen(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ uint16_t narrow(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};
template <> struct Bits16<__bf16> {
    static __device__ __forceinline__ float widen(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
    static __device__ __forceinline__ uint16_t narrow(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }  // RNE, quiet NaNs
};
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce16_kernel(const float *ws, int splits, int64_t ws_ld, int64_t ws_split_stride,
                                                              uint16_t *c, int64_t c_rs, int m, int n, int accumulate,
                                                              int bias_mode, const uint16_t *bias, KsumParts ks) {
    if (ks.ws && (int)blockIdx.x < ks.blocks) {   // uniform over the workgroup
        if (blockIdx.y == 0) combine_ksum<T>(ks, m);
        return;   // the same block index in the other grid rows has no work
    }
    const int col = (blockIdx.y * 64 + threadIdx.x % 64) * 8;
    const int row = ((int)blockIdx.x - (ks.ws ? ks.blocks : 0)) * 4 + threadIdx.x / 64;
    if (row >= m || col >= n) return;   // n is a multiple of 8: a thread's 8 columns are all inside or all outside
    const float *src = ws + (int64_t)row * ws_ld + col;
    uint16_t *dst = c + (int64_t)row * c_rs + col;
    u32x4 old = {0u, 0u, 0u, 0u}, cb = {0u, 0u, 0u, 0u};
    if (accumulate) old = *(const u32x4 *)dst;
    if (bias_mode == BIAS_PER_COL) cb = *(const u32x4 *)(bias + col);
    // eight splits requested at a time (a tail repeats the last one, unused) and added in ascending order: with the old
    // C values and the bias that is ONE round trip to memory for up to eight splits (a loop that waited for split after
    // split paid five for eight splits: 9.2 us for the 1024 x 1024 weight gradients)
    f32x4 lo, hi;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        f32x4 a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float *q = src + (int64_t)min(s0 + u, splits - 1) * ws_split_stride;
            a[u] = *(const f32x4 *)q;
            b[u] = *(const f32x4 *)(q + 4);
        }
        if (s0 == 0) {
            lo = a[0];
            hi = b[0];
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (s0 + u < splits && s0 + u > 0) {
                lo += a[u];
                hi += b[u];
            }
    }
    const float rb = (bias_mode == BIAS_PER_ROW) ? Bits16<T>::widen(bias[row]) : 0.0f;
    u32x4 out;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        float x = (e < 4 ? lo[e] : hi[e - 4]) + rb;
        const int sh = (e & 1) * 16;
        if (bias_mode == BIAS_PER_COL) x += Bits16<T>::widen((uint16_t)(cb[e / 2] >> sh));
        if (accumulate) x += Bits16<T>::widen((uint16_t)(old[e / 2] >> sh));
        const uint32_t bits = Bits16<T>::narrow(x);
        out[e / 2] = (e & 1) ? (out[e / 2] | (bits << 16)) : bits;
    }
    *(u32x4 *)dst = out;
}

}  // namespace

// C of `p` must have unit column stride and no batch (the planner only splits such problems).
hipError_t launch_splitk_reduce(const GemmProblem &p, int64_t ws_ld, int64_t ws_split_stride, hipStream_t stream,
                                const float *ws_ksum, int64_t ws_ksum_stride, int ksum_slots) {
    const bool with_ksum = p.ksum && ws_ksum;
    const KsumParts ks{with_ksum ? ws_ksum : nullptr, ws_ksum_stride, p.ksum, p.ksum_accumulate, ksum_slots,
                       with_ksum ? (int)((p.m + KSUM_ROWS - 1) / KSUM_ROWS) : 0};
    dim3 grid((unsigned)((p.m + 3) / 4 + ks.blocks), (unsigned)((p.n + 255) / 256)), block(256);
    if ((p.n + 255) / 256 > 65535) return hipErrorInvalidValue;  // 16.7 M columns: no planner splits such a product
    const int64_t c_rs = p.m == 1 ? p.n : p.c_rs;
    const int bias_mode = p.bias ? p.bias_mode : BIAS_NONE;
    const bool is16 = p.dtype == DT_F16 || p.dtype == DT_BF16;
    if (is16 && p.n % 8 == 0 && c_rs % 8 == 0 && ws_ld % 4 == 0 && ws_split_stride % 4 == 0 && ((uintptr_t)p.c & 15u) == 0 &&
        ((uintptr_t)p.workspace & 15u) == 0 && (bias_mode != BIAS_PER_COL || ((uintptr_t)p.bias & 15u) == 0)) {
        dim3 grid16((unsigned)((p.m + 3) / 4 + ks.blocks), (unsigned)((p.n + 511) / 512));
        if (p.dtype == DT_F16)
            splitk_reduce16_kernel<_Float16><<<grid16, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (uint16_t *)p.c,
                                                                            c_rs, (int)p.m, (int)p.n, p.accumulate, bias_mode,
                                                                            (const uint16_t *)p.bias, ks);
        else
            splitk_reduce16_kernel<__bf16><<<grid16, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (uint16_t *)p.c,
                                                                          c_rs, (int)p.m, (int)p.n, p.accumulate, bias_mode,
                                                                          (const uint16_t *)p.bias, ks);
        return hipGetLastError();
    }
    const int vec4 = p.dtype == DT_F32 && c_rs % 4 == 0 && ((uintptr_t)p.c & 15u) == 0 && ws_ld % 4 == 0 && ws_split_stride % 4 == 0 &&
                     ((uintptr_t)p.workspace & 15u) == 0 && (bias_mode != BIAS_PER_COL || ((uintptr_t)p.bias & 15u) == 0);
    switch (p.dtype) {
    case DT_F32:
        splitk_reduce_kernel<float><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (float *)p.c, c_rs,
                                                                 (int)p.m, (int)p.n, p.accumulate, bias_mode, (const float *)p.bias, vec4, ks);
        break;
    case DT_F16:
        splitk_reduce_kernel<_Float16><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (_Float16 *)p.c,
                                                                    c_rs, (int)p.m, (int)p.n, p.accumulate, bias_mode,
                                                                    (const _Float16 *)p.bias, 0, ks);
        break;
    case DT_BF16:
        splitk_reduce_kernel<__bf16><<<grid, block, 0, stream>>>(p.workspace, p.splits, ws_ld, ws_split_stride, (__bf16 *)p.c, c_rs,
                                                                  (int)p.m, (int)p.n, p.accumulate, bias_mode, (const __bf16 *)p.bias, 0, ks);
        break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace dfdx_rocm
