// Bandwidth-bound vector products: (1,K).(K,N) and (M,K).(K,1), i.e. dfdx's vec.mat and mat.vec
// (rank-1 operands are reshapes to M = 1 / N = 1, dfdx-core/src/tensor_ops/matmul/mod.rs:147-175).
// Both are one kernel family over  out[j] = sum_k vec[k] * mat[k, j]  with the matrix streamed exactly once
// from HBM in 16 B pieces:
//   "cols" kernel  matrix rows are contiguous in j (vec.mat with row-major rhs): a thread owns VEC adjacent
//                  outputs, the 4 waves of a workgroup take interleaved k, workgroups along grid.y take k slices;
//   "dots" kernel  matrix is contiguous in k (mat.vec with row-major lhs, vec.mat with a permuted weight):
//                  one wave per output, lanes stride over k, wave-level reduction.
// Partial sums of k slices go to a small f32 workspace and are combined in slice order (deterministic).
#include "gemm_internal.h"

namespace dfdx_rocm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elt;
template <> struct Elt<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
    static __device__ __forceinline__ void unpack(u32x4 r, float (&o)[4]) {
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = __uint_as_float(r[i]);
    }
};
template <> struct Elt<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
    static __device__ __forceinline__ void unpack(u32x4 r, float (&o)[8]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r[i] & 0xffffu));
            o[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r[i] >> 16));
        }
    }
};
template <> struct Elt<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float load(const __bf16 *p) { return __uint_as_float((uint32_t)(*(const uint16_t *)p) << 16); }
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }  // RNE, quiet NaNs (v_cvt_pk_bf16_f32)
    static __device__ __forceinline__ void unpack(u32x4 r, float (&o)[8]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o[2 * i] = __uint_as_float(r[i] << 16);
            o[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
};

// A 16-byte load of the matrix; `stream` = non-temporal.  A matrix of 256 MiB or more cannot stay in the last-level cache
// between two products, and read this way it does not sweep the cache either: 16384^2 f16 95 -> 82 us (5.6 -> 6.6 TB/s),
// f32 180 -> 163 us, on one buffer set and over rotating sets alike.  Below that size the cached form keeps a matrix that
// fits the cache there for the next product (4096^2 f16 launch after launch: 4.8 us cached, 7.6 us streamed).
template <bool STREAM> __device__ __forceinline__ u32x4 ldm(const void *p) {
    if constexpr (STREAM) return __builtin_nontemporal_load((const u32x4 *)p);
    else return *(const u32x4 *)p;
}
constexpr size_t kStreamMatrixBytes = (size_t)256 << 20;

struct Params {
    const void *vec;
    const void *mat;
    void *out;
    const void *bias;
    int64_t vec_stride, mat_k_stride, mat_j_stride, out_stride, bias_stride;
    int k, j;
    int kslices, kchunk;  // grid.y slices of kchunk k values each
    int stream;           // the matrix is read with non-temporal loads (see ldm): picks the STREAM instance
    int accumulate, has_bias;
    float *ws;            // [kslices][j] partial sums when kslices > 1
};

template <typename T> __device__ __forceinline__ void finish(const Params &p, int j, float v) {
    T *dst = (T *)p.out + (int64_t)j * p.out_stride;
    if (p.has_bias) v += Elt<T>::load((const T *)p.bias + (int64_t)j * p.bias_stride);
    if (p.accumulate) v += Elt<T>::load(dst);
    Elt<T>::store(dst, v);
}

constexpr int KCHUNK_MAX = 2048;

// matrix contiguous in j: thread owns VEC outputs; block = 4 waves sharing 64*VEC outputs, interleaved in k
template <typename T, bool STREAM> __global__ __launch_bounds__(256) void gemv_cols_kernel(const Params p) {
    constexpr int VEC = Elt<T>::VEC;
    __shared__ float vsh[KCHUNK_MAX];
    __shared__ float red[4][64 * VEC];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int j0 = (blockIdx.x * 64 + lane) * VEC;
    const int k0 = blockIdx.y * p.kchunk;
    const int kn = min(p.kchunk, p.k - k0);
    for (int i = tid; i < kn; i += 256) vsh[i] = Elt<T>::load((const T *)p.vec + (int64_t)(k0 + i) * p.vec_stride);
    __syncthreads();
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = 0.f;
    if (j0 < p.j) {  // j % VEC == 0: the whole vector is in range
        const T *col = (const T *)p.mat + (int64_t)k0 * p.mat_k_stride + j0;
        int kk = wave;
        for (; kk + 12 < kn; kk += 16) {  // 4 loads in flight
            u32x4 r[4];
#pragma unroll
            for (int u = 0; u < 4; u++) r[u] = ldm<STREAM>(col + (int64_t)(kk + 4 * u) * p.mat_k_stride);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                float x[VEC];
                Elt<T>::unpack(r[u], x);
                const float v = vsh[kk + 4 * u];
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[e] += v * x[e];
            }
        }
        for (; kk < kn; kk += 4) {
            float x[VEC];
            Elt<T>::unpack(ldm<STREAM>(col + (int64_t)kk * p.mat_k_stride), x);
            const float v = vsh[kk];
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] += v * x[e];
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) red[wave][lane * VEC + e] = acc[e];
    __syncthreads();
    for (int o = tid; o < 64 * VEC; o += 256) {
        const int j = blockIdx.x * 64 * VEC + o;
        if (j >= p.j) continue;
        const float v = ((red[0][o] + red[1][o]) + red[2][o]) + red[3][o];
        if (p.kslices > 1) p.ws[(int64_t)blockIdx.y * p.j + j] = v;
        else finish<T>(p, j, v);
    }
}

// matrix contiguous in k: one wave per output, 16 B per lane per step
template <typename T, bool STREAM> __global__ __launch_bounds__(256) void gemv_dots_kernel(const Params p) {
    constexpr int VEC = Elt<T>::VEC;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int j = blockIdx.x * 4 + wave;
    if (j >= p.j) return;
    const int k0 = blockIdx.y * p.kchunk;
    const int kn = min(p.kchunk, p.k - k0);  // multiple of VEC
    const T *row = (const T *)p.mat + (int64_t)j * p.mat_j_stride + k0;
    const T *vec = (const T *)p.vec + k0;     // unit stride (checked on the host)
    float acc = 0.f;
    for (int kk = lane * VEC; kk < kn; kk += 64 * VEC) {
        float x[VEC], v[VEC];
        Elt<T>::unpack(ldm<STREAM>(row + kk), x);
        Elt<T>::unpack(*(const u32x4 *)(vec + kk), v);
#pragma unroll
        for (int e = 0; e < VEC; e++) acc += x[e] * v[e];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) {
        if (p.kslices > 1) p.ws[(int64_t)blockIdx.y * p.j + j] = acc;
        else finish<T>(p, j, acc);
    }
}

// Eight lanes per output: lane `part` adds the slices part, part + 8, ... (their loads in flight together), then the
// eight partial sums meet in a fixed tree of three exchanges: one round trip to the workspace for up to 64 slices.
template <typename T> __global__ __launch_bounds__(256) void gemv_combine_kernel(const Params p) {
    const int j = blockIdx.x * 32 + threadIdx.x / 8, part = threadIdx.x % 8;
    const bool in = j < p.j;
    const float *src = p.ws + (in ? j : 0);
    float v = 0.0f;
    for (int s = part; s < p.kslices; s += 64) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = (s + 8 * u < p.kslices) ? src[(int64_t)(s + 8 * u) * p.j] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) v += t[u];
    }
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    if (in && part == 0) finish<T>(p, j, v);
}

struct Shape {
    bool ok, cols;
    Params p;
};

inline bool al16(const void *q) { return ((uintptr_t)q & 15u) == 0; }

Shape classify(const GemmProblem &g) {
    Shape s{};
    if (g.dtype == DT_F64 || g.reduce || g.nb1 * g.nb2 != 1 || g.k < 1 || g.k >= (1ll << 31)) return s;
    if (g.m != 1 && g.n != 1) return s;
    if (g.m == 1 && g.n == 1) return s;  // a dot product: the generic kernel is fine
    Params &p = s.p;
    const int vec = g.dtype == DT_F32 ? 4 : 8;
    if (g.m == 1) {  // out[j] = sum_k a[k] b[k, j]
        p.vec = g.a; p.vec_stride = g.a_cs;
        p.mat = g.b; p.mat_k_stride = g.b_rs; p.mat_j_stride = g.b_cs;
        p.out = g.c; p.out_stride = g.c_cs;
        p.j = (int)g.n;
        p.bias_stride = (g.bias_mode == BIAS_PER_COL) ? 1 : 0;
    } else {  // out[i] = sum_k a[i, k] b[k]
        p.vec = g.b; p.vec_stride = g.b_rs;
        p.mat = g.a; p.mat_k_stride = g.a_cs; p.mat_j_stride = g.a_rs;
        p.out = g.c; p.out_stride = g.c_rs;
        p.j = (int)g.m;
        p.bias_stride = (g.bias_mode == BIAS_PER_ROW) ? 1 : 0;
    }
    if (g.n >= (1ll << 31) || g.m >= (1ll << 31)) return s;
    p.k = (int)g.k;
    p.bias = g.bias;
    p.has_bias = g.bias && g.bias_mode != BIAS_NONE;
    p.accumulate = g.accumulate;
    p.stream = (size_t)g.k * (size_t)p.j * (g.dtype == DT_F32 ? 4 : 2) >= kStreamMatrixBytes;
    if (p.out_stride < 1 && p.j > 1) return s;
    if (!al16(p.mat)) return s;
    if (p.mat_j_stride == 1 && p.j % vec == 0 && p.mat_k_stride % vec == 0 && p.mat_k_stride >= p.j) {
        s.ok = true; s.cols = true;
    } else if (p.mat_k_stride == 1 && p.k % vec == 0 && p.mat_j_stride % vec == 0 && p.mat_j_stride >= p.k &&
               p.vec_stride == 1 && al16(p.vec)) {
        s.ok = true; s.cols = false;
    }
    return s;
}

// k slices so that the grid has a few workgroups per compute unit
void plan_slices(Shape &s, int dtype) {
    Params &p = s.p;
    const int vec = dtype == DT_F32 ? 4 : 8;
    const int64_t blocks_j = s.cols ? (p.j + 64 * vec - 1) / (64 * vec) : (p.j + 3) / 4;
    int slices = 1;
    if (s.cols) {
        slices = (p.k + KCHUNK_MAX - 1) / KCHUNK_MAX;  // the vector slice must fit the LDS buffer
        while (blocks_j * slices < 512 && p.k / (slices * 2) >= 128) slices *= 2;
    } else {
        while (blocks_j * slices < 512 && p.k / (slices * 2) >= 64 * vec) slices *= 2;
    }
    int chunk = (p.k + slices - 1) / slices;
    chunk = (chunk + vec - 1) / vec * vec;
    if (s.cols && chunk > KCHUNK_MAX) chunk = KCHUNK_MAX;
    p.kchunk = chunk;
    p.kslices = (p.k + chunk - 1) / chunk;
}

template <typename T> hipError_t launch_t(const Shape &s, hipStream_t stream) {
    const Params &p = s.p;
    constexpr int VEC = Elt<T>::VEC;
    if (s.cols) {
        dim3 grid((unsigned)((p.j + 64 * VEC - 1) / (64 * VEC)), (unsigned)p.kslices);
        if (p.stream) gemv_cols_kernel<T, true><<<grid, 256, 0, stream>>>(p);
        else gemv_cols_kernel<T, false><<<grid, 256, 0, stream>>>(p);
    } else {
        dim3 grid((unsigned)((p.j + 3) / 4), (unsigned)p.kslices);
        if (p.stream) gemv_dots_kernel<T, true><<<grid, 256, 0, stream>>>(p);
        else gemv_dots_kernel<T, false><<<grid, 256, 0, stream>>>(p);
    }
    if (p.kslices > 1) gemv_combine_kernel<T><<<dim3((unsigned)((p.j + 31) / 32)), 256, 0, stream>>>(p);
    return hipGetLastError();
}

}  // namespace

bool gemv_supported(const GemmProblem &g) {
    Shape s = classify(g);
    if (!s.ok) return false;
    plan_slices(s, g.dtype);
    return s.p.kslices <= 65535;  // the k slices are grid.y; beyond its limit the product goes to another kernel
}

size_t gemv_workspace_bytes(const GemmProblem &g) {
    Shape s = classify(g);
    if (!s.ok) return 0;
    plan_slices(s, g.dtype);
    return s.p.kslices > 1 ? (size_t)s.p.kslices * s.p.j * sizeof(float) : 0;
}

hipError_t launch_gemv(const GemmProblem &g, hipStream_t stream) {
    Shape s = classify(g);
    if (!s.ok) return hipErrorInvalidValue;
    plan_slices(s, g.dtype);
    if (s.p.kslices > 1 && !g.workspace) return hipErrorInvalidValue;
    s.p.ws = g.workspace;
    switch (g.dtype) {
    case DT_F32: return launch_t<float>(s, stream);
    case DT_F16: return launch_t<_Float16>(s, stream);
    case DT_BF16: return launch_t<__bf16>(s, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace dfdx_rocm
