// Element types of the elementwise / reduction kernels: storage <-> f32 conversion, 16-byte vector access.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace dfdx_rocm {

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;  // elements per 16 bytes
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Elem<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float load(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct Elem<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float load(const __bf16 *p) {
        return __uint_as_float((uint32_t)(*(const uint16_t *)p) << 16);
    }
    // round to nearest even, quiet NaNs: the hardware conversion (v_cvt_pk_bf16_f32)
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }
};

// f64 takes part in the plain (row-walking) kernels only: no 16-byte vector path, f64 arithmetic throughout.
template <> struct Elem<double> {
    static constexpr int VEC = 2;
    static __device__ __forceinline__ double load(const double *p) { return *p; }
    static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
};
// The type a kernel computes in: f32 for the 16- and 32-bit element types, f64 for f64.
template <typename T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

// Sum / maximum over the 64 lanes of a wave, every lane receiving the result, without the LDS crossbar (`__shfl_xor` is a
// ds_bpermute per step): four DPP steps inside the 16-lane rows (two quad permutations, the half-row and the row
// mirror), then the rows pairwise and the wave's halves through v_permlane16_swap / v_permlane32_swap.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);  // row_half_mirror
    return v + dpp_move<0x140>(v);  // row_mirror
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    return fmaxf(v, dpp_move<0x140>(v));
}
__device__ __forceinline__ float wave64_sum(float v) {
    v = row16_sum(v);
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);  // rows (0,0,2,2) and (1,1,3,3)
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);      // (lower, lower) and (upper, upper)
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float wave64_max(float v) {
    v = row16_max(v);
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// N consecutive elements as f32; N == Elem<T>::VEC moves 16 bytes at once (p must then be 16-byte aligned).
template <typename T, int N> __device__ __forceinline__ void load_elems(const T *p, float (&v)[N]) {
    if constexpr (N == Elem<T>::VEC) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 raw = *(const u32x4 *)p;
        T tmp[N];
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
    } else {
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = Elem<T>::load(p + i);
    }
}
// The same with the non-temporal form of the 16-byte load (STREAM): for an input that one launch reads once and that is
// large enough (the callers' rule: 128 MiB or more of read-only input) to push what later ops want out of the caches if it
// were kept there.  Measured on MI355X in an encoder block (softmax and ReLU gradients of 134 MB tensors): the step as a
// whole gains 1.2 %, mostly in the GEMMs that run next; small inputs that the previous op has just written lose with it
// (LayerNorm forward on 16 MB 8.0 -> 10.4 us), hence the size rule.  A compile-time choice: written as a run-time select
// of the two loads, the compiler merges them into one plain load.
template <typename T, int N, bool STREAM> __device__ __forceinline__ void load_elems_as(const T *p, float (&v)[N]) {
    if constexpr (STREAM && N == Elem<T>::VEC) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 raw = __builtin_nontemporal_load((const u32x4 *)p);
        T tmp[N];
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
    } else {
        load_elems<T, N>(p, v);
    }
}
constexpr size_t kStreamInputBytes = (size_t)128 << 20;  // read-only input of one launch from which its loads are non-temporal
// The same from an address that is only element-aligned (one unaligned 16-byte load; global memory allows it).
template <typename T, int N> __device__ __forceinline__ void load_elems_unaligned(const T *p, float (&v)[N]) {
    if constexpr (N == Elem<T>::VEC) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));
        const u32x4 raw = *(const u32x4_unaligned *)p;
        T tmp[N];
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
    } else {
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = Elem<T>::load(p + i);
    }
}
template <typename T, int N> __device__ __forceinline__ void store_elems(T *p, const float (&v)[N]) {
    if constexpr (N == Elem<T>::VEC) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        T tmp[N];
#pragma unroll
        for (int i = 0; i < N; i++) Elem<T>::store(&tmp[i], v[i]);
        u32x4 raw;
        __builtin_memcpy(&raw, tmp, 16);
        *(u32x4 *)p = raw;
    } else {
#pragma unroll
        for (int i = 0; i < N; i++) Elem<T>::store(p + i, v[i]);
    }
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));

// A 16-byte vector moved by `bits` towards element 0 (bits > 0) or away from it (bits < 0), zeros moving in.
__device__ __forceinline__ u32x4 shift128(u32x4 r, int bits) {
    uint64_t lo = r[0] | ((uint64_t)r[1] << 32), hi = r[2] | ((uint64_t)r[3] << 32);
    if (bits >= 0) {
        const unsigned s = (unsigned)bits;
        if (s >= 64) { lo = hi; hi = 0; }
        const unsigned t = s & 63;
        if (t) { lo = (lo >> t) | (hi << (64 - t)); hi >>= t; }
        if (s >= 128) lo = 0;
    } else {
        const unsigned s = (unsigned)(-bits);
        if (s >= 64) { hi = lo; lo = 0; }
        const unsigned t = s & 63;
        if (t) { hi = (hi << t) | (lo >> (64 - t)); lo <<= t; }
        if (s >= 128) hi = 0;
    }
    return u32x4{(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}
// 16 bytes of elements (ELEM_BYTES each) of one image row starting at column x0, zeros outside [0, width): one
// (unaligned) vector load from the nearest window inside the row, then a shift -- no per-element path for the lanes at
// the image border, which a wave would otherwise execute in full next to the vector path of its interior lanes.
// width >= 16 / ELEM_BYTES.
template <int ELEM_BYTES> __device__ __forceinline__ u32x4 row_window_bytes(const void *row, bool row_ok, int x0, int width) {
    constexpr int N = 16 / ELEM_BYTES;
    const int x0c = min(max(x0, 0), width - N);
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (row_ok) raw = *(const u32x4_unaligned *)((const char *)row + (int64_t)x0c * ELEM_BYTES);
    return shift128(raw, (x0 - x0c) * (8 * ELEM_BYTES));
}
template <typename T> __device__ __forceinline__ u32x4 row_window(const T *row, bool row_ok, int x0, int width) {
    return row_window_bytes<(int)sizeof(T)>(row, row_ok, x0, width);
}

}  // namespace dfdx_rocm
