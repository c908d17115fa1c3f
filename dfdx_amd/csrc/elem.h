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
    static __device__ __forceinline__ void store(__bf16 *p, float v) {  // round to nearest even, quiet NaNs
        const uint32_t x = __float_as_uint(v);
        const uint16_t r = ((x & 0x7fffffffu) > 0x7f800000u) ? (uint16_t)((x >> 16) | 0x40u)
                                                             : (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
        *(uint16_t *)p = r;
    }
};

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

}  // namespace dfdx_rocm
