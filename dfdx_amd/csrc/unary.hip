// Multiplication by a scalar (`t * s`, a unary op in dfdx): forward over the physical storage of the tensor,
// backward grad_inp += s * grad_out.  The scalar is rounded to the element type first, as the reference holds it
// in that type.
#include "ctx_internal.h"
#include "elem.h"

namespace dfdx_rocm {
namespace {

// ACC: out[i] += s * x[i] (backward), else out[i] = s * x[i]
template <typename T, int N, bool ACC>
__global__ __launch_bounds__(256) void scalar_mul_kernel(const T *x, T *out, int64_t groups, float s) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float v[N];
        load_elems<T, N>(x + g * N, v);
        if constexpr (ACC) {
            float o[N];
            load_elems<T, N>(out + g * N, o);
#pragma unroll
            for (int i = 0; i < N; i++) v[i] = o[i] + s * v[i];
        } else {
#pragma unroll
            for (int i = 0; i < N; i++) v[i] *= s;
        }
        store_elems<T, N>(out + g * N, v);
    }
}

template <typename T> float round_scalar(double s) {
    T tmp;
    float f = (float)s;
    if constexpr (sizeof(T) == 4) return f;
    else if constexpr (std::is_same<T, _Float16>::value) {
        tmp = (_Float16)f;
        return (float)tmp;
    } else {
        uint32_t x;
        __builtin_memcpy(&x, &f, 4);
        x = (x + 0x7fffu + ((x >> 16) & 1u)) & 0xffff0000u;
        __builtin_memcpy(&f, &x, 4);
        return f;
    }
}

template <typename T, bool ACC> int launch_t(dfdx_rocm_ctx *ctx, int64_t len, const void *x, double scalar, void *out) {
    constexpr int V = Elem<T>::VEC;
    const bool vec = len % V == 0 && (((uintptr_t)x | (uintptr_t)out) & 15u) == 0;
    const int64_t groups = vec ? len / V : len;
    const unsigned grid = (unsigned)std::min<int64_t>((groups + 255) / 256, (int64_t)ctx->compute_units * 16);
    const float s = round_scalar<T>(scalar);
    if (vec) scalar_mul_kernel<T, V, ACC><<<grid, 256, 0, ctx->stream>>>((const T *)x, (T *)out, groups, s);
    else scalar_mul_kernel<T, 1, ACC><<<grid, 256, 0, ctx->stream>>>((const T *)x, (T *)out, groups, s);
    return (int)hipGetLastError();
}

template <bool ACC> int dispatch(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, double scalar, void *out) {
    if (int e = bind(ctx)) return e;
    if (len < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (len == 0) return DFDX_ROCM_OK;
    if (!x || !out) return DFDX_ROCM_ERR_INVALID_ARG;
    switch (dtype) {
    case DFDX_ROCM_F32: return launch_t<float, ACC>(ctx, len, x, scalar, out);
    case DFDX_ROCM_F16: return launch_t<_Float16, ACC>(ctx, len, x, scalar, out);
    case DFDX_ROCM_BF16: return launch_t<__bf16, ACC>(ctx, len, x, scalar, out);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

}  // namespace
}  // namespace dfdx_rocm

extern "C" {

int dfdx_rocm_scalar_mul_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, double scalar, void *out) {
    return dfdx_rocm::dispatch<false>(ctx, dtype, len, x, scalar, out);
}

int dfdx_rocm_scalar_mul_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, double scalar, void *grad_inp,
                                  const void *grad_out) {
    return dfdx_rocm::dispatch<true>(ctx, dtype, len, grad_out, scalar, grad_inp);
}

}  // extern "C"
