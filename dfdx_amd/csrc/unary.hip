// Elementwise ops over the physical storage of a tensor, forward and backward (gradients accumulate):
//   * multiplication by a scalar (`t * s`, a unary op in dfdx); the scalar is rounded to the element type first, as
//     the reference holds it in that type;
//   * ReLU;
//   * the binary add of two tensors of one shape (ResidualAdd).
#include "ctx_internal.h"
#include "elem.h"

namespace dfdx_rocm {
namespace {

// ACC: out[i] += s * x[i] (backward; `fresh`: out counts as zero and is not read), else out[i] = s * x[i]
template <typename T, int N, bool ACC, bool STREAM>
__global__ __launch_bounds__(256) void scalar_mul_kernel(const T *x, T *out, int64_t groups, float s, bool fresh) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float v[N];
        load_elems_as<T, N, STREAM>(x + g * N, v);
        if constexpr (ACC) {
            float o[N];
            if (fresh) {
#pragma unroll
                for (int i = 0; i < N; i++) o[i] = 0.0f;
            } else {
                load_elems<T, N>(out + g * N, o);
            }
#pragma unroll
            for (int i = 0; i < N; i++) v[i] = o[i] + s * v[i];
        } else {
#pragma unroll
            for (int i = 0; i < N; i++) v[i] *= s;
        }
        store_elems<T, N>(out + g * N, v);
    }
}

// out = max(x, 0)
template <typename T, int N, bool STREAM> __global__ __launch_bounds__(256) void relu_forward_kernel(const T *x, T *out, int64_t groups) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float v[N];
        load_elems_as<T, N, STREAM>(x + g * N, v);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], 0.0f);
        store_elems<T, N>(out + g * N, v);
    }
}

// grad_x += (x > 0 ? 1 : 0) * grad_out; `fresh`: grad_x counts as zero and is not read
template <typename T, int N, bool STREAM>
__global__ __launch_bounds__(256) void relu_backward_kernel(const T *x, const T *go, T *gx, int64_t groups, bool fresh) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float v[N], d[N], o[N];
        load_elems_as<T, N, STREAM>(x + g * N, v);
        load_elems_as<T, N, STREAM>(go + g * N, d);
        if (fresh) {
#pragma unroll
            for (int i = 0; i < N; i++) o[i] = 0.0f;
        } else {
            load_elems<T, N>(gx + g * N, o);
        }
#pragma unroll
        for (int i = 0; i < N; i++) o[i] += v[i] > 0.0f ? d[i] : 0.0f;
        store_elems<T, N>(gx + g * N, o);
    }
}

// out = a + b
template <typename T, int N, bool STREAM> __global__ __launch_bounds__(256) void add_forward_kernel(const T *a, const T *b, T *out, int64_t groups) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float v[N], w[N];
        load_elems_as<T, N, STREAM>(a + g * N, v);
        load_elems_as<T, N, STREAM>(b + g * N, w);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] += w[i];
        store_elems<T, N>(out + g * N, v);
    }
}

// grad_lhs += grad_out, grad_rhs += grad_out (two distinct buffers); fresh_l / fresh_r: that one counts as zero, not read
template <typename T, int N, bool STREAM>
__global__ __launch_bounds__(256) void add_backward_kernel(const T *go, T *gl, T *gr, int64_t groups, bool fresh_l, bool fresh_r) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        float d[N], l[N], r[N];
        load_elems_as<T, N, STREAM>(go + g * N, d);
#pragma unroll
        for (int i = 0; i < N; i++) l[i] = r[i] = 0.0f;
        if (!fresh_l) load_elems<T, N>(gl + g * N, l);
        if (!fresh_r) load_elems<T, N>(gr + g * N, r);
#pragma unroll
        for (int i = 0; i < N; i++) {
            l[i] += d[i];
            r[i] += d[i];
        }
        store_elems<T, N>(gl + g * N, l);
        store_elems<T, N>(gr + g * N, r);
    }
}

// ---- f64: the reference's fourth element type (its CI runs every test in f64 as well); plain kernels, f64 arithmetic
enum { F64_SCALE, F64_SCALE_ACC, F64_RELU_FWD, F64_RELU_BWD, F64_ADD_FWD, F64_ADD_BWD };
template <int OP>
__global__ __launch_bounds__(256) void unary_f64_kernel(const double *a, const double *b, double *c, double *d, int64_t len, double s,
                                                        bool fresh_c, bool fresh_d) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < len; i += (int64_t)gridDim.x * 256) {
        if constexpr (OP == F64_SCALE) c[i] = s * a[i];
        else if constexpr (OP == F64_SCALE_ACC) c[i] = (fresh_c ? 0.0 : c[i]) + s * a[i];
        else if constexpr (OP == F64_RELU_FWD) c[i] = fmax(a[i], 0.0);
        else if constexpr (OP == F64_RELU_BWD) c[i] = (fresh_c ? 0.0 : c[i]) + (a[i] > 0.0 ? b[i] : 0.0);
        else if constexpr (OP == F64_ADD_FWD) c[i] = a[i] + b[i];
        else {
            const double g = a[i];
            c[i] = (fresh_c ? 0.0 : c[i]) + g;
            d[i] = (fresh_d ? 0.0 : d[i]) + g;
        }
    }
}
template <int OP>
int launch_f64(dfdx_rocm_ctx *ctx, int64_t len, const void *a, const void *b, void *c, void *d, double s, bool fresh_c, bool fresh_d) {
    const unsigned grid = (unsigned)std::min<int64_t>((len + 255) / 256, (int64_t)ctx->compute_units * 16);
    unary_f64_kernel<OP><<<grid, 256, 0, ctx->stream>>>((const double *)a, (const double *)b, (double *)c, (double *)d, len, s, fresh_c, fresh_d);
    return (int)hipGetLastError();
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

template <typename T, bool ACC> int launch_t(dfdx_rocm_ctx *ctx, int64_t len, const void *x, double scalar, void *out, bool fresh) {
    constexpr int V = Elem<T>::VEC;
    const bool vec = len % V == 0 && (((uintptr_t)x | (uintptr_t)out) & 15u) == 0;
    const int64_t groups = vec ? len / V : len;
    const unsigned grid = (unsigned)std::min<int64_t>((groups + 255) / 256, (int64_t)ctx->compute_units * 16);
    const float s = round_scalar<T>(scalar);
    const bool stream = (size_t)len * sizeof(T) >= kStreamInputBytes;
    if (vec && stream) scalar_mul_kernel<T, V, ACC, true><<<grid, 256, 0, ctx->stream>>>((const T *)x, (T *)out, groups, s, fresh);
    else if (vec) scalar_mul_kernel<T, V, ACC, false><<<grid, 256, 0, ctx->stream>>>((const T *)x, (T *)out, groups, s, fresh);
    else scalar_mul_kernel<T, 1, ACC, false><<<grid, 256, 0, ctx->stream>>>((const T *)x, (T *)out, groups, s, fresh);
    return (int)hipGetLastError();
}

template <bool ACC> int dispatch(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, double scalar, void *out) {
    if (int e = bind(ctx)) return e;
    if (len < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (len == 0) return DFDX_ROCM_OK;
    if (!x || !out) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    bool fresh = false;  // a gradient whose zero fill is still deferred: stored without being read
    if (int e = settle(ctx, x)) return e;
    if (int e = settle_output(ctx, out, (size_t)len * (dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2), ACC, &fresh)) return e;
    switch (dtype) {
    case DFDX_ROCM_F64: return launch_f64<ACC ? F64_SCALE_ACC : F64_SCALE>(ctx, len, x, nullptr, out, nullptr, scalar, fresh, false);
    case DFDX_ROCM_F32: return launch_t<float, ACC>(ctx, len, x, scalar, out, fresh);
    case DFDX_ROCM_F16: return launch_t<_Float16, ACC>(ctx, len, x, scalar, out, fresh);
    case DFDX_ROCM_BF16: return launch_t<__bf16, ACC>(ctx, len, x, scalar, out, fresh);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

enum { OP_RELU_FWD, OP_RELU_BWD, OP_ADD_FWD, OP_ADD_BWD };

// a, b: read-only inputs (b unused by OP_RELU_FWD); c, d: written (d only by OP_ADD_BWD)
template <typename T, int OP>
int launch_op(dfdx_rocm_ctx *ctx, int64_t len, const void *a, const void *b, void *c, void *d, bool fresh_c, bool fresh_d) {
    constexpr int V = Elem<T>::VEC;
    const bool vec = len % V == 0 && (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)d) & 15u) == 0;
    const int64_t groups = vec ? len / V : len;
    const unsigned grid = (unsigned)std::min<int64_t>((groups + 255) / 256, (int64_t)ctx->compute_units * 16);
    hipStream_t s = ctx->stream;
    constexpr int INPUTS = (OP == OP_RELU_BWD || OP == OP_ADD_FWD) ? 2 : 1;  // read-only operands of the op
    const bool stream = vec && (size_t)len * sizeof(T) * INPUTS >= kStreamInputBytes;
#define DFDX_OP(N, STREAM)                                                                                                       \
    do {                                                                                                                 \
        if constexpr (OP == OP_RELU_FWD) relu_forward_kernel<T, N, STREAM><<<grid, 256, 0, s>>>((const T *)a, (T *)c, groups);    \
        else if constexpr (OP == OP_RELU_BWD) relu_backward_kernel<T, N, STREAM><<<grid, 256, 0, s>>>((const T *)a, (const T *)b, (T *)c, groups, fresh_c); \
        else if constexpr (OP == OP_ADD_FWD) add_forward_kernel<T, N, STREAM><<<grid, 256, 0, s>>>((const T *)a, (const T *)b, (T *)c, groups);    \
        else add_backward_kernel<T, N, STREAM><<<grid, 256, 0, s>>>((const T *)a, (T *)c, (T *)d, groups, fresh_c, fresh_d);      \
    } while (0)
    if (stream) DFDX_OP(V, true);
    else if (vec) DFDX_OP(V, false);
    else DFDX_OP(1, false);
#undef DFDX_OP
    return (int)hipGetLastError();
}

template <int OP> int dispatch_op(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *a, const void *b, void *c, void *d) {
    if (int e = bind(ctx)) return e;
    if (len < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (len == 0) return DFDX_ROCM_OK;
    if (!a || !c || (OP != OP_RELU_FWD && OP != OP_ADD_BWD && !b) || (OP == OP_ADD_BWD && !d)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    bool fresh_c = false, fresh_d = false;  // gradients whose zero fill is still deferred: stored without being read
    constexpr bool BWD = OP == OP_RELU_BWD || OP == OP_ADD_BWD;
    const size_t bytes = (size_t)len * (dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2);
    if (int e = settle(ctx, a)) return e;
    if (int e = settle(ctx, b)) return e;
    if (int e = settle_output(ctx, c, bytes, BWD, &fresh_c)) return e;
    if (int e = settle_output(ctx, d, bytes, BWD, &fresh_d)) return e;
    switch (dtype) {
    case DFDX_ROCM_F64:
        return launch_f64<OP == OP_RELU_FWD ? F64_RELU_FWD : OP == OP_RELU_BWD ? F64_RELU_BWD : OP == OP_ADD_FWD ? F64_ADD_FWD : F64_ADD_BWD>(
            ctx, len, a, b, c, d, 0.0, fresh_c, fresh_d);
    case DFDX_ROCM_F32: return launch_op<float, OP>(ctx, len, a, b, c, d, fresh_c, fresh_d);
    case DFDX_ROCM_F16: return launch_op<_Float16, OP>(ctx, len, a, b, c, d, fresh_c, fresh_d);
    case DFDX_ROCM_BF16: return launch_op<__bf16, OP>(ctx, len, a, b, c, d, fresh_c, fresh_d);
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

int dfdx_rocm_relu_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, void *out) {
    return dfdx_rocm::dispatch_op<dfdx_rocm::OP_RELU_FWD>(ctx, dtype, len, x, nullptr, out, nullptr);
}

int dfdx_rocm_relu_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, void *grad_x, const void *grad_out) {
    return dfdx_rocm::dispatch_op<dfdx_rocm::OP_RELU_BWD>(ctx, dtype, len, x, grad_out, grad_x, nullptr);
}

int dfdx_rocm_add_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *lhs, const void *rhs, void *out) {
    return dfdx_rocm::dispatch_op<dfdx_rocm::OP_ADD_FWD>(ctx, dtype, len, lhs, rhs, out, nullptr);
}

int dfdx_rocm_add_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, void *grad_lhs, void *grad_rhs, const void *grad_out) {
    if (grad_lhs && grad_lhs == grad_rhs) {  // t + t: the one buffer receives grad_out twice, one add after the other
        if (int e = dfdx_rocm::dispatch<true>(ctx, dtype, len, grad_out, 1.0, grad_lhs)) return e;
        return dfdx_rocm::dispatch<true>(ctx, dtype, len, grad_out, 1.0, grad_lhs);
    }
    return dfdx_rocm::dispatch_op<dfdx_rocm::OP_ADD_BWD>(ctx, dtype, len, grad_out, nullptr, grad_lhs, grad_rhs);
}

}  // extern "C"
