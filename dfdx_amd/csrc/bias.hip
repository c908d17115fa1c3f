// Bias1D on the device: the broadcast add of a (cols,) bias over the rows of a contiguous (rows, cols) matrix,
// and its backward, the column sum of grad_out accumulated into grad_bias.  Both are HBM-bound: one read (and for
// the forward one write) of the matrix.
#include "ctx_internal.h"
#include "elem.h"

namespace dfdx_rocm {
namespace {

// ---- forward: out[r][c] = x[r][c] + bias[c] ------------------------------------------------------------------
// One thread per N consecutive columns, grid-stride over the matrix; cols % N == 0.
template <typename T, int N>
__global__ __launch_bounds__(256) void bias_forward_kernel(const T *x, const T *bias, T *out, int64_t groups, int groups_per_row) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        const int c = (int)(g % groups_per_row) * N;
        float v[N], b[N];
        load_elems<T, N>(x + g * N, v);
        load_elems<T, N>(bias + c, b);
#pragma unroll
        for (int i = 0; i < N; i++) v[i] += b[i];
        store_elems<T, N>(out + g * N, v);
    }
}

// ---- backward: grad_bias[c] += sum_r grad_out[r][c] ----------------------------------------------------------
// A workgroup owns a strip of LPR * N columns and one slice of the rows.  LPR lanes cover the strip (256 bytes of
// a row when N is a 16-byte vector), the other 256 / LPR lane groups walk the rows of the slice; their partial
// sums meet in LDS and are added in a fixed order.  With several row slices the strip sums go to an f32 workspace
// [slices][cols] and a second kernel adds them, again in a fixed order, so the result does not depend on timing.
template <typename T, int N, int LPR>
__global__ __launch_bounds__(256) void bias_backward_kernel(const T *go, int rows, int cols, int rows_per_slice,
                                                            float *partial, T *grad_bias, bool fresh) {
    constexpr int RL = 256 / LPR;  // row lanes
    __shared__ float red[RL][LPR * N + 1];
    const int c_lane = threadIdx.x % LPR, r_lane = threadIdx.x / LPR;
    const int col = (blockIdx.x * LPR + c_lane) * N;
    const int r0 = blockIdx.y * rows_per_slice, r1 = min(rows, r0 + rows_per_slice);
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; i++) acc[i] = 0.0f;
    if (col < cols) {
        const T *src = go + (int64_t)col;
        int r = r0 + r_lane;
        for (; r + 3 * RL < r1; r += 4 * RL) {  // four independent loads in flight
            float v0[N], v1[N], v2[N], v3[N];
            load_elems<T, N>(src + (int64_t)r * cols, v0);
            load_elems<T, N>(src + (int64_t)(r + RL) * cols, v1);
            load_elems<T, N>(src + (int64_t)(r + 2 * RL) * cols, v2);
            load_elems<T, N>(src + (int64_t)(r + 3 * RL) * cols, v3);
#pragma unroll
            for (int i = 0; i < N; i++) acc[i] += (v0[i] + v1[i]) + (v2[i] + v3[i]);
        }
        for (; r < r1; r += RL) {
            float v[N];
            load_elems<T, N>(src + (int64_t)r * cols, v);
#pragma unroll
            for (int i = 0; i < N; i++) acc[i] += v[i];
        }
    }
#pragma unroll
    for (int i = 0; i < N; i++) red[r_lane][c_lane * N + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < LPR * N) {
        const int c = blockIdx.x * LPR * N + threadIdx.x;
        if (c < cols) {
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < RL; j++) s += red[j][threadIdx.x];
            if (partial) partial[(int64_t)blockIdx.y * cols + c] = s;
            else Elem<T>::store(grad_bias + c, (fresh ? 0.0f : Elem<T>::load(grad_bias + c)) + s);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(64) void bias_backward_combine_kernel(const float *partial, int slices, int cols, T *grad_bias, bool fresh) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= cols) return;
    const float *src = partial + c;
    float s = 0.0f;
    int j = 0;
    for (; j + 8 <= slices; j += 8) {  // eight loads in flight, added in slice order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = src[(int64_t)(j + u) * cols];
#pragma unroll
        for (int u = 0; u < 8; u++) s += v[u];
    }
    for (; j < slices; j++) s += src[(int64_t)j * cols];
    Elem<T>::store(grad_bias + c, (fresh ? 0.0f : Elem<T>::load(grad_bias + c)) + s);
}

// ---- f64 (the reference runs its whole test suite in f64 as well): plain kernels, f64 arithmetic -----------------
__global__ __launch_bounds__(256) void bias_forward_f64_kernel(const double *x, const double *bias, double *out, int64_t total, int64_t cols) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) out[i] = x[i] + bias[i % cols];
}
// One thread per column walks the rows in order (the order of the reference's row-after-row adds), neighbouring
// threads read neighbouring columns.
__global__ __launch_bounds__(256) void bias_backward_f64_kernel(const double *go, int64_t rows, int64_t cols, double *grad_bias, bool fresh) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    double s = fresh ? 0.0 : grad_bias[c];
    for (int64_t r = 0; r < rows; r++) s += go[r * cols + c];
    grad_bias[c] = s;
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T>
int bias_forward_t(dfdx_rocm_ctx *ctx, int64_t rows, int64_t cols, const void *x, const void *bias, void *out) {
    constexpr int V = Elem<T>::VEC;
    const bool vec = cols % V == 0 && aligned16(x) && aligned16(bias) && aligned16(out);
    const int n = vec ? V : 1;
    const int64_t groups = rows * cols / n;
    const int64_t want = (groups + 255) / 256;
    const unsigned grid = (unsigned)std::min<int64_t>(want, (int64_t)ctx->compute_units * 8);
    if (vec) bias_forward_kernel<T, V><<<grid, 256, 0, ctx->stream>>>((const T *)x, (const T *)bias, (T *)out, groups, (int)(cols / V));
    else bias_forward_kernel<T, 1><<<grid, 256, 0, ctx->stream>>>((const T *)x, (const T *)bias, (T *)out, groups, (int)cols);
    return (int)hipGetLastError();
}

template <typename T>
int bias_backward_t(dfdx_rocm_ctx *ctx, int64_t rows, int64_t cols, const void *go, void *gb, bool fresh) {
    constexpr int V = Elem<T>::VEC;
    const bool vec = cols % V == 0 && aligned16(go);
    constexpr int LPR_VEC = 16, LPR_SCALAR = 64;
    const int strip = vec ? LPR_VEC * V : LPR_SCALAR;
    const int row_lanes = 256 / (vec ? LPR_VEC : LPR_SCALAR);
    const int64_t strips = (cols + strip - 1) / strip;
    // two workgroups per compute unit, but at least 8 rows per lane group and slice
    int64_t slices = std::max<int64_t>(1, (int64_t)ctx->compute_units * 2 / strips);
    slices = std::min<int64_t>(slices, std::max<int64_t>(1, rows / (8 * row_lanes)));
    slices = std::min<int64_t>(slices, 65535);
    const int64_t rows_per_slice = (rows + slices - 1) / slices;
    slices = (rows + rows_per_slice - 1) / rows_per_slice;
    CtxLock lock(ctx->mu);  // two launches around the shared workspace
    float *partial = nullptr;
    if (slices > 1) {
        if (int rc = ensure_workspace(ctx, (size_t)slices * cols * sizeof(float))) return rc;
        partial = (float *)ctx->workspace;
    }
    dim3 grid((unsigned)strips, (unsigned)slices);
    if (vec)
        bias_backward_kernel<T, V, LPR_VEC><<<grid, 256, 0, ctx->stream>>>((const T *)go, (int)rows, (int)cols, (int)rows_per_slice, partial, (T *)gb, fresh);
    else
        bias_backward_kernel<T, 1, LPR_SCALAR><<<grid, 256, 0, ctx->stream>>>((const T *)go, (int)rows, (int)cols, (int)rows_per_slice, partial, (T *)gb, fresh);
    HIP_TRY(hipGetLastError());
    if (slices > 1) {
        bias_backward_combine_kernel<T><<<(unsigned)((cols + 63) / 64), 64, 0, ctx->stream>>>(partial, (int)slices, (int)cols, (T *)gb, fresh);
        HIP_TRY(hipGetLastError());
    }
    return DFDX_ROCM_OK;
}

size_t elem_bytes(int dtype) { return dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2; }
bool dims_ok(int64_t rows, int64_t cols) { return rows >= 0 && cols >= 0 && rows < (1ll << 31) && cols < (1ll << 31); }

}  // namespace
}  // namespace dfdx_rocm

using namespace dfdx_rocm;

extern "C" {

int dfdx_rocm_bias_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *bias,
                           void *out) {
    if (int e = bind(ctx)) return e;
    if (!dims_ok(rows, cols)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return DFDX_ROCM_OK;
    if (!x || !bias || !out) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    if (int e = settle(ctx, x)) return e;
    if (int e = settle(ctx, bias)) return e;
    if (int e = settle_output(ctx, out, (size_t)(rows * cols) * elem_bytes(dtype), false, nullptr)) return e;
    switch (dtype) {
    case DFDX_ROCM_F32: return bias_forward_t<float>(ctx, rows, cols, x, bias, out);
    case DFDX_ROCM_F16: return bias_forward_t<_Float16>(ctx, rows, cols, x, bias, out);
    case DFDX_ROCM_BF16: return bias_forward_t<__bf16>(ctx, rows, cols, x, bias, out);
    case DFDX_ROCM_F64: {
        const int64_t total = rows * cols;
        const unsigned grid = (unsigned)std::min<int64_t>((total + 255) / 256, (int64_t)ctx->compute_units * 8);
        bias_forward_f64_kernel<<<grid, 256, 0, ctx->stream>>>((const double *)x, (const double *)bias, (double *)out, total, cols);
        return (int)hipGetLastError();
    }
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

int dfdx_rocm_bias_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *grad_out,
                            void *grad_bias) {
    if (int e = bind(ctx)) return e;
    if (!dims_ok(rows, cols)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return DFDX_ROCM_OK;
    if (!grad_out || !grad_bias) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    bool fresh = false;  // a gradient whose zero fill is still deferred: stored without being read
    if (int e = settle(ctx, grad_out)) return e;
    if (int e = settle_output(ctx, grad_bias, (size_t)cols * elem_bytes(dtype), true, &fresh)) return e;
    switch (dtype) {
    case DFDX_ROCM_F32: return bias_backward_t<float>(ctx, rows, cols, grad_out, grad_bias, fresh);
    case DFDX_ROCM_F16: return bias_backward_t<_Float16>(ctx, rows, cols, grad_out, grad_bias, fresh);
    case DFDX_ROCM_BF16: return bias_backward_t<__bf16>(ctx, rows, cols, grad_out, grad_bias, fresh);
    case DFDX_ROCM_F64:
        bias_backward_f64_kernel<<<(unsigned)((cols + 255) / 256), 256, 0, ctx->stream>>>((const double *)grad_out, rows, cols, (double *)grad_bias, fresh);
        return (int)hipGetLastError();
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

}  // extern "C"
