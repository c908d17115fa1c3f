// Softmax over the last (contiguous) axis of a (rows, cols) matrix and its backward, with an optional scale of
// the logits folded in (attention's `q.k^T * scalar` followed by softmax).  HBM-bound: the forward reads and
// writes the matrix once, the backward reads p and grad_out, and reads and writes grad_x.
//
// One wave owns a row.  Rows of up to 64 * VEC * MAX_CHUNKS elements stay in registers between the passes; longer
// rows are walked three times (max, sum, store) from memory.
#include "ctx_internal.h"
#include "elem.h"

#include <cfloat>

namespace dfdx_rocm {
namespace {

constexpr int WAVES = 4;  // rows per workgroup

__device__ __forceinline__ float wave_max(float v) { return wave64_max(v); }
__device__ __forceinline__ float wave_sum(float v) { return wave64_sum(v); }

// ---- rows held in registers -----------------------------------------------------------------------------------
// Lane l owns the N-element groups l, l + 64, ... of the row (CH of them; groups past the row end are skipped).
template <typename T, int N, int CH, bool STREAM>
__global__ __launch_bounds__(WAVES * 64) void softmax_forward_reg_kernel(const T *x, T *out, int64_t rows, int cols, float scale) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *src = x + row * cols;
        float v[CH][N];
        float m = -FLT_MAX;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                load_elems_as<T, N, STREAM>(src + col, v[c]);
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] *= scale;
                    m = fmaxf(m, v[c][i]);
                }
            }
        }
        m = wave_max(m);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] = expf(v[c][i] - m);
                    s += v[c][i];
                }
            }
        }
        s = wave_sum(s);
        const float inv = 1.0f / s;
        T *dst = out + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) v[c][i] *= inv;
                store_elems<T, N>(dst + col, v[c]);
            }
        }
    }
}

// grad_x += scale * p * (g - sum_j g_j p_j); `fresh`: grad_x counts as zero and is not read
template <typename T, int N, int CH, bool STREAM>
__global__ __launch_bounds__(WAVES * 64) void softmax_backward_reg_kernel(const T *p, const T *go, T *gx, int64_t rows, int cols,
                                                                          float scale, bool fresh) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *ps = p + row * cols, *gs = go + row * cols;
        float pv[CH][N], gv[CH][N];
        float dot = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                load_elems_as<T, N, STREAM>(ps + col, pv[c]);
                load_elems_as<T, N, STREAM>(gs + col, gv[c]);
#pragma unroll
                for (int i = 0; i < N; i++) dot += pv[c][i] * gv[c][i];
            }
        }
        dot = wave_sum(dot);
        T *dst = gx + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                float old[N];
                if (fresh) {
#pragma unroll
                    for (int i = 0; i < N; i++) old[i] = 0.0f;
                } else {
                    load_elems<T, N>(dst + col, old);
                }
#pragma unroll
                for (int i = 0; i < N; i++) old[i] += scale * (pv[c][i] * (gv[c][i] - dot));
                store_elems<T, N>(dst + col, old);
            }
        }
    }
}

// ---- short rows: four rows per wave, 16 lanes each -------------------------------------------------------------
// A row of up to 16 * N * CH elements (1024 16-bit values) is spread over the 16 lanes of one DPP row: lane j of the row
// owns the N-element groups j, j + 16, ...  Its maximum and its sums then need four DPP steps that ride on the max / add
// itself (two quad permutations, the half-row and the row mirror) instead of six cross-lane moves through the LDS
// crossbar, and a wave keeps four rows' loads in flight.
template <typename T, int N, int CH, bool STREAM>
__global__ __launch_bounds__(WAVES * 64) void softmax_forward_row16_kernel(const T *x, T *out, int64_t rows, int cols, float scale) {
    const int lane = threadIdx.x % 64, j = lane % 16, sub = lane / 16;
    for (int64_t row0 = ((int64_t)blockIdx.x * WAVES + threadIdx.x / 64) * 4; row0 < rows; row0 += (int64_t)gridDim.x * WAVES * 4) {
        const bool live = row0 + sub < rows;
        const int64_t row = live ? row0 + sub : rows - 1;  // lanes past the last row repeat it and store nothing
        const T *src = x + row * cols;
        float v[CH][N];
        float m = -FLT_MAX;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 16 + j) * N;
            if (col < cols) {
                load_elems_as<T, N, STREAM>(src + col, v[c]);
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] *= scale;
                    m = fmaxf(m, v[c][i]);
                }
            }
        }
        m = row16_max(m);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 16 + j) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] = expf(v[c][i] - m);
                    s += v[c][i];
                }
            }
        }
        s = row16_sum(s);
        const float inv = 1.0f / s;
        T *dst = out + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 16 + j) * N;
            if (live && col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) v[c][i] *= inv;
                store_elems<T, N>(dst + col, v[c]);
            }
        }
    }
}

template <typename T, int N, int CH, bool STREAM>
__global__ __launch_bounds__(WAVES * 64) void softmax_backward_row16_kernel(const T *p, const T *go, T *gx, int64_t rows, int cols,
                                                                            float scale, bool fresh) {
    const int lane = threadIdx.x % 64, j = lane % 16, sub = lane / 16;
    for (int64_t row0 = ((int64_t)blockIdx.x * WAVES + threadIdx.x / 64) * 4; row0 < rows; row0 += (int64_t)gridDim.x * WAVES * 4) {
        const bool live = row0 + sub < rows;
        const int64_t row = live ? row0 + sub : rows - 1;
        const T *ps = p + row * cols, *gs = go + row * cols;
        float pv[CH][N], gv[CH][N];
        float dot = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 16 + j) * N;
            if (col < cols) {
                load_elems_as<T, N, STREAM>(ps + col, pv[c]);
                load_elems_as<T, N, STREAM>(gs + col, gv[c]);
#pragma unroll
                for (int i = 0; i < N; i++) dot += pv[c][i] * gv[c][i];
            }
        }
        dot = row16_sum(dot);
        T *dst = gx + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 16 + j) * N;
            if (live && col < cols) {
                float old[N];
                if (fresh) {
#pragma unroll
                    for (int i = 0; i < N; i++) old[i] = 0.0f;
                } else {
                    load_elems<T, N>(dst + col, old);
                }
#pragma unroll
                for (int i = 0; i < N; i++) old[i] += scale * (pv[c][i] * (gv[c][i] - dot));
                store_elems<T, N>(dst + col, old);
            }
        }
    }
}

// ---- long rows: three passes over memory --------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVES * 64) void softmax_forward_loop_kernel(const T *x, T *out, int64_t rows, int cols, float scale) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *src = x + row * cols;
        float m = -FLT_MAX;
        for (int c = lane; c < cols; c += 64) m = fmaxf(m, Elem<T>::load(src + c) * scale);
        m = wave_max(m);
        float s = 0.0f;
        for (int c = lane; c < cols; c += 64) s += expf(Elem<T>::load(src + c) * scale - m);
        s = wave_sum(s);
        const float inv = 1.0f / s;
        T *dst = out + row * cols;
        for (int c = lane; c < cols; c += 64) Elem<T>::store(dst + c, expf(Elem<T>::load(src + c) * scale - m) * inv);
    }
}

template <typename T>
__global__ __launch_bounds__(WAVES * 64) void softmax_backward_loop_kernel(const T *p, const T *go, T *gx, int64_t rows, int cols,
                                                                           float scale, bool fresh) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *ps = p + row * cols, *gs = go + row * cols;
        float dot = 0.0f;
        for (int c = lane; c < cols; c += 64) dot += Elem<T>::load(ps + c) * Elem<T>::load(gs + c);
        dot = wave_sum(dot);
        T *dst = gx + row * cols;
        for (int c = lane; c < cols; c += 64)
            Elem<T>::store(dst + c, (fresh ? 0.0f : Elem<T>::load(dst + c)) + scale * (Elem<T>::load(ps + c) * (Elem<T>::load(gs + c) - dot)));
    }
}

// ---- long rows: a workgroup per row ------------------------------------------------------------------------------
// Rows past what a wave keeps in registers used to go to the three-pass kernels above, one WAVE per row: a 5120-wide row
// ran at 1 TB/s and the 64 rows of a 50257-wide logit matrix kept 64 waves of the chip busy (360 us for 6 MB).  Here 256
// threads share a row and each keeps NV vectors of it in registers between the passes (one read, one write); the row's
// maximum and sums go wave -> LDS -> all threads, in a fixed order.
constexpr int BLOCK = 256;
__device__ __forceinline__ float block_reduce(float v, float *slots, bool is_max) {
    v = is_max ? wave_max(v) : wave_sum(v);
    __syncthreads();  // (the slots of the previous reduction have been read)
    if (threadIdx.x % 64 == 0) slots[threadIdx.x / 64] = v;
    __syncthreads();
    return is_max ? fmaxf(fmaxf(slots[0], slots[1]), fmaxf(slots[2], slots[3])) : (slots[0] + slots[1]) + (slots[2] + slots[3]);
}
template <typename T, int NV, bool STREAM>
__global__ __launch_bounds__(BLOCK) void softmax_forward_block_kernel(const T *x, T *out, int cols, float scale) {
    constexpr int V = Elem<T>::VEC;
    __shared__ float slots[4];
    const T *src = x + (int64_t)blockIdx.x * cols;
    float v[NV][V];
    float m = -FLT_MAX;
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * BLOCK + threadIdx.x) * V;
        if (col < cols) {
            load_elems_as<T, V, STREAM>(src + col, v[c]);
#pragma unroll
            for (int i = 0; i < V; i++) {
                v[c][i] *= scale;
                m = fmaxf(m, v[c][i]);
            }
        }
    }
    m = block_reduce(m, slots, true);
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < NV; c++) {
        if ((c * BLOCK + threadIdx.x) * V < cols) {
#pragma unroll
            for (int i = 0; i < V; i++) {
                v[c][i] = expf(v[c][i] - m);
                sum += v[c][i];
            }
        }
    }
    sum = block_reduce(sum, slots, false);
    const float inv = 1.0f / sum;
    T *dst = out + (int64_t)blockIdx.x * cols;
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * BLOCK + threadIdx.x) * V;
        if (col < cols) {
#pragma unroll
            for (int i = 0; i < V; i++) v[c][i] *= inv;
            store_elems<T, V>(dst + col, v[c]);
        }
    }
}
template <typename T, int NV, bool STREAM>
__global__ __launch_bounds__(BLOCK) void softmax_backward_block_kernel(const T *p, const T *go, T *gx, int cols, float scale, bool fresh) {
    constexpr int V = Elem<T>::VEC;
    __shared__ float slots[4];
    const T *ps = p + (int64_t)blockIdx.x * cols, *gs = go + (int64_t)blockIdx.x * cols;
    float pv[NV][V], gv[NV][V];
    float dot = 0.0f;
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * BLOCK + threadIdx.x) * V;
        if (col < cols) {
            load_elems_as<T, V, STREAM>(ps + col, pv[c]);
            load_elems_as<T, V, STREAM>(gs + col, gv[c]);
#pragma unroll
            for (int i = 0; i < V; i++) dot += pv[c][i] * gv[c][i];
        }
    }
    dot = block_reduce(dot, slots, false);
    T *dst = gx + (int64_t)blockIdx.x * cols;
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * BLOCK + threadIdx.x) * V;
        if (col < cols) {
            float old[V];
            if (!fresh) load_elems<T, V>(dst + col, old);
#pragma unroll
            for (int i = 0; i < V; i++) gv[c][i] = (fresh ? 0.0f : old[i]) + scale * (pv[c][i] * (gv[c][i] - dot));
            store_elems<T, V>(dst + col, gv[c]);
        }
    }
}
// Rows that fit no register form (unaligned, or longer still): a workgroup of 1024 threads per row, three passes over the
// row (the second and third find it in the cache), element loads.
template <typename T>
__global__ __launch_bounds__(1024) void softmax_forward_block_loop_kernel(const T *x, T *out, int cols, float scale) {
    __shared__ float slots[16];
    const T *src = x + (int64_t)blockIdx.x * cols;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    auto reduce = [&](float v, bool is_max) {
        v = is_max ? wave_max(v) : wave_sum(v);
        __syncthreads();
        if (lane == 0) slots[wave] = v;
        __syncthreads();
        float r = slots[0];
        for (int w = 1; w < 16; w++) r = is_max ? fmaxf(r, slots[w]) : r + slots[w];
        return r;
    };
    float m = -FLT_MAX;
    for (int c = threadIdx.x; c < cols; c += 1024) m = fmaxf(m, Elem<T>::load(src + c) * scale);
    m = reduce(m, true);
    float sum = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 1024) sum += expf(Elem<T>::load(src + c) * scale - m);
    sum = reduce(sum, false);
    const float inv = 1.0f / sum;
    T *dst = out + (int64_t)blockIdx.x * cols;
    for (int c = threadIdx.x; c < cols; c += 1024) Elem<T>::store(dst + c, expf(Elem<T>::load(src + c) * scale - m) * inv);
}
template <typename T>
__global__ __launch_bounds__(1024) void softmax_backward_block_loop_kernel(const T *p, const T *go, T *gx, int cols, float scale, bool fresh) {
    __shared__ float slots[16];
    const T *ps = p + (int64_t)blockIdx.x * cols, *gs = go + (int64_t)blockIdx.x * cols;
    float dot = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 1024) dot += Elem<T>::load(ps + c) * Elem<T>::load(gs + c);
    dot = wave_sum(dot);
    if (threadIdx.x % 64 == 0) slots[threadIdx.x / 64] = dot;
    __syncthreads();
    dot = slots[0];
    for (int w = 1; w < 16; w++) dot += slots[w];
    T *dst = gx + (int64_t)blockIdx.x * cols;
    for (int c = threadIdx.x; c < cols; c += 1024)
        Elem<T>::store(dst + c, (fresh ? 0.0f : Elem<T>::load(dst + c)) + scale * (Elem<T>::load(ps + c) * (Elem<T>::load(gs + c) - dot)));
}

// ---- f64: one wave per row, three passes over memory, f64 arithmetic ------------------------------------------
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ double wave_max_f64(double v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmax(v, __shfl_xor(v, o, 64));
    return v;
}
__global__ __launch_bounds__(WAVES * 64) void softmax_forward_f64_kernel(const double *x, double *out, int64_t rows, int cols, double scale) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const double *src = x + row * cols;
        double m = -DBL_MAX;
        for (int c = lane; c < cols; c += 64) m = fmax(m, src[c] * scale);
        m = wave_max_f64(m);
        double s = 0.0;
        for (int c = lane; c < cols; c += 64) s += exp(src[c] * scale - m);
        s = wave_sum_f64(s);
        double *dst = out + row * cols;
        for (int c = lane; c < cols; c += 64) dst[c] = exp(src[c] * scale - m) / s;
    }
}
__global__ __launch_bounds__(WAVES * 64) void softmax_backward_f64_kernel(const double *p, const double *go, double *gx, int64_t rows,
                                                                          int cols, double scale, bool fresh) {
    const int lane = threadIdx.x % 64;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const double *ps = p + row * cols, *gs = go + row * cols;
        double dot = 0.0;
        for (int c = lane; c < cols; c += 64) dot += ps[c] * gs[c];
        dot = wave_sum_f64(dot);
        double *dst = gx + row * cols;
        for (int c = lane; c < cols; c += 64) dst[c] = (fresh ? 0.0 : dst[c]) + scale * (ps[c] * (gs[c] - dot));
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T, bool FWD>
int launch_t(dfdx_rocm_ctx *ctx, int64_t rows, int64_t cols, const void *a, const void *b, void *c, float scale, bool fresh) {
    // forward: a = x, c = out;  backward: a = p, b = grad_out, c = grad_x
    constexpr int V = Elem<T>::VEC;
    const bool vec = cols % V == 0 && aligned16(a) && aligned16(c) && (FWD || aligned16(b));
    const unsigned grid = (unsigned)std::min<int64_t>((rows + WAVES - 1) / WAVES, (int64_t)ctx->compute_units * 16);
    const dim3 block(WAVES * 64);
    hipStream_t s = ctx->stream;
    const int n = (int)cols;
    // read-only input of the launch: x (forward), the probabilities and grad_out (backward)
    const bool stream = vec && (size_t)rows * (size_t)cols * sizeof(T) * (FWD ? 1 : 2) >= kStreamInputBytes;
#define DFDX_SOFTMAX_REG_AS(N, CH, STREAM)                                                                             \
    do {                                                                                                               \
        if constexpr (FWD) softmax_forward_reg_kernel<T, N, CH, STREAM><<<grid, block, 0, s>>>((const T *)a, (T *)c, rows, n, scale); \
        else softmax_backward_reg_kernel<T, N, CH, STREAM><<<grid, block, 0, s>>>((const T *)a, (const T *)b, (T *)c, rows, n, scale, fresh); \
        return (int)hipGetLastError();                                                                                 \
    } while (0)
#define DFDX_SOFTMAX_REG(N, CH)                                                                                        \
    do {                                                                                                               \
        if (stream) DFDX_SOFTMAX_REG_AS(N, CH, true);                                                                  \
        else DFDX_SOFTMAX_REG_AS(N, CH, false);                                                                        \
    } while (0)
#define DFDX_SOFTMAX_ROW16_AS(N, CH, STREAM)                                                                           \
    do {                                                                                                               \
        const unsigned g16 = (unsigned)std::min<int64_t>((rows + WAVES * 4 - 1) / (WAVES * 4), (int64_t)ctx->compute_units * 16); \
        if constexpr (FWD) softmax_forward_row16_kernel<T, N, CH, STREAM><<<g16, block, 0, s>>>((const T *)a, (T *)c, rows, n, scale); \
        else softmax_backward_row16_kernel<T, N, CH, STREAM><<<g16, block, 0, s>>>((const T *)a, (const T *)b, (T *)c, rows, n, scale, fresh); \
        return (int)hipGetLastError();                                                                                 \
    } while (0)
#define DFDX_SOFTMAX_ROW16(N, CH)                                                                                      \
    do {                                                                                                               \
        if (stream) DFDX_SOFTMAX_ROW16_AS(N, CH, true);                                                                \
        else DFDX_SOFTMAX_ROW16_AS(N, CH, false);                                                                      \
    } while (0)
    if (vec) {
        const int64_t groups = cols / V;
        if (groups <= 16) DFDX_SOFTMAX_ROW16(V, 1);
        if (groups <= 32) DFDX_SOFTMAX_ROW16(V, 2);
        if (FWD && groups <= 64) DFDX_SOFTMAX_ROW16(V, 4);  // the backward holds two rows of values per lane: no gain at 4 groups
        if (groups <= 64) DFDX_SOFTMAX_REG(V, 1);
        if (groups <= 128) DFDX_SOFTMAX_REG(V, 2);
        if (groups <= 256) DFDX_SOFTMAX_REG(V, 4);
        if (groups <= 512) DFDX_SOFTMAX_REG(V, 8);
    } else {
        if (cols <= 64) DFDX_SOFTMAX_REG(1, 1);
        if (cols <= 256) DFDX_SOFTMAX_REG(1, 4);
        if (cols <= 1024) DFDX_SOFTMAX_REG(1, 16);
    }
#undef DFDX_SOFTMAX_REG
#undef DFDX_SOFTMAX_ROW16
#undef DFDX_SOFTMAX_REG_AS
#undef DFDX_SOFTMAX_ROW16_AS
    // long rows: a workgroup per row (grid.x = rows)
    if (rows < (1ll << 31)) {
#define DFDX_SOFTMAX_BLOCK_AS(NV, STREAM)                                                                              \
    do {                                                                                                               \
        if constexpr (FWD) softmax_forward_block_kernel<T, NV, STREAM><<<(unsigned)rows, BLOCK, 0, s>>>((const T *)a, (T *)c, n, scale); \
        else softmax_backward_block_kernel<T, NV, STREAM><<<(unsigned)rows, BLOCK, 0, s>>>((const T *)a, (const T *)b, (T *)c, n, scale, fresh); \
        return (int)hipGetLastError();                                                                                 \
    } while (0)
#define DFDX_SOFTMAX_BLOCK(NV)                                                                                         \
    do {                                                                                                               \
        if (stream) DFDX_SOFTMAX_BLOCK_AS(NV, true);                                                                   \
        else DFDX_SOFTMAX_BLOCK_AS(NV, false);                                                                         \
    } while (0)
        if (vec) {
            const int64_t per_thread = (cols / V + BLOCK - 1) / BLOCK;  // vectors of a row per thread
            if (per_thread <= 4) DFDX_SOFTMAX_BLOCK(4);
            if (per_thread <= 8) DFDX_SOFTMAX_BLOCK(8);
            if (FWD && per_thread <= 16) DFDX_SOFTMAX_BLOCK(16);  // (the backward holds two rows of values)
        }
#undef DFDX_SOFTMAX_BLOCK
#undef DFDX_SOFTMAX_BLOCK_AS
        if constexpr (FWD) softmax_forward_block_loop_kernel<T><<<(unsigned)rows, 1024, 0, s>>>((const T *)a, (T *)c, n, scale);
        else softmax_backward_block_loop_kernel<T><<<(unsigned)rows, 1024, 0, s>>>((const T *)a, (const T *)b, (T *)c, n, scale, fresh);
        return (int)hipGetLastError();
    }
    if constexpr (FWD) softmax_forward_loop_kernel<T><<<grid, block, 0, s>>>((const T *)a, (T *)c, rows, n, scale);
    else softmax_backward_loop_kernel<T><<<grid, block, 0, s>>>((const T *)a, (const T *)b, (T *)c, rows, n, scale, fresh);
    return (int)hipGetLastError();
}

template <bool FWD>
int dispatch(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *a, const void *b, void *c, float scale) {
    if (int e = bind(ctx)) return e;
    if (rows < 0 || cols < 0 || cols >= (1ll << 31)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return DFDX_ROCM_OK;
    if (!a || !c || (!FWD && !b)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    bool fresh = false;  // a gradient whose zero fill is still deferred: stored without being read
    if (int e = settle(ctx, a)) return e;
    if (int e = settle(ctx, b)) return e;
    if (int e = settle_output(ctx, c, (size_t)(rows * cols) * (dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2), !FWD, &fresh)) return e;
    switch (dtype) {
    case DFDX_ROCM_F64: {
        const unsigned grid = (unsigned)std::min<int64_t>((rows + WAVES - 1) / WAVES, (int64_t)ctx->compute_units * 16);
        if constexpr (FWD) softmax_forward_f64_kernel<<<grid, WAVES * 64, 0, ctx->stream>>>((const double *)a, (double *)c, rows, (int)cols, (double)scale);
        else softmax_backward_f64_kernel<<<grid, WAVES * 64, 0, ctx->stream>>>((const double *)a, (const double *)b, (double *)c, rows, (int)cols, (double)scale, fresh);
        return (int)hipGetLastError();
    }
    case DFDX_ROCM_F32: return launch_t<float, FWD>(ctx, rows, cols, a, b, c, scale, fresh);
    case DFDX_ROCM_F16: return launch_t<_Float16, FWD>(ctx, rows, cols, a, b, c, scale, fresh);
    case DFDX_ROCM_BF16: return launch_t<__bf16, FWD>(ctx, rows, cols, a, b, c, scale, fresh);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

}  // namespace
}  // namespace dfdx_rocm

extern "C" {

int dfdx_rocm_softmax_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, float scale,
                              void *out) {
    return dfdx_rocm::dispatch<true>(ctx, dtype, rows, cols, x, nullptr, out, scale);
}

int dfdx_rocm_softmax_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *out, float scale,
                               void *grad_x, const void *grad_out) {
    return dfdx_rocm::dispatch<false>(ctx, dtype, rows, cols, out, grad_out, grad_x, scale);
}

}  // extern "C"
