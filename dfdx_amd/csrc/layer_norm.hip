// LayerNorm1D over the last (contiguous) axis of a (rows, cols) matrix and its backward:
//   xhat = (x - mean) / sqrt(var + eps),  var = mean((x - mean)^2),  out = gamma * xhat + beta.
// The reference composes it from mean / sub / square / mean / add / sqrt / div / mul / add tensor ops
// (dfdx-core/src/tensor_ops/normalize.rs:35-49, dfdx/src/nn/layers/layer_norm1d.rs:87-91); here one wave owns a row,
// evaluates the formula in f32 and rounds once.  HBM-bound: the forward reads x and writes out; the backward reads x
// and grad_out, reads and writes grad_x, and leaves per-slice column sums for grad_gamma / grad_beta that a second
// launch adds up in slice order.
#include "ctx_internal.h"
#include "elem.h"

#include <algorithm>

namespace dfdx_rocm {
namespace {

constexpr int WAVES = 4;      // rows in flight per workgroup (forward)
constexpr int WAVES_BWD = 8;  // backward: more rows per workgroup, so fewer slices of column sums to combine

__device__ __forceinline__ float wave_sum(float v) { return wave64_sum(v); }
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Lane l owns the N-element groups l, l + 64, ... of the row (CH of them; groups past the row end are skipped).
template <typename T, int N, int CH>
__global__ __launch_bounds__(WAVES * 64) void layer_norm_forward_kernel(const T *x, const T *gamma, const T *beta, T *out,
                                                                        int64_t rows, int cols, float eps) {
    const int lane = threadIdx.x % 64;
    const float inv_n = 1.0f / (float)cols;
    float gm[CH][N], bt[CH][N];
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int col = (c * 64 + lane) * N;
        if (col < cols) {
            load_elems<T, N>(gamma + col, gm[c]);
            load_elems<T, N>(beta + col, bt[c]);
        }
    }
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *src = x + row * cols;
        float v[CH][N];
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                load_elems<T, N>(src + col, v[c]);
#pragma unroll
                for (int i = 0; i < N; i++) s += v[c][i];
            }
        }
        const float mean = wave_sum(s) * inv_n;
        float q = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] -= mean;
                    q += v[c][i] * v[c][i];
                }
            }
        }
        const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_n + eps);
        T *dst = out + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) v[c][i] = v[c][i] * rstd * gm[c][i] + bt[c][i];
                store_elems<T, N>(dst + col, v[c]);
            }
        }
    }
}

// grad_x += rstd * (gh - mean(gh) - xhat * mean(gh * xhat)),  gh = grad_out * gamma;
// partial[slice][0][col] = sum over the slice's rows of grad_out * xhat, partial[slice][1][col] = of grad_out.
template <typename T, int N, int CH>
__global__ __launch_bounds__(WAVES_BWD * 64) void layer_norm_backward_kernel(const T *x, const T *gamma, const T *go, T *gx,
                                                                         float *partial, int64_t rows, int cols, float eps, bool fresh_x) {
    __shared__ float red[WAVES_BWD][2][64 * N];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const float inv_n = 1.0f / (float)cols;
    float gm[CH][N], dg[CH][N], db[CH][N];
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int col = (c * 64 + lane) * N;
        if (col < cols) load_elems<T, N>(gamma + col, gm[c]);
#pragma unroll
        for (int i = 0; i < N; i++) dg[c][i] = db[c][i] = 0.0f;
    }
    for (int64_t row = (int64_t)blockIdx.x * WAVES_BWD + wave; row < rows; row += (int64_t)gridDim.x * WAVES_BWD) {
        const T *src = x + row * cols, *gs = go + row * cols;
        float v[CH][N], g[CH][N];
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                load_elems<T, N>(src + col, v[c]);
                load_elems<T, N>(gs + col, g[c]);
#pragma unroll
                for (int i = 0; i < N; i++) s += v[c][i];
            }
        }
        const float mean = wave_sum(s) * inv_n;
        float q = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] -= mean;
                    q += v[c][i] * v[c][i];
                }
            }
        }
        const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_n + eps);
        float s1 = 0.0f, s2 = 0.0f;  // sum gh, sum gh * xhat
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] *= rstd;  // xhat
                    dg[c][i] += g[c][i] * v[c][i];
                    db[c][i] += g[c][i];
                    g[c][i] *= gm[c][i];  // gh
                    s1 += g[c][i];
                    s2 += g[c][i] * v[c][i];
                }
            }
        }
        const float m1 = wave_sum(s1) * inv_n, m2 = wave_sum(s2) * inv_n;
        T *dst = gx + row * cols;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * N;
            if (col < cols) {
                float old[N];
                if (fresh_x) {  // grad_x counts as zero and is not read
#pragma unroll
                    for (int i = 0; i < N; i++) old[i] = 0.0f;
                } else {
                    load_elems<T, N>(dst + col, old);
                }
#pragma unroll
                for (int i = 0; i < N; i++) old[i] += rstd * (g[c][i] - m1 - v[c][i] * m2);
                store_elems<T, N>(dst + col, old);
            }
        }
    }
    // column sums of the workgroup's rows: the waves through LDS, one chunk of 64 * N columns at a time
#pragma unroll
    for (int c = 0; c < CH; c++) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < N; i++) {
            red[wave][0][lane * N + i] = dg[c][i];
            red[wave][1][lane * N + i] = db[c][i];
        }
        __syncthreads();
        for (int t = threadIdx.x; t < 2 * 64 * N; t += WAVES_BWD * 64) {
            const int which = t / (64 * N), j = t % (64 * N), col = c * 64 * N + j;
            if (col < cols) {
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < WAVES_BWD; w++) sum += red[w][which][j];
                partial[((int64_t)blockIdx.x * 2 + which) * cols + col] = sum;
            }
        }
    }
}

// ---- long rows: 256 threads share a row ----------------------------------------------------------------------------
// Rows past what a wave keeps in registers (2048 16-bit / 1024 f32 elements: a model width of 4096 or 5120) went to the
// kernels that walk the row from memory once per pass, a wave per row -- 1 TB/s forward, 0.6-0.9 backward.  Here a workgroup
// walks rows blockIdx.x, + gridDim.x, ...; each thread keeps NV vectors of the row (and of gamma, beta and the column sums) in
// registers, the row's sums go wave -> LDS -> all threads in a fixed order.  The same formulas, one read, one write.
constexpr int LN_BLOCK = 256;
__device__ __forceinline__ float ln_block_sum(float v, float *slots) {
    v = wave_sum(v);
    __syncthreads();  // (the slots of the previous sum have been read)
    if (threadIdx.x % 64 == 0) slots[threadIdx.x / 64] = v;
    __syncthreads();
    return (slots[0] + slots[1]) + (slots[2] + slots[3]);
}
// two sums at once (one pair of barriers)
__device__ __forceinline__ void ln_block_sum2(float &a, float &b, float (*slots)[2]) {
    a = wave_sum(a);
    b = wave_sum(b);
    __syncthreads();
    if (threadIdx.x % 64 == 0) {
        slots[threadIdx.x / 64][0] = a;
        slots[threadIdx.x / 64][1] = b;
    }
    __syncthreads();
    a = (slots[0][0] + slots[1][0]) + (slots[2][0] + slots[3][0]);
    b = (slots[0][1] + slots[1][1]) + (slots[2][1] + slots[3][1]);
}
template <typename T, int NV>
__global__ __launch_bounds__(LN_BLOCK) void layer_norm_forward_block_kernel(const T *x, const T *gamma, const T *beta, T *out, int64_t rows, int cols,
                                                                            float eps) {
    constexpr int N = Elem<T>::VEC;
    __shared__ float slots[4];
    const float inv_n = 1.0f / (float)cols;
    float gm[NV][N], bt[NV][N];
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * LN_BLOCK + threadIdx.x) * N;
        if (col < cols) {
            load_elems<T, N>(gamma + col, gm[c]);
            load_elems<T, N>(beta + col, bt[c]);
        }
    }
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const T *src = x + row * cols;
        float v[NV][N];
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            const int col = (c * LN_BLOCK + threadIdx.x) * N;
            if (col < cols) {
                load_elems<T, N>(src + col, v[c]);
#pragma unroll
                for (int i = 0; i < N; i++) s += v[c][i];
            }
        }
        const float mean = ln_block_sum(s, slots) * inv_n;
        float q = 0.0f;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            if ((c * LN_BLOCK + threadIdx.x) * N < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] -= mean;
                    q += v[c][i] * v[c][i];
                }
            }
        }
        const float rstd = 1.0f / sqrtf(ln_block_sum(q, slots) * inv_n + eps);
        T *dst = out + row * cols;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            const int col = (c * LN_BLOCK + threadIdx.x) * N;
            if (col < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) v[c][i] = v[c][i] * rstd * gm[c][i] + bt[c][i];
                store_elems<T, N>(dst + col, v[c]);
            }
        }
    }
}
// partial[blockIdx.x][0 / 1][col]: the workgroup's column sums (every column belongs to one thread: no combining here)
template <typename T, int NV>
__global__ __launch_bounds__(LN_BLOCK) void layer_norm_backward_block_kernel(const T *x, const T *gamma, const T *go, T *gx, float *partial, int64_t rows,
                                                                             int cols, float eps, bool fresh_x) {
    constexpr int N = Elem<T>::VEC;
    __shared__ float slots[4];
    __shared__ float slots2[4][2];
    const float inv_n = 1.0f / (float)cols;
    float gm[NV][N], dg[NV][N], db[NV][N];
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * LN_BLOCK + threadIdx.x) * N;
        if (col < cols) load_elems<T, N>(gamma + col, gm[c]);
#pragma unroll
        for (int i = 0; i < N; i++) dg[c][i] = db[c][i] = 0.0f;
    }
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const T *src = x + row * cols, *gs = go + row * cols;
        float v[NV][N], g[NV][N];
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            const int col = (c * LN_BLOCK + threadIdx.x) * N;
            if (col < cols) {
                load_elems<T, N>(src + col, v[c]);
                load_elems<T, N>(gs + col, g[c]);
#pragma unroll
                for (int i = 0; i < N; i++) s += v[c][i];
            }
        }
        const float mean = ln_block_sum(s, slots) * inv_n;
        float q = 0.0f;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            if ((c * LN_BLOCK + threadIdx.x) * N < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] -= mean;
                    q += v[c][i] * v[c][i];
                }
            }
        }
        const float rstd = 1.0f / sqrtf(ln_block_sum(q, slots) * inv_n + eps);
        float s1 = 0.0f, s2 = 0.0f;  // sum gh, sum gh * xhat
#pragma unroll
        for (int c = 0; c < NV; c++) {
            if ((c * LN_BLOCK + threadIdx.x) * N < cols) {
#pragma unroll
                for (int i = 0; i < N; i++) {
                    v[c][i] *= rstd;  // xhat
                    dg[c][i] += g[c][i] * v[c][i];
                    db[c][i] += g[c][i];
                    g[c][i] *= gm[c][i];  // gh
                    s1 += g[c][i];
                    s2 += g[c][i] * v[c][i];
                }
            }
        }
        ln_block_sum2(s1, s2, slots2);
        const float m1 = s1 * inv_n, m2 = s2 * inv_n;
        T *dst = gx + row * cols;
#pragma unroll
        for (int c = 0; c < NV; c++) {
            const int col = (c * LN_BLOCK + threadIdx.x) * N;
            if (col < cols) {
                float old[N];
                if (fresh_x) {
#pragma unroll
                    for (int i = 0; i < N; i++) old[i] = 0.0f;
                } else {
                    load_elems<T, N>(dst + col, old);
                }
#pragma unroll
                for (int i = 0; i < N; i++) old[i] += rstd * (g[c][i] - m1 - v[c][i] * m2);
                store_elems<T, N>(dst + col, old);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NV; c++) {
        const int col = (c * LN_BLOCK + threadIdx.x) * N;
        if (col < cols) {
#pragma unroll
            for (int i = 0; i < N; i++) {
                partial[((int64_t)blockIdx.x * 2 + 0) * cols + col + i] = dg[c][i];
                partial[((int64_t)blockIdx.x * 2 + 1) * cols + col + i] = db[c][i];
            }
        }
    }
}

// Long or unaligned rows: the same formulas with the row walked from memory once per pass.
template <typename T>
__global__ __launch_bounds__(WAVES * 64) void layer_norm_forward_loop_kernel(const T *x, const T *gamma, const T *beta, T *out,
                                                                             int64_t rows, int cols, typename Acc<T>::type eps) {
    typedef typename Acc<T>::type A;  // f32, or f64 for f64 rows
    const int lane = threadIdx.x % 64;
    const A inv_n = A(1) / (A)cols;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + threadIdx.x / 64; row < rows; row += (int64_t)gridDim.x * WAVES) {
        const T *src = x + row * cols;
        A s = A(0);
        for (int c = lane; c < cols; c += 64) s += Elem<T>::load(src + c);
        const A mean = wave_sum(s) * inv_n;
        A q = A(0);
        for (int c = lane; c < cols; c += 64) {
            const A d = Elem<T>::load(src + c) - mean;
            q += d * d;
        }
        const A rstd = A(1) / sqrt(wave_sum(q) * inv_n + eps);
        T *dst = out + row * cols;
        for (int c = lane; c < cols; c += 64)
            Elem<T>::store(dst + c, (Elem<T>::load(src + c) - mean) * rstd * Elem<T>::load(gamma + c) + Elem<T>::load(beta + c));
    }
}

// One workgroup per slice of rows; the column sums go through atomics-free per-wave accumulation in memory order:
// wave w adds its rows into partial[slice * WAVES_BWD + w], so `slices` counts waves here.
template <typename T>
__global__ __launch_bounds__(WAVES_BWD * 64) void layer_norm_backward_loop_kernel(const T *x, const T *gamma, const T *go, T *gx,
                                                                              typename Acc<T>::type *partial, int64_t rows, int cols, typename Acc<T>::type eps, bool fresh_x) {
    typedef typename Acc<T>::type A;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const A inv_n = A(1) / (A)cols;
    A *pg = partial + ((int64_t)(blockIdx.x * WAVES_BWD + wave) * 2) * cols, *pb = pg + cols;
    for (int c = lane; c < cols; c += 64) pg[c] = pb[c] = A(0);
    for (int64_t row = (int64_t)blockIdx.x * WAVES_BWD + wave; row < rows; row += (int64_t)gridDim.x * WAVES_BWD) {
        const T *src = x + row * cols, *gs = go + row * cols;
        A s = A(0);
        for (int c = lane; c < cols; c += 64) s += Elem<T>::load(src + c);
        const A mean = wave_sum(s) * inv_n;
        A q = A(0);
        for (int c = lane; c < cols; c += 64) {
            const A d = Elem<T>::load(src + c) - mean;
            q += d * d;
        }
        const A rstd = A(1) / sqrt(wave_sum(q) * inv_n + eps);
        A s1 = A(0), s2 = 0.0f;
        for (int c = lane; c < cols; c += 64) {
            const A xh = (Elem<T>::load(src + c) - mean) * rstd, g = Elem<T>::load(gs + c), gh = g * Elem<T>::load(gamma + c);
            pg[c] += g * xh;  // column c of this wave's partial belongs to this lane alone
            pb[c] += g;
            s1 += gh;
            s2 += gh * xh;
        }
        const A m1 = wave_sum(s1) * inv_n, m2 = wave_sum(s2) * inv_n;
        T *dst = gx + row * cols;
        for (int c = lane; c < cols; c += 64) {
            const A xh = (Elem<T>::load(src + c) - mean) * rstd, gh = Elem<T>::load(gs + c) * Elem<T>::load(gamma + c);
            Elem<T>::store(dst + c, (fresh_x ? A(0) : Elem<T>::load(dst + c)) + rstd * (gh - m1 - xh * m2));
        }
    }
}

// grad_gamma[c] += sum_s partial[s][0][c], grad_beta[c] += sum_s partial[s][1][c].  A workgroup owns 64 columns; its
// 16 lane rows each add up a contiguous sixteenth of the slices (four loads in flight), then lane row 0 adds the 16
// sums in order: the result does not depend on timing.
constexpr int COMBINE_GROUPS = 16;
template <typename T>
__global__ __launch_bounds__(64 * COMBINE_GROUPS) void layer_norm_combine_kernel(const typename Acc<T>::type *partial, int slices, int cols, T *grad_gamma,
                                                                                 T *grad_beta, bool fresh_gamma, bool fresh_beta) {
    typedef typename Acc<T>::type A;
    __shared__ A red[COMBINE_GROUPS][2][64];
    const int lane = threadIdx.x % 64, grp = threadIdx.x / 64;
    const int c = blockIdx.x * 64 + lane;
    const int per = (slices + COMBINE_GROUPS - 1) / COMBINE_GROUPS;
    const int j0 = grp * per, j1 = min(slices, j0 + per);
    A sg = A(0), sb = 0.0f;
    if (c < cols) {
        int j = j0;
        for (; j + 4 <= j1; j += 4) {
            A a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                a[u] = partial[((int64_t)(j + u) * 2) * cols + c];
                b[u] = partial[((int64_t)(j + u) * 2 + 1) * cols + c];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                sg += a[u];
                sb += b[u];
            }
        }
        for (; j < j1; j++) {
            sg += partial[((int64_t)j * 2) * cols + c];
            sb += partial[((int64_t)j * 2 + 1) * cols + c];
        }
    }
    red[grp][0][lane] = sg;
    red[grp][1][lane] = sb;
    __syncthreads();
    if (grp == 0 && c < cols) {
        A tg = A(0), tb = 0.0f;
#pragma unroll
        for (int g = 0; g < COMBINE_GROUPS; g++) {
            tg += red[g][0][lane];
            tb += red[g][1][lane];
        }
        Elem<T>::store(grad_gamma + c, (fresh_gamma ? A(0) : Elem<T>::load(grad_gamma + c)) + tg);
        Elem<T>::store(grad_beta + c, (fresh_beta ? A(0) : Elem<T>::load(grad_beta + c)) + tb);
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T>
int forward_t(dfdx_rocm_ctx *ctx, int64_t rows, int64_t cols, const void *x, const void *gamma, const void *beta,
              typename Acc<T>::type eps, void *out) {
    constexpr int V = Elem<T>::VEC;
    constexpr bool F64 = sizeof(T) == 8;  // the plain kernel only
    const bool vec = !F64 && cols % V == 0 && aligned16(x) && aligned16(gamma) && aligned16(beta) && aligned16(out);
    const unsigned grid = (unsigned)std::min<int64_t>((rows + WAVES - 1) / WAVES, (int64_t)ctx->compute_units * 16);
    const dim3 block(WAVES * 64);
    hipStream_t s = ctx->stream;
#define DFDX_LN_FWD(CH)                                                                                                           \
    do {                                                                                                                          \
        layer_norm_forward_kernel<T, V, CH><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)beta, (T *)out, rows, \
                                                                   (int)cols, eps);                                               \
        return (int)hipGetLastError();                                                                                            \
    } while (0)
    if constexpr (!F64) {
        if (vec) {
            const int64_t groups = cols / V;
            if (groups <= 64) DFDX_LN_FWD(1);
            if (groups <= 128) DFDX_LN_FWD(2);
            if (groups <= 256) DFDX_LN_FWD(4);
            // long rows: 256 threads per row, as many workgroups as keep the chip busy (they loop over the rows)
            const unsigned bgrid = (unsigned)std::min<int64_t>(rows, (int64_t)ctx->compute_units * 4);
#define DFDX_LN_FWD_BLOCK(NV)                                                                                                     \
    do {                                                                                                                          \
        layer_norm_forward_block_kernel<T, NV><<<bgrid, LN_BLOCK, 0, s>>>((const T *)x, (const T *)gamma, (const T *)beta, (T *)out, rows, (int)cols, \
                                                                         eps);                                                    \
        return (int)hipGetLastError();                                                                                            \
    } while (0)
            if (groups <= 2 * LN_BLOCK) DFDX_LN_FWD_BLOCK(2);
            if (groups <= 4 * LN_BLOCK) DFDX_LN_FWD_BLOCK(4);
            if (groups <= 8 * LN_BLOCK) DFDX_LN_FWD_BLOCK(8);
#undef DFDX_LN_FWD_BLOCK
        } else {  // rows off the 16-byte grid (a width of 100 in a 16-bit type): element loads, the row still in registers
#define DFDX_LN_FWD1(CH)                                                                                                          \
    do {                                                                                                                          \
        layer_norm_forward_kernel<T, 1, CH><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)beta, (T *)out, rows, \
                                                                   (int)cols, eps);                                               \
        return (int)hipGetLastError();                                                                                            \
    } while (0)
            if (cols <= 64) DFDX_LN_FWD1(1);
            if (cols <= 256) DFDX_LN_FWD1(4);
            if (cols <= 1024) DFDX_LN_FWD1(16);
#undef DFDX_LN_FWD1
        }
    }
#undef DFDX_LN_FWD
    layer_norm_forward_loop_kernel<T><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)beta, (T *)out, rows, (int)cols, eps);
    return (int)hipGetLastError();
}

template <typename T>
int backward_t(dfdx_rocm_ctx *ctx, int64_t rows, int64_t cols, const void *x, const void *gamma, typename Acc<T>::type eps,
               const void *go, void *gx, void *ggamma, void *gbeta, const bool fresh[3]) {
    typedef typename Acc<T>::type A;
    constexpr int V = Elem<T>::VEC;
    constexpr bool F64 = sizeof(T) == 8;
    const bool vec = !F64 && cols % V == 0 && aligned16(x) && aligned16(gamma) && aligned16(go) && aligned16(gx);
    const int64_t groups = cols / V;
    const bool reg1 = !F64 && !vec && cols <= 1024;  // rows off the 16-byte grid: element loads, the row still in registers
    const bool reg = (vec && groups <= 256) || reg1;
    const bool by_block = vec && !reg && groups <= 8 * LN_BLOCK;  // long rows: 256 threads per row, a slice per workgroup
    // at least 2 rows per wave so that the column sums amortise; two workgroups (16 waves) per compute unit
    const unsigned grid = by_block ? (unsigned)std::max<int64_t>(1, std::min<int64_t>((rows + 3) / 4, (int64_t)ctx->compute_units * 2))
                                   : (unsigned)std::max<int64_t>(1, std::min<int64_t>((rows + 2 * WAVES_BWD - 1) / (2 * WAVES_BWD), (int64_t)ctx->compute_units * 2));
    const int slices = (int)grid * ((reg || by_block) ? 1 : WAVES_BWD);
    const dim3 block(WAVES_BWD * 64);
    hipStream_t s = ctx->stream;
    CtxLock lock(ctx->mu);  // two launches around the shared workspace
    if (int rc = ensure_workspace(ctx, (size_t)slices * 2 * cols * sizeof(A))) return rc;
    A *partial = (A *)ctx->workspace;
#define DFDX_LN_BWD(CH)                                                                                                         \
    layer_norm_backward_kernel<T, V, CH><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, \
                                                                rows, (int)cols, eps, fresh[0])
    bool launched = false;
    if constexpr (!F64) {
        if (reg1) {
#define DFDX_LN_BWD1(CH)                                                                                                        \
    layer_norm_backward_kernel<T, 1, CH><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, \
                                                                rows, (int)cols, eps, fresh[0])
            if (cols <= 64) DFDX_LN_BWD1(1);
            else if (cols <= 256) DFDX_LN_BWD1(4);
            else DFDX_LN_BWD1(16);
#undef DFDX_LN_BWD1
            launched = true;
        } else if (reg) {
            if (groups <= 64) DFDX_LN_BWD(1);
            else if (groups <= 128) DFDX_LN_BWD(2);
            else DFDX_LN_BWD(4);
            launched = true;
        } else if (by_block) {
            if (groups <= 2 * LN_BLOCK)
                layer_norm_backward_block_kernel<T, 2><<<grid, LN_BLOCK, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, rows, (int)cols, eps, fresh[0]);
            else if (groups <= 4 * LN_BLOCK)
                layer_norm_backward_block_kernel<T, 4><<<grid, LN_BLOCK, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, rows, (int)cols, eps, fresh[0]);
            else
                layer_norm_backward_block_kernel<T, 8><<<grid, LN_BLOCK, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, rows, (int)cols, eps, fresh[0]);
            launched = true;
        }
    }
    if (!launched) layer_norm_backward_loop_kernel<T><<<grid, block, 0, s>>>((const T *)x, (const T *)gamma, (const T *)go, (T *)gx, partial, rows, (int)cols, eps, fresh[0]);
#undef DFDX_LN_BWD
    HIP_TRY(hipGetLastError());
    layer_norm_combine_kernel<T><<<(unsigned)((cols + 63) / 64), 64 * COMBINE_GROUPS, 0, s>>>(partial, slices, (int)cols, (T *)ggamma, (T *)gbeta, fresh[1], fresh[2]);
    return (int)hipGetLastError();
}

bool dims_ok(int64_t rows, int64_t cols) { return rows >= 0 && cols >= 0 && rows < (1ll << 40) && cols < (1ll << 24); }

}  // namespace
}  // namespace dfdx_rocm

using namespace dfdx_rocm;

extern "C" {

int dfdx_rocm_layer_norm_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *gamma,
                                 const void *beta, double epsilon, void *out) {
    if (int e = bind(ctx)) return e;
    if (!dims_ok(rows, cols)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return DFDX_ROCM_OK;
    if (!x || !gamma || !beta || !out) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    if (int e = settle(ctx, x)) return e;
    if (int e = settle(ctx, gamma)) return e;
    if (int e = settle(ctx, beta)) return e;
    if (int e = settle_output(ctx, out, (size_t)(rows * cols) * (dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2), false, nullptr)) return e;
    switch (dtype) {
    case DFDX_ROCM_F64: return forward_t<double>(ctx, rows, cols, x, gamma, beta, epsilon, out);
    case DFDX_ROCM_F32: return forward_t<float>(ctx, rows, cols, x, gamma, beta, (float)epsilon, out);
    case DFDX_ROCM_F16: return forward_t<_Float16>(ctx, rows, cols, x, gamma, beta, (float)epsilon, out);
    case DFDX_ROCM_BF16: return forward_t<__bf16>(ctx, rows, cols, x, gamma, beta, (float)epsilon, out);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

int dfdx_rocm_layer_norm_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *gamma,
                                  double epsilon, void *grad_x, void *grad_gamma, void *grad_beta, const void *grad_out) {
    if (int e = bind(ctx)) return e;
    if (!dims_ok(rows, cols)) return DFDX_ROCM_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0) return DFDX_ROCM_OK;
    if (!x || !gamma || !grad_x || !grad_gamma || !grad_beta || !grad_out) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    const size_t es = dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2;
    bool fresh[3] = {false, false, false};  // gradients whose zero fill is still deferred: stored without being read
    if (int e = settle(ctx, x)) return e;
    if (int e = settle(ctx, gamma)) return e;
    if (int e = settle(ctx, grad_out)) return e;
    if (int e = settle_output(ctx, grad_x, (size_t)(rows * cols) * es, true, &fresh[0])) return e;
    if (int e = settle_output(ctx, grad_gamma, (size_t)cols * es, true, &fresh[1])) return e;
    if (int e = settle_output(ctx, grad_beta, (size_t)cols * es, true, &fresh[2])) return e;
    switch (dtype) {
    case DFDX_ROCM_F64: return backward_t<double>(ctx, rows, cols, x, gamma, epsilon, grad_out, grad_x, grad_gamma, grad_beta, fresh);
    case DFDX_ROCM_F32: return backward_t<float>(ctx, rows, cols, x, gamma, (float)epsilon, grad_out, grad_x, grad_gamma, grad_beta, fresh);
    case DFDX_ROCM_F16: return backward_t<_Float16>(ctx, rows, cols, x, gamma, (float)epsilon, grad_out, grad_x, grad_gamma, grad_beta, fresh);
    case DFDX_ROCM_BF16: return backward_t<__bf16>(ctx, rows, cols, x, gamma, (float)epsilon, grad_out, grad_x, grad_gamma, grad_beta, fresh);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

}  // extern "C"
