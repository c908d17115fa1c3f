// A few vectors against one large matrix: (2..8, K).(K, N) and (M, K).(K, 2..8) -- a Linear layer on a batch of a
// handful of rows, the gradients of a layer with a handful of outputs.  (Sixteen vectors were tried and dropped: 128 sums per
// thread, and only the f32 weight gradient of a 10-output layer gained, 20 against 35 - 41 us.)  Like the vector products of gemv.hip these are
// bound by streaming the matrix once from HBM; a matrix-core tile would be 7/8 empty and, worse, leave most of the chip
// without a workgroup unless the contraction is split and combined by a second launch (16 x 4096 x 4096 f16: 15.8 us on
// the tiled kernels against 6 us for the bytes).  Same two forms as gemv.hip over
//     out[r, j] = sum_k vec[r, k] * mat[k, j],   r < R <= 8:
//   "cols"  the matrix is contiguous in j: a thread owns VEC adjacent outputs of every r, the R vector slices sit in LDS
//           (f32: as f32), the 4 waves of a workgroup take interleaved k, workgroups along grid.y take k slices;
//   "dots"  the matrix is contiguous in k (a Linear weight viewed transposed): a wave owns 4 outputs j of every r, its
//           lanes stride over k, each 16-byte piece of a vector is loaded once for the 4 matrix rows.
// The 16-bit types multiply pairs of k-adjacent values with v_dot2c_f32_f16 / _bf16 (f32 sums, operands stay packed).
// Partial sums of k slices go to an f32 workspace [slice][r][j] and are combined in slice order (deterministic).
#include "elem.h"
#include "gemm_internal.h"
#include <algorithm>
#include <type_traits>

namespace dfdx_rocm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct MultiParams {
    const void *vec, *mat, *bias;
    void *out;
    int64_t vec_k_stride, vec_r_stride, mat_k_stride, mat_j_stride, out_j_stride, out_r_stride, bias_j_stride, bias_r_stride;
    int k, j, r;
    int kslices, kchunk;
    int accumulate, has_bias;
    int stream;  // the matrix is read with non-temporal loads: 256 MiB or more, as in the single-vector kernel (gemv.hip)
    float *ws;
};
template <bool STREAM> __device__ __forceinline__ u32x4 ldm(const void *p) {
    if constexpr (STREAM) return __builtin_nontemporal_load((const u32x4 *)p);
    else return *(const u32x4 *)p;
}

// k values of a slice in the cols form: R x kchunk_of(R) values in LDS (32 KiB of f32 at most)
constexpr int kchunk_of(int r) { return r > 8 ? 512 : 1024; }
// matrix rows a wave of the dots form takes: 4 * R or 2 * R sums per lane
constexpr int rows_of(int r) { return r > 8 ? 2 : 4; }

template <typename T, int N> __device__ __forceinline__ void unpack16(const T *p, float (&v)[N]) {
    const u32x4 raw = *(const u32x4 *)p;
    T tmp[N];
    __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = Elem<T>::load(&tmp[i]);
}

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// acc + the products of two values that sit side by side along k in both operands (one dword each).  The 16-bit types
// take v_dot2c_f32_*: two multiply-adds into an f32 sum per lane and instruction and no widening of the operands, which is
// what keeps eight vectors against an f16 matrix bound by HBM and not by the vector ALUs.
template <typename T> __device__ __forceinline__ float dot_pair(uint32_t x, uint32_t v, float acc);
template <> __device__ __forceinline__ float dot_pair<_Float16>(uint32_t x, uint32_t v, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, x), __builtin_bit_cast(f16x2, v), acc, false);
}
template <> __device__ __forceinline__ float dot_pair<__bf16>(uint32_t x, uint32_t v, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, v), acc, false);
}
// acc + the dot product of 16 bytes of k-adjacent values of both operands
template <typename T> __device__ __forceinline__ float dot16(u32x4 x, u32x4 v, float acc) {
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int i = 0; i < 4; i++) acc += __uint_as_float(x[i]) * __uint_as_float(v[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) acc = dot_pair<T>(x[i], v[i], acc);
    }
    return acc;
}

template <typename T> __device__ __forceinline__ void finish(const MultiParams &p, int r, int j, float v) {
    T *dst = (T *)p.out + (int64_t)j * p.out_j_stride + (int64_t)r * p.out_r_stride;
    if (p.has_bias) v += Elem<T>::load((const T *)p.bias + (int64_t)j * p.bias_j_stride + (int64_t)r * p.bias_r_stride);
    if (p.accumulate) v += Elem<T>::load(dst);
    Elem<T>::store(dst, v);
}

// The cols form.  f32: a wave takes every fourth k and multiplies value by value.  16-bit types: a wave takes every fourth
// PAIR of k (2 q, 2 q + 1), the vector slices sit in LDS in their own type so that one dword holds a vector's pair, and the
// two matrix rows of a pair are interleaved column by column into dwords for dot_pair.
template <typename T, int R, bool STREAM> __global__ __launch_bounds__(256) void gemv_multi_cols_kernel(const MultiParams p) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr bool PAIRS = sizeof(T) == 2;
    typedef typename std::conditional<PAIRS, T, float>::type S;  // what the vector slices are kept as
    constexpr int KCH = kchunk_of(R);
    __shared__ __align__(16) S vsh[R][KCH];
    __shared__ float red[4][R < 4 ? R : 4][64 * VEC];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int j0 = (blockIdx.x * 64 + lane) * VEC;
    const int k0 = blockIdx.y * p.kchunk;
    const int kn = min(p.kchunk, p.k - k0);
    const int kn2 = (kn + 1) & ~1;  // PAIRS: an odd slice gets a zero partner for its last value
    const bool r_first = p.vec_r_stride == 1 && p.vec_k_stride != 1;  // neighbouring threads on neighbouring addresses
    for (int i = tid; i < R * kn2; i += 256) {
        const int r = r_first ? i % R : i / kn2, kk = r_first ? i / R : i % kn2;
        const bool in = r < p.r && kk < kn;
        const T v = *((const T *)p.vec + (int64_t)(k0 + min(kk, kn - 1)) * p.vec_k_stride + (int64_t)(in ? r : 0) * p.vec_r_stride);
        if constexpr (PAIRS) {
            const uint16_t bits = in ? __builtin_bit_cast(uint16_t, v) : (uint16_t)0;
            vsh[r][kk] = __builtin_bit_cast(T, bits);
        } else {  // a wave's k values (every fourth) side by side: four of them are one 16-byte LDS read
            vsh[r][(kk & 3) * (KCH / 4) + (kk >> 2)] = in ? Elem<T>::load(&v) : 0.0f;
        }
    }
    __syncthreads();
    float acc[R][VEC];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[r][e] = 0.f;
    if (j0 < p.j) {  // j % VEC == 0: the whole piece is in range
        const T *col = (const T *)p.mat + (int64_t)k0 * p.mat_k_stride + j0;
        if constexpr (PAIRS) {
            for (int kk = 2 * wave; kk < kn; kk += 16) {  // two pairs = 4 loads in flight
                u32x4 raw[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int row = kk + 8 * (u / 2) + (u & 1);
                    raw[u] = ldm<STREAM>(col + (int64_t)min(row, kn - 1) * p.mat_k_stride);  // (a row past the end meets a zero)
                }
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int kp = kk + 8 * h;
                    if (kp >= kn) break;   // the same in every lane
                    uint32_t x[VEC];       // column e of rows kp (low half) and kp + 1 (high half)
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        const uint32_t lo = raw[2 * h][d], hi = raw[2 * h + 1][d];
                        x[2 * d] = (lo & 0xffffu) | (hi << 16);
                        x[2 * d + 1] = (lo >> 16) | (hi & 0xffff0000u);
                    }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const uint32_t v = *(const uint32_t *)&vsh[r][kp];
#pragma unroll
                        for (int e = 0; e < VEC; e++) acc[r][e] = dot_pair<T>(x[e], v, acc[r][e]);
                    }
                }
            }
        } else {
            int kk = wave;
            for (; kk + 12 < kn; kk += 16) {  // 4 loads in flight
                u32x4 raw[4];
#pragma unroll
                for (int u = 0; u < 4; u++) raw[u] = ldm<STREAM>(col + (int64_t)(kk + 4 * u) * p.mat_k_stride);
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const f32x4 v = *(const f32x4 *)&vsh[r][wave * (KCH / 4) + (kk >> 2)];  // k = kk, kk + 4, kk + 8, kk + 12
#pragma unroll
                    for (int u = 0; u < 4; u++)
#pragma unroll
                        for (int e = 0; e < VEC; e++) acc[r][e] += v[u] * __uint_as_float(raw[u][e]);
                }
            }
            for (; kk < kn; kk += 4) {
                const u32x4 raw = ldm<STREAM>(col + (int64_t)kk * p.mat_k_stride);
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const float v = vsh[r][wave * (KCH / 4) + (kk >> 2)];
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[r][e] += v * __uint_as_float(raw[e]);
                }
            }
        }
    }
    // the four waves' sums meet in LDS, up to four vectors at a time (two barriers per group, not per vector)
    constexpr int G = R < 4 ? R : 4;
#pragma unroll
    for (int r0 = 0; r0 < R; r0 += G) {
        if (r0 < p.r) {  // the same in every thread
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int e = 0; e < VEC; e++) red[wave][g][lane * VEC + e] = acc[r0 + g][e];
            __syncthreads();
            for (int o = tid; o < G * 64 * VEC; o += 256) {
                const int g = o / (64 * VEC), c = o % (64 * VEC);
                const int j = blockIdx.x * 64 * VEC + c, r = r0 + g;
                if (j >= p.j || r >= p.r) continue;
                const float v = ((red[0][g][c] + red[1][g][c]) + red[2][g][c]) + red[3][g][c];
                if (p.kslices > 1) p.ws[((int64_t)blockIdx.y * p.r + r) * p.j + j] = v;
                else finish<T>(p, r, j, v);
            }
            __syncthreads();
        }
    }
}

// One step of the all-at-once wave reduction below: N values per lane become N / 2.
template <int NV, int N> __device__ __forceinline__ void halve(float (&vals)[NV], int lane, int &mine) {
    if constexpr (N > 1) {
        constexpr int OFF = 32 / (NV / N);
        const bool upper = lane & OFF;
#pragma unroll
        for (int i = 0; i < N / 2; i++) {
            const float keep = upper ? vals[i + N / 2] : vals[i];
            const float send = upper ? vals[i] : vals[i + N / 2];
            vals[i] = keep + __shfl_xor(send, OFF, 64);
        }
        mine += upper ? N / 2 : 0;
        halve<NV, N / 2>(vals, lane, mine);
    }
}

template <typename T, int R, bool STREAM> __global__ __launch_bounds__(256) void gemv_multi_dots_kernel(const MultiParams p) {
    constexpr int VEC = Elem<T>::VEC, J = rows_of(R);
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int j0 = (blockIdx.x * 4 + wave) * J;
    if (j0 >= p.j) return;
    const int k0 = blockIdx.y * p.kchunk;
    const int kn = min(p.kchunk, p.k - k0);  // a multiple of VEC
    const T *rows[J];
#pragma unroll
    for (int jj = 0; jj < J; jj++) rows[jj] = (const T *)p.mat + (int64_t)min(j0 + jj, p.j - 1) * p.mat_j_stride + k0;
    const T *vecs[R];
#pragma unroll
    for (int r = 0; r < R; r++) vecs[r] = (const T *)p.vec + (int64_t)(r < p.r ? r : 0) * p.vec_r_stride + k0;  // unit stride in k
    float acc[J][R];
#pragma unroll
    for (int jj = 0; jj < J; jj++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[jj][r] = 0.f;
    for (int kk = lane * VEC; kk < kn; kk += 64 * VEC) {
        u32x4 x[J];
#pragma unroll
        for (int jj = 0; jj < J; jj++) x[jj] = ldm<STREAM>(rows[jj] + kk);
#pragma unroll
        for (int r = 0; r < R; r++) {
            const u32x4 v = *(const u32x4 *)(vecs[r] + kk);
#pragma unroll
            for (int jj = 0; jj < J; jj++) acc[jj][r] = dot16<T>(x[jj], v, acc[jj][r]);
        }
    }
    // The J * R sums over the 64 lanes, all at once: in every step a lane hands one half of the values it still holds to
    // the lane `off` away and adds what it receives to the half it keeps, so that log2(J * R) steps leave every lane with
    // ONE value summed over as many lanes, and the remaining steps finish that one -- J * R exchanges instead of
    // 6 * J * R, and J * R lanes that store side by side instead of lane 0 storing them one after the other.
    constexpr int NV = J * R;
    float vals[NV];
#pragma unroll
    for (int jj = 0; jj < J; jj++)
#pragma unroll
        for (int r = 0; r < R; r++) vals[jj * R + r] = acc[jj][r];
    int mine = 0;  // which value this lane ends up with
    halve<NV, NV>(vals, lane, mine);
    constexpr int REST = 32 / NV;  // the lane distances not used up yet: REST, REST / 2, ... 1
    float total = vals[0];
    if constexpr (REST >= 4) total += __shfl_xor(total, 4, 64);
    if constexpr (REST >= 2) total += __shfl_xor(total, 2, 64);
    total += __shfl_xor(total, 1, 64);
    const int jj = mine / R, r = mine % R;
    if ((lane & (2 * REST - 1)) == 0 && j0 + jj < p.j && r < p.r) {  // one lane of each group that shares a value
        if (p.kslices > 1) p.ws[((int64_t)blockIdx.y * p.r + r) * p.j + j0 + jj] = total;
        else finish<T>(p, r, j0 + jj, total);
    }
}

// Eight lanes per output: lane `part` of an output adds the slices part, part + 8, ... (their loads in flight together),
// then the eight partial sums meet in a fixed tree of three exchanges -- one round trip to the workspace instead of
// kslices / 8 of them behind one another (64 slices of a 4 x 4096 x 4096 product: 14 -> 9 us for the whole product).
template <typename T> __global__ __launch_bounds__(256) void gemv_multi_combine_kernel(const MultiParams p) {
    const int o = blockIdx.x * 32 + threadIdx.x / 8, part = threadIdx.x % 8;
    const int64_t outs = (int64_t)p.r * p.j;
    const bool in = o < outs;
    const float *src = p.ws + (in ? o : 0);
    float v = 0.0f;
    for (int s = part; s < p.kslices; s += 64) {  // eight loads in flight, added in slice order
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = (s + 8 * u < p.kslices) ? src[(int64_t)(s + 8 * u) * outs] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) v += t[u];
    }
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    if (in && part == 0) finish<T>(p, o / p.j, o % p.j, v);
}

// Eight outputs per workgroup, thirty-two threads each (eight lanes in each of the four waves): thread `part` of an
// output adds the slices part, part + 32, ... (their loads in flight together), the eight partial sums of a wave meet in
// a fixed tree of three exchanges and the four waves' in LDS, in wave order -- one or two round trips to the workspace
// for 512 slices and more (a narrow matrix with a long k: few outputs, long chains of partial sums; 8 x 65536 x 256 with its
// 512 slices 22.6 -> 19.8 us).  Below, the form above is ahead (256 slices of 8 x 16384 x 1024 f16: 16.7 against 19.1 us): this
// one starts four times the workgroups.
template <typename T> __global__ __launch_bounds__(256) void gemv_multi_combine_deep_kernel(const MultiParams p) {
    __shared__ float sums[4][8];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int o = blockIdx.x * 8 + lane / 8, part = wave * 8 + lane % 8;
    const int64_t outs = (int64_t)p.r * p.j;
    const bool in = o < outs;
    const float *src = p.ws + (in ? o : 0);
    float v = 0.0f;
    for (int s = part; s < p.kslices; s += 256) {  // eight loads in flight, added in slice order
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = (s + 32 * u < p.kslices) ? src[(int64_t)(s + 32 * u) * outs] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) v += t[u];
    }
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    if (lane % 8 == 0) sums[wave][lane / 8] = v;
    __syncthreads();
    if (threadIdx.x < 8 && blockIdx.x * 8 + threadIdx.x < outs) {
        const int oo = blockIdx.x * 8 + threadIdx.x;
        const float total = ((sums[0][threadIdx.x] + sums[1][threadIdx.x]) + sums[2][threadIdx.x]) + sums[3][threadIdx.x];
        finish<T>(p, oo / p.j, oo % p.j, total);
    }
}

struct Shape {
    bool ok, cols;
    MultiParams p;
};

inline bool al16(const void *q) { return ((uintptr_t)q & 15u) == 0; }

Shape classify(const GemmProblem &g) {
    Shape s{};
    if (g.dtype == DT_F64 || g.reduce || g.nb1 * g.nb2 != 1 || g.k < 1 || g.k >= (1ll << 31)) return s;
    if (g.m >= (1ll << 30) || g.n >= (1ll << 30)) return s;  // 32-bit output indices with room for a block past the end
    if (g.c_rs < 1 || g.c_cs < 1) return s;  // no aliased outputs
    MultiParams &p = s.p;
    const int vec = g.dtype == DT_F32 ? 4 : 8;
    // the cols form keeps up to sixteen vectors where the contraction is long (see below)
    const int rmax = 16;
    if (g.m >= 2 && g.m <= rmax && g.n > rmax) {  // out[r = i, j] = sum_k a[i, k] b[k, j]
        p.vec = g.a; p.vec_k_stride = g.a_cs; p.vec_r_stride = g.a_rs;
        p.mat = g.b; p.mat_k_stride = g.b_rs; p.mat_j_stride = g.b_cs;
        p.out_j_stride = g.c_cs; p.out_r_stride = g.c_rs;
        p.j = (int)g.n; p.r = (int)g.m;
        p.bias_j_stride = g.bias_mode == BIAS_PER_COL; p.bias_r_stride = g.bias_mode == BIAS_PER_ROW;
    } else if (g.n >= 2 && g.n <= rmax && g.m > rmax) {  // out[r = j, i] = sum_k b[k, j] a[i, k]
        p.vec = g.b; p.vec_k_stride = g.b_rs; p.vec_r_stride = g.b_cs;
        p.mat = g.a; p.mat_k_stride = g.a_cs; p.mat_j_stride = g.a_rs;
        p.out_j_stride = g.c_rs; p.out_r_stride = g.c_cs;
        p.j = (int)g.m; p.r = (int)g.n;
        p.bias_j_stride = g.bias_mode == BIAS_PER_ROW; p.bias_r_stride = g.bias_mode == BIAS_PER_COL;
    } else {
        return s;
    }
    // the combine kernels number the r * j outputs with a 32-bit index, a block of 256 past the end included
    if ((int64_t)p.r * (int64_t)p.j >= (1ll << 31) - 256) return s;
    // worth a kernel of its own where streaming the matrix is the cost: a megabyte of it at least
    if ((double)p.j * (double)g.k * (double)dtype_size(g.dtype) < 1048576.0) return s;
    // 16-bit types: once 128-column matrix-core tiles give every compute unit a workgroup they stream the matrix as fast
    // (8 x 1024 x 50264 f16: 18.5 us there, 22.3 us here; f32: 76 against 41 us)
    if (g.dtype != DT_F32 && p.j >= 32768) return s;
    p.out = g.c;
    p.k = (int)g.k;
    p.bias = g.bias;
    p.has_bias = g.bias && g.bias_mode != BIAS_NONE;
    p.accumulate = g.accumulate;
    p.stream = (double)p.j * (double)g.k * (double)dtype_size(g.dtype) >= 268435456.0;
    const uintptr_t mask = dtype_size(g.dtype) - 1;
    if (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c | (uintptr_t)g.bias) & mask) return s;
    if (!al16(p.mat)) return s;
    if (p.mat_j_stride == 1 && p.j % vec == 0 && p.mat_k_stride % vec == 0 && p.mat_k_stride >= p.j) {
        s.ok = true; s.cols = true;
    } else if (p.mat_k_stride == 1 && p.k % vec == 0 && p.mat_j_stride % vec == 0 && p.mat_j_stride >= p.k &&
               p.vec_k_stride == 1 && (p.vec_r_stride % vec == 0) && al16(p.vec)) {
        s.ok = true; s.cols = false;
    }
    // nine to sixteen vectors: where the contraction is long (below, the small-product kernel's k slices are ahead:
    // 16 x 4096 x 4096 24 against 30 us; 10 x 8192 x 1024 with both operands stored k-major 34.5 -> 17 us here)
    // (16-bit types: 128 accumulators a lane, ahead of the split tiles from 16384 terms on -- 10 x 65536 x 256 102 -> 36 us,
    // 9 x 16384 x 2048 55 -> 35 us; at 8192 the tiles lead, 16 x 8192 x 1024 12.4 against 20 us)
    if (p.r > 8 && !(s.cols && g.k >= (g.dtype == DT_F32 ? 8192 : 16384))) s.ok = false;
    return s;
}

// k slices so that the grid has a few workgroups per compute unit
void plan_slices(Shape &s, int dtype) {
    MultiParams &p = s.p;
    const int vec = dtype == DT_F32 ? 4 : 8;
    const int kchunk_max = kchunk_of(p.r), per_wg = 4 * rows_of(p.r);
    const int64_t blocks_j = s.cols ? (p.j + 64 * vec - 1) / (64 * vec) : (p.j + per_wg - 1) / per_wg;
    int slices = 1;
    if (s.cols) {
        slices = (p.k + kchunk_max - 1) / kchunk_max;  // the vector slices must fit the LDS buffer
        // few column blocks (a narrow matrix with a long k): half as many workgroups -- every slice adds R x j partial sums
        // for the combining launch, and with few outputs that launch walks long chains of them (8 x 16384 x 1024 f32:
        // 24.0 -> 17.7 us, 8 x 65536 x 256: 28.9 -> 22.1 us; 4096 columns and more are faster with the thousand)
        const int want = blocks_j <= 4 ? 512 : 1024;
        while (blocks_j * slices < want && p.k / (slices * 2) >= 64) slices *= 2;
    } else {
        // a wave of this form is heavy (4 + R loads a step): it takes eight of them per SIMD to hide the latency of HBM
        while (blocks_j * slices < 2048 && p.k / (slices * 2) >= 64 * vec) slices *= 2;
    }
    int chunk = (p.k + slices - 1) / slices;
    chunk = (chunk + vec - 1) / vec * vec;
    if (s.cols && chunk > kchunk_max) chunk = kchunk_max;
    p.kchunk = chunk;
    p.kslices = (p.k + chunk - 1) / chunk;
}

template <typename T, int R> hipError_t launch_r(const Shape &s, hipStream_t stream) {
    const MultiParams &p = s.p;
    constexpr int VEC = Elem<T>::VEC;
    if (s.cols) {
        dim3 grid((unsigned)((p.j + 64 * VEC - 1) / (64 * VEC)), (unsigned)p.kslices);
        if (p.stream) gemv_multi_cols_kernel<T, R, true><<<grid, 256, 0, stream>>>(p);
        else gemv_multi_cols_kernel<T, R, false><<<grid, 256, 0, stream>>>(p);
    } else if constexpr (R <= 8) {
        constexpr int PER_WG = 4 * rows_of(R);
        dim3 grid((unsigned)((p.j + PER_WG - 1) / PER_WG), (unsigned)p.kslices);
        if (p.stream) gemv_multi_dots_kernel<T, R, true><<<grid, 256, 0, stream>>>(p);
        else gemv_multi_dots_kernel<T, R, false><<<grid, 256, 0, stream>>>(p);
    } else {
        return hipErrorInvalidValue;
    }
    if (p.kslices > 1) {
        const int64_t outs = (int64_t)p.r * p.j;
        if (p.kslices >= 512) gemv_multi_combine_deep_kernel<T><<<dim3((unsigned)((outs + 7) / 8)), 256, 0, stream>>>(p);
        else gemv_multi_combine_kernel<T><<<dim3((unsigned)((outs + 31) / 32)), 256, 0, stream>>>(p);
    }
    return hipGetLastError();
}
template <typename T> hipError_t launch_t(const Shape &s, hipStream_t stream) {
    if (s.p.r > 8) return launch_r<T, 16>(s, stream);
    return s.p.r <= 2 ? launch_r<T, 2>(s, stream) : s.p.r <= 4 ? launch_r<T, 4>(s, stream) : launch_r<T, 8>(s, stream);
}

}  // namespace

bool gemv_multi_supported(const GemmProblem &g) {
    Shape s = classify(g);
    if (!s.ok) return false;
    plan_slices(s, g.dtype);
    return s.p.kslices <= 65535;  // the k slices are grid.y
}

// Estimated seconds, for the planner's comparison with the matrix-core kernels (forced sweeps over 2 - 16 vectors against
// matrices of 2 MB - 270 MB, both layouts, f16 and f32): the launch (two with the combining pass) plus the matrix at the
// rate the form streams it.  The 16-bit forms are bound by their multiply-adds, not by memory, once there are more than a
// few vectors (the rate falls with every vector: 4 x 4096 x 4096 f16 A.B 12.9 us, 8 vectors 17.6 us), f32 hardly.
double gemv_multi_time(const GemmProblem &g) {
    Shape s = classify(g);
    if (!s.ok) return 1e300;
    plan_slices(s, g.dtype);
    const bool half = g.dtype != DT_F32;
    const double bytes = (double)s.p.j * (double)g.k * (double)dtype_size(g.dtype);
    const double more = (double)s.p.r - 2.0;
    double rate = s.cols ? (half ? 8.0e12 / (1.0 + 0.19 * more) : 6.3e12 / (1.0 + 0.045 * more))
                         : (half ? 7.5e12 / (1.0 + 0.13 * more) : 6.0e12 / (1.0 + 0.05 * more));
    if (half && bytes > 48e6) rate = std::min(rate, s.cols ? 4.8e12 : 5.4e12);  // beyond what the caches hold between launches
    // two launches (slices + combine) and, in the "cols" form, the vector slices staged through LDS: a matrix of 2 MB takes
    // 5.7 - 6.5 us as dots and 7.4 - 10.7 us as columns (f16, 2 - 8 vectors), f32 5.6 - 8.1 us
    const double fixed = !s.cols ? 5.2e-6 + 0.12e-6 * more : half ? 6.5e-6 + 0.45e-6 * more : 5.0e-6 + 0.3e-6 * more;
    return (s.p.kslices > 1 ? fixed : fixed - 2.0e-6) + bytes / rate;
}

size_t gemv_multi_workspace_bytes(const GemmProblem &g) {
    Shape s = classify(g);
    if (!s.ok) return 0;
    plan_slices(s, g.dtype);
    return s.p.kslices > 1 ? (size_t)s.p.kslices * s.p.r * s.p.j * sizeof(float) : 0;
}

hipError_t launch_gemv_multi(const GemmProblem &g, hipStream_t stream) {
    Shape s = classify(g);
    if (!s.ok) return hipErrorInvalidValue;
    plan_slices(s, g.dtype);
    if (s.p.kslices > 65535 || (s.p.kslices > 1 && !g.workspace)) return hipErrorInvalidValue;
    s.p.ws = g.workspace;
    switch (g.dtype) {
    case DT_F32: return launch_t<float>(s, stream);
    case DT_F16: return launch_t<_Float16>(s, stream);
    case DT_BF16: return launch_t<__bf16>(s, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace dfdx_rocm
