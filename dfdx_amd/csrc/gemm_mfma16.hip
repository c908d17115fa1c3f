// MFMA GEMM for 16-bit inputs (f16 / bf16) with f32 accumulation on gfx950 (CDNA4).
//
// One workgroup computes a BM x BN tile of C.  A and B tiles of BK k-values are
// staged in LDS as [row][k] (k contiguous, rows padded by 16 B so that the 16 B
// fragment reads of consecutive rows fall into distinct banks), double buffered:
// while the matrix cores work on buffer `cur`, the global loads for the next k
// step are in flight into registers and are written to the other buffer after the
// MFMAs have been issued.  One barrier per k step.
//
// Operand layouts are handled in the loaders, with no transpose copy in HBM:
//   k-contiguous operand (A row-major, or B stored [N][K]): 16 B global loads along k
//     go straight to LDS.
//   m/n-contiguous operand (A stored [K][M], or B row-major [K][N]): 16 B global loads
//     along m/n for KR consecutive k rows, transposed 8xKR in registers with 16-bit
//     packs, then written to LDS k-contiguous.
// The MFMA is issued with the operands swapped (D^T = B^T A^T) so that every lane
// ends up holding 4 consecutive n for one m, i.e. vector stores into row-major C.
//
// Preconditions (checked by mfma16_supported): C has unit column stride; each of A, B
// has one unit stride; pointers, leading strides and batch strides are multiples of
// 8 elements (16 B) and the contiguous extent is a multiple of 8.
#include "gemm_internal.h"
#include "elem.h"
#include <type_traits>

namespace dfdx_rocm {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct Params {
    const uint16_t *a;
    const uint16_t *b;
    uint16_t *c;
    const uint16_t *bias;
    int m, n, k;
    int lda, ldb;  // stride (elements) of the non-unit axis of A / B
    int64_t ldc;
    int64_t a_b1, a_b2, b_b1, b_b2, c_b1, c_b2;
    int nb2;       // inner batch count (batch id -> b1 = id / nb2, b2 = id % nb2)
    int kbatches;  // batches folded into the k loop (reduce mode), else 1
    int tiles_m, tiles_n, tiles_per_batch, total_blocks;
    int accumulate, bias_mode, c_vec;
    int window;  // operands that 16 B-aligned vector loads cannot walk (odd leading dimension, extent or address): window loads
    int group_m;
    // split-k: k-loop steps [split * chunk, +chunk) per workgroup, f32 partial tiles to ws[split][row][col]
    int splits, chunk;
    float *ws;
    int64_t ws_ld, ws_split_stride;
    ConvPatches conv;  // CONV_B kernels: B is the patch matrix of a unit-stride convolution, formed on the fly
};

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};
template <> struct Mma<__bf16> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }  // RNE, quiet NaNs
};

__device__ __forceinline__ u32x4 ldg16(const uint16_t *p, bool pred) {
    u32x4 z = {0u, 0u, 0u, 0u};
    return pred ? *(const u32x4 *)p : z;
}

// Loader of one operand tile: ROWS (m or n extent) x BK, NT threads.
// KC = operand is k-contiguous in global memory.
//
// Per-thread element offsets are computed once (init).  Rows beyond the matrix edge are
// clamped onto the last valid row: they only feed C rows/columns that are never stored, so
// their values do not matter but their addresses must be valid.  Only the k tail needs
// zero fill; full k steps take the unpredicated path.
template <int ROWS, int BK, int NT, bool KC> struct Loader {
    static constexpr int LOADS = ROWS * BK / 8 / NT;  // 16 B loads per thread per k step
    static_assert(LOADS >= 1 && (ROWS * BK / 8) % NT == 0, "tile does not divide over the threads");
    // m/n-contiguous: each unit is KR k-rows x 8 columns
    static constexpr int KR = LOADS >= 8 ? 8 : LOADS;
    static constexpr int UNITS = LOADS / KR;
    static constexpr int NKB = BK / KR;
    static constexpr int CPR = BK / 8;  // 16 B chunks per row (k-contiguous case)
    static constexpr int LDS_ROW = BK + 8;

    u32x4 regs[LOADS];
    uint32_t goff[LOADS];  // byte offset of each load from the tile origin
    int koff[LOADS];  // k index of each load inside the tile (for the tail predicate)
    int soff[KC ? LOADS : UNITS];  // LDS element offset of each store

    __device__ __forceinline__ void init(int ld, int rows_left, int tid) {
        if constexpr (KC) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) {
                const int cid = i * NT + tid;
                const int row = cid / CPR, ch = cid % CPR;
                goff[i] = (uint32_t)(min(row, rows_left - 1) * ld + ch * 8) * 2u;
                koff[i] = ch * 8;
                soff[i] = row * LDS_ROW + ch * 8;
            }
        } else {
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                const int uid = u * NT + tid;
                const int kb = uid % NKB, mb = uid / NKB;
                soff[u] = (mb * 8) * LDS_ROW + kb * KR;
#pragma unroll
                for (int r = 0; r < KR; r++) {
                    goff[u * KR + r] = (uint32_t)((kb * KR + r) * ld + max(min(mb * 8, rows_left - 8), 0)) * 2u;
                    koff[u * KR + r] = kb * KR + r;
                }
            }
        }
    }

    // Patch-matrix form of an m/n-contiguous operand (convolutions at unit stride): row k = (channel, tap) of the
    // matrix is the channel's plane moved by the tap, zero where the window leaves the image; column = pixel.  A
    // unit's 8 columns are 8 consecutive pixels: one window of an image row, or -- when the row width is not a
    // multiple of 8 -- the end of one row and the start of the next (rows are at least 8 pixels wide).  Columns past
    // the last pixel only feed C columns that are never stored.  `planes` points at channel 0 of the image (uniform),
    // k0 is the tile's first k.
    int py[KC ? 1 : UNITS], px[KC ? 1 : UNITS];
    __device__ __forceinline__ void init_conv(const ConvPatches &cv, int col0, int cols_left, int tid) {
        if constexpr (!KC) {
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                const int mb = (u * NT + tid) / NKB;
                const int col = col0 + min(mb * 8, ((cols_left + 7) & ~7) - 8);
                py[u] = col / cv.w_dst;
                px[u] = col - py[u] * cv.w_dst;
            }
        }
    }
    __device__ __forceinline__ void load_conv(const ConvPatches &cv, const uint16_t *planes, int k0, int k_total) {
        if constexpr (!KC) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) {
                const int k = k0 + koff[i], u = i / KR;
                const int c = cv.taps == 9 ? k / 9 : (cv.taps == 1 ? k : k / cv.taps);
                const int tap = k - c * cv.taps;
                const int k1 = cv.ksize == 3 ? tap / 3 : (cv.ksize == 1 ? 0 : tap / cv.ksize);
                const int k2 = tap - k1 * cv.ksize;
                const int y = py[u] + cv.off_y + cv.step_y * k1, x = cv.off_x + cv.step_x * k2;
                const uint16_t *row = planes + (int64_t)c * cv.plane + (int64_t)y * cv.w_src;
                u32x4 w = row_window_bytes<2>(row, k < k_total && y >= 0 && y < cv.h_src, px[u] + x, cv.w_src);
                const int n1 = cv.w_dst - px[u];  // pixels left in this image row
                if (n1 < 8) {  // the other 8 - n1 pixels start the next row
                    const u32x4 w2 = row_window_bytes<2>(row + cv.w_src, k < k_total && y + 1 >= 0 && y + 1 < cv.h_src, x, cv.w_src);
#pragma unroll
                    for (int j = 0; j < 4; j++) w[j] &= n1 >= 2 * j + 2 ? 0xffffffffu : (n1 == 2 * j + 1 ? 0x0000ffffu : 0u);
                    const u32x4 hi = shift128(w2, -16 * n1);
#pragma unroll
                    for (int j = 0; j < 4; j++) w[j] |= hi[j];
                }
                regs[i] = w;
            }
        }
    }

    // `g` points at the tile origin (uniform across the workgroup).
    __device__ __forceinline__ void load(const uint16_t *g) {
#pragma unroll
        for (int i = 0; i < LOADS; i++) regs[i] = *(const u32x4 *)((const char *)g + goff[i]);
    }
    __device__ __forceinline__ void load_tail(const uint16_t *g, int k_left) {
#pragma unroll
        for (int i = 0; i < LOADS; i++) regs[i] = ldg16((const uint16_t *)((const char *)g + goff[i]), koff[i] < k_left);
    }

    // The same tile for an operand whose rows do not start on 16 B boundaries, or whose contiguous extent is not a
    // multiple of 8: every 8-element piece is one unaligned 16 B load from the nearest window inside the matrix,
    // shifted into place, zeros beyond the extent (row_window_bytes).  `g` = tile origin (first row r0, first k k0);
    // the contiguous extent (k_total if KC, else rows_total) is at least 8.
    __device__ __forceinline__ void load_window(const uint16_t *g, int ld, int k0, int k_total, int r0, int rows_total, int tid) {
        if constexpr (KC) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) {
                const char *row = (const char *)g + (goff[i] - (uint32_t)koff[i] * 2u) - (int64_t)k0 * 2;  // k = 0 of the (clamped) row
                regs[i] = row_window_bytes<2>(row, true, k0 + koff[i], k_total);
            }
        } else {
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                const int mb = (u * NT + tid) / NKB;
#pragma unroll
                for (int r = 0; r < KR; r++) {
                    const int i = u * KR + r;
                    const char *krow = (const char *)g + (int64_t)koff[i] * ld * 2 - (int64_t)r0 * 2;  // row 0 of this k
                    regs[i] = row_window_bytes<2>(krow, k0 + koff[i] < k_total, r0 + mb * 8, rows_total);
                }
            }
        }
    }

    __device__ __forceinline__ void store(uint16_t *lds) const {
        if constexpr (KC) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) *(u32x4 *)(lds + soff[i]) = regs[i];
        } else {
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                uint16_t *dst = lds + soff[u];
#pragma unroll
                for (int j = 0; j < 8; j++) {  // output row j: column mb*8+j of the unit, KR k-values
                    uint32_t w[KR / 2];
#pragma unroll
                    for (int q = 0; q < KR / 2; q++) {
                        const uint32_t lo = regs[u * KR + 2 * q][j / 2], hi = regs[u * KR + 2 * q + 1][j / 2];
                        w[q] = (j & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
                    }
                    if constexpr (KR == 8) {
                        u32x4 v = {w[0], w[1], w[2], w[3]};
                        *(u32x4 *)(dst + j * LDS_ROW) = v;
                    } else if constexpr (KR == 4) {
                        u32x2 v = {w[0], w[1]};
                        *(u32x2 *)(dst + j * LDS_ROW) = v;
                    } else {
                        *(uint32_t *)(dst + j * LDS_ROW) = w[0];
                    }
                }
            }
        }
    }
};

template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool CONV_B = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_mfma16_kernel(const Params p) {
    static_assert(!CONV_B || !B_KC, "the patch-matrix form is an n-contiguous B");
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int LDS_ROW = BK + 8;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 16 == 0, "bad tile");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *As = (uint16_t *)smem;          // [2][BM][LDS_ROW]
    uint16_t *Bs = As + 2 * BM * LDS_ROW;     // [2][BN][LDS_ROW]

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = tid / 64;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    const int l32 = lane % 32, lh = lane / 32;

    // ---- which tile -------------------------------------------------------
    const int work = xcd_remap(blockIdx.x, p.total_blocks);
    const int bidx = work / p.tiles_per_batch;  // batch, or k split
    const int batch = p.splits > 1 ? 0 : bidx;
    const int split = p.splits > 1 ? bidx : 0;
    const int tile = work % p.tiles_per_batch;
    const int gsize = p.group_m * p.tiles_n;
    const int group = tile / gsize;
    const int first_m = group * p.group_m;
    const int gm = min(p.tiles_m - first_m, p.group_m);
    const int tm_idx = first_m + (tile % gsize) % gm;
    const int tn_idx = (tile % gsize) / gm;
    const int bm0 = tm_idx * BM, bn0 = tn_idx * BN;

    const int ktiles = (p.k + BK - 1) / BK;
    const int it0 = split * p.chunk;  // this workgroup owns k-loop steps [it0, it0 + iters)
    const int iters = min(ktiles * p.kbatches - it0, p.chunk);

    // Uniform pointers to the origin of the NEXT tile to fetch, advanced incrementally; the
    // divisions needed to locate a batch run once per batch, not once per k step.
    auto a_origin = [&](int kb) -> const uint16_t * {
        const uint16_t *base = p.a + (int64_t)(kb / p.nb2) * p.a_b1 + (int64_t)(kb % p.nb2) * p.a_b2;
        return A_KC ? base + (int64_t)bm0 * p.lda : base + bm0;
    };
    auto b_origin = [&](int kb) -> const uint16_t * {
        const uint16_t *base = p.b + (int64_t)(kb / p.nb2) * p.b_b1 + (int64_t)(kb % p.nb2) * p.b_b2;
        if constexpr (CONV_B) return base;  // channel 0 of this batch's image
        return B_KC ? base + (int64_t)bn0 * p.ldb : base + bn0;
    };
    const int64_t a_step = A_KC ? BK : (int64_t)BK * p.lda;
    const int64_t b_step = B_KC ? BK : (int64_t)BK * p.ldb;
    int f_kb = p.kbatches > 1 ? it0 / ktiles : batch;  // batch of the next tile to fetch
    int f_kt = p.kbatches > 1 ? it0 % ktiles : it0;    // its k-tile index
    const uint16_t *a_next = a_origin(f_kb) + f_kt * a_step;
    const uint16_t *b_next = CONV_B ? b_origin(f_kb) : b_origin(f_kb) + f_kt * b_step;

    Loader<BM, BK, NT, A_KC> la;
    Loader<BN, BK, NT, B_KC> lb;
    la.init(p.lda, p.m - bm0, tid);
    lb.init(p.ldb, p.n - bn0, tid);
    if constexpr (CONV_B) lb.init_conv(p.conv, bn0, p.n - bn0, tid);
    auto advance = [&]() {
        a_next += a_step;
        if constexpr (!CONV_B) b_next += b_step;
        if (++f_kt == ktiles) {
            f_kt = 0;
            if (p.kbatches > 1 && ++f_kb < p.kbatches) {
                a_next = a_origin(f_kb);
                b_next = b_origin(f_kb);
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const uint16_t *a_frag0 = As + (wm0 + l32) * LDS_ROW + lh * 8;
    const uint16_t *b_frag0 = Bs + (wn0 + l32) * LDS_ROW + lh * 8;

    // The k loop exists twice: K a multiple of BK runs with unpredicated loads only; any
    // other K runs with the k-tail predicate on every load.
    auto k_loop = [&](auto tail_tag, auto window_tag) {
        constexpr bool TAIL = decltype(tail_tag)::value, WINDOW = decltype(window_tag)::value;
        auto fetch = [&]() {
            if constexpr (WINDOW) {
                la.load_window(a_next, p.lda, f_kt * BK, p.k, bm0, p.m, tid);
                if constexpr (!CONV_B) lb.load_window(b_next, p.ldb, f_kt * BK, p.k, bn0, p.n, tid);
            } else if constexpr (TAIL) {
                const int kl = p.k - f_kt * BK;
                la.load_tail(a_next, kl);
                if constexpr (!CONV_B) lb.load_tail(b_next, kl);
            } else {
                la.load(a_next);
                if constexpr (!CONV_B) lb.load(b_next);
            }
            if constexpr (CONV_B) lb.load_conv(p.conv, b_next, f_kt * BK, p.k);
            advance();
        };
        if (iters > 0) {
            fetch();
            la.store(As);
            lb.store(Bs);
        }
        __syncthreads();
        for (int it = 0; it < iters; it++) {
            const int cur = it & 1;
            const bool more = it + 1 < iters;
            if (more) fetch();
            const uint16_t *af_base = a_frag0 + cur * BM * LDS_ROW;
            const uint16_t *bf_base = b_frag0 + cur * BN * LDS_ROW;
#pragma unroll
            for (int ks = 0; ks < BK / 16; ks++) {
                u32x4 af[TM], bf[TN];
#pragma unroll
                for (int i = 0; i < TM; i++) af[i] = *(const u32x4 *)(af_base + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
                for (int j = 0; j < TN; j++) bf[j] = *(const u32x4 *)(bf_base + j * 32 * LDS_ROW + ks * 16);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = Mma<T>::mfma(bf[j], af[i], acc[i][j]);
            }
            if (more) {
                la.store(As + (cur ^ 1) * BM * LDS_ROW);
                lb.store(Bs + (cur ^ 1) * BN * LDS_ROW);
            }
            __syncthreads();
        }
    };
    if constexpr (!CONV_B) {
        if (p.window) k_loop(std::true_type{}, std::true_type{});
        else if (p.k % BK == 0) k_loop(std::false_type{}, std::false_type{});
        else k_loop(std::true_type{}, std::false_type{});
    } else {
        if (p.k % BK == 0) k_loop(std::false_type{}, std::false_type{});
        else k_loop(std::true_type{}, std::false_type{});
    }

    // ---- epilogue: lane holds m = l32 (per tile), n = 8g + 4*lh + 0..3 --------
    if (p.splits > 1) {  // f32 partial tile into the workspace (padded to whole tiles: no bounds checks)
        float *wbase = p.ws + split * p.ws_split_stride;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            float *wrow = wbase + (int64_t)(bm0 + wm0 + i * 32 + l32) * p.ws_ld + bn0 + wn0 + lh * 4;
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    typedef float f32x4 __attribute__((ext_vector_type(4)));
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][g * 4 + e];
                    *(f32x4 *)(wrow + j * 32 + g * 8) = v;
                }
        }
        return;
    }
    const int cb = p.kbatches > 1 ? 0 : batch;
    uint16_t *cbase = p.c + (int64_t)(cb / p.nb2) * p.c_b1 + (int64_t)(cb % p.nb2) * p.c_b2;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int gm_row = bm0 + wm0 + i * 32 + l32;
        if (gm_row >= p.m) continue;
        uint16_t *crow = cbase + (int64_t)gm_row * p.ldc;
        const float rbias = (p.bias_mode == BIAS_PER_ROW) ? Mma<T>::to_f32(p.bias[gm_row]) : 0.0f;
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int gn = bn0 + wn0 + j * 32 + g * 8 + lh * 4;
                if (gn >= p.n) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[i][j][g * 4 + e] + rbias;
                // four columns as one 8-byte access: where everything is on the 8-byte grid (c_vec: n % 4 == 0, so the four
                // are all in range), and otherwise wherever the four are in range -- from an address that is only
                // element-aligned (global memory allows it; a 197-column row of attention scores otherwise goes out as
                // 2-byte stores, one row per lane)
                typedef u32x2 u32x2_unaligned __attribute__((aligned(2)));
                if (p.c_vec || gn + 4 <= p.n) {
                    if (p.bias_mode == BIAS_PER_COL) {
                        const u32x2 bv = *(const u32x2_unaligned *)(p.bias + gn);
                        v[0] += Mma<T>::to_f32((uint16_t)(bv[0] & 0xffffu));
                        v[1] += Mma<T>::to_f32((uint16_t)(bv[0] >> 16));
                        v[2] += Mma<T>::to_f32((uint16_t)(bv[1] & 0xffffu));
                        v[3] += Mma<T>::to_f32((uint16_t)(bv[1] >> 16));
                    }
                    if (p.accumulate) {
                        const u32x2 old = *(const u32x2_unaligned *)(crow + gn);
                        v[0] += Mma<T>::to_f32((uint16_t)(old[0] & 0xffffu));
                        v[1] += Mma<T>::to_f32((uint16_t)(old[0] >> 16));
                        v[2] += Mma<T>::to_f32((uint16_t)(old[1] & 0xffffu));
                        v[3] += Mma<T>::to_f32((uint16_t)(old[1] >> 16));
                    }
                    u32x2 o;
                    o[0] = (uint32_t)Mma<T>::from_f32(v[0]) | ((uint32_t)Mma<T>::from_f32(v[1]) << 16);
                    o[1] = (uint32_t)Mma<T>::from_f32(v[2]) | ((uint32_t)Mma<T>::from_f32(v[3]) << 16);
                    *(u32x2_unaligned *)(crow + gn) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (gn + e >= p.n) break;
                        float x = v[e];
                        if (p.bias_mode == BIAS_PER_COL) x += Mma<T>::to_f32(p.bias[gn + e]);
                        if (p.accumulate) x += Mma<T>::to_f32(crow[gn + e]);
                        crow[gn + e] = Mma<T>::from_f32(x);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ host side --

struct Variant {
    const char *name;
    int bm, bn, bk, waves_m, waves_n;
};

// Variant ids are 1-based indices into this list: X(id, BM, BN, BK, WAVES_M, WAVES_N).
#define DFDX_MFMA16_VARIANTS(X) \
    X(1, 256, 256, 64, 2, 4)    \
    X(2, 256, 256, 64, 2, 2)    \
    X(3, 256, 128, 64, 2, 2)    \
    X(4, 128, 128, 64, 2, 2)    \
    X(5, 128, 64, 64, 4, 1)     \
    X(6, 64, 64, 64, 2, 2)      \
    X(7, 256, 256, 32, 2, 4)    \
    X(8, 256, 128, 32, 2, 2)    \
    X(9, 128, 128, 32, 2, 2)    \
    X(10, 128, 256, 32, 2, 2)

constexpr Variant kVariants[] = {
#define X(id, bm, bn, bk, wm, wn) {#bm "x" #bn "x" #bk "_w" #wm "x" #wn, bm, bn, bk, wm, wn},
    DFDX_MFMA16_VARIANTS(X)
#undef X
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <typename T, int BM, int BN, int BK, int WM, int WN>
hipError_t launch_layout(const Params &p, bool a_kc, bool b_kc, hipStream_t stream) {
    constexpr int NT = WM * WN * 64;
    constexpr size_t lds = (size_t)2 * (BM + BN) * (BK + 8) * 2;
    dim3 grid((unsigned)p.total_blocks), block(NT);
#define DFDX_LAUNCH(AKC, BKC)                                                                                   \
    do {                                                                                                        \
        auto kern = gemm_mfma16_kernel<T, BM, BN, BK, WM, WN, AKC, BKC>;                                        \
        static PerDevice configured_on;                                                                         \
        std::atomic<int> &configured = configured_on.here();                                                    \
        if (!configured.load(std::memory_order_acquire)) {                                                      \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                               (int)lds);                                                       \
            if (e != hipSuccess) return e;                                                                      \
            configured.store(1, std::memory_order_release);                                                     \
        }                                                                                                       \
        kern<<<grid, block, lds, stream>>>(p);                                                                  \
    } while (0)
    if (a_kc && b_kc) DFDX_LAUNCH(true, true);
    else if (a_kc && !b_kc) DFDX_LAUNCH(true, false);
    else if (!a_kc && b_kc) DFDX_LAUNCH(false, true);
    else DFDX_LAUNCH(false, false);
#undef DFDX_LAUNCH
    return hipGetLastError();
}

// The patch-matrix kernels: A k-contiguous (filters), B formed from image planes.
template <typename T, int BM, int BN, int BK, int WM, int WN> hipError_t launch_conv_layout(const Params &p, hipStream_t stream) {
    constexpr int NT = WM * WN * 64;
    constexpr size_t lds = (size_t)2 * (BM + BN) * (BK + 8) * 2;
    auto kern = gemm_mfma16_kernel<T, BM, BN, BK, WM, WN, true, false, true>;
    static PerDevice configured_on;
    std::atomic<int> &configured = configured_on.here();
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured.store(1, std::memory_order_release);
    }
    kern<<<dim3((unsigned)p.total_blocks), dim3(NT), lds, stream>>>(p);
    return hipGetLastError();
}
template <typename T> hipError_t launch_conv_variant(int variant, const Params &p, hipStream_t s) {
    switch (variant) {
    case 1: return launch_conv_layout<T, 256, 256, 64, 2, 4>(p, s);
    case 3: return launch_conv_layout<T, 256, 128, 64, 2, 2>(p, s);
    case 4: return launch_conv_layout<T, 128, 128, 64, 2, 2>(p, s);
    case 5: return launch_conv_layout<T, 128, 64, 64, 4, 1>(p, s);
    case 6: return launch_conv_layout<T, 64, 64, 64, 2, 2>(p, s);
    default: return hipErrorInvalidValue;
    }
}

template <typename T> hipError_t launch_variant(int variant, const Params &p, bool a_kc, bool b_kc, hipStream_t s) {
    switch (variant) {
#define X(id, bm, bn, bk, wm, wn) \
    case id: return launch_layout<T, bm, bn, bk, wm, wn>(p, a_kc, b_kc, s);
        DFDX_MFMA16_VARIANTS(X)
#undef X
    default: return hipErrorInvalidValue;
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// Layout of a (rows x kdim) operand: k-contiguous when the k stride is 1 (or k has one
// element and rows are 16 B apart), rows-contiguous when the row stride is 1.
struct OperandLayout {
    bool ok, kc;
    bool window;  // walkable, but not by 16 B-aligned loads: odd leading dimension or extent (the kernel's window loads)
    int64_t ld;
};
inline OperandLayout classify(int64_t rows, int64_t kdim, int64_t row_stride, int64_t k_stride) {
    OperandLayout r{false, false, false, 0};
    if (k_stride == 1 && kdim % 8 == 0 && (rows == 1 || (row_stride % 8 == 0 && row_stride >= kdim))) {
        r.ok = true; r.kc = true; r.ld = rows == 1 ? kdim : row_stride;
    } else if (row_stride == 1 && rows % 8 == 0 && (kdim == 1 || (k_stride % 8 == 0 && k_stride >= rows))) {
        r.ok = true; r.kc = false; r.ld = kdim == 1 ? rows : k_stride;
    } else if (k_stride == 1 && kdim >= 8 && (rows == 1 || row_stride >= kdim)) {
        r.ok = true; r.kc = true; r.window = true; r.ld = rows == 1 ? kdim : row_stride;
    } else if (row_stride == 1 && rows >= 8 && (kdim == 1 || k_stride >= rows)) {
        r.ok = true; r.kc = false; r.window = true; r.ld = kdim == 1 ? rows : k_stride;
    }
    return r;
}
// Window loads for the whole launch when either operand needs them, or an address / batch stride is not 16 B-aligned.
inline bool needs_window(const GemmProblem &p, const OperandLayout &la, const OperandLayout &lb) {
    if (la.window || lb.window || !aligned16(p.a) || !aligned16(p.b)) return true;
    return p.nb1 * p.nb2 > 1 && (p.a_b1 % 8 || p.a_b2 % 8 || p.b_b1 % 8 || p.b_b2 % 8);
}

}  // namespace

// Variant ids 1..kNumVariants are the register-staged kernels of this file; higher ids are the LDS-DMA kernels; the
// last id is the small-product kernel (gemm_small.hip).
int mfma16_small_variant() { return kNumVariants + mfma16dma_variant_count() + 1; }
int mfma16_variant_count() { return mfma16_small_variant(); }
const char *mfma16_variant_name(int v) {
    if (v == mfma16_small_variant()) return "small_16x16_ksliced";
    if (v > kNumVariants) return mfma16dma_variant_name(v - kNumVariants);
    return (v >= 1) ? kVariants[v - 1].name : "?";
}

bool mfma16_supported(const GemmProblem &p, int variant) {
    if (variant == mfma16_small_variant()) return (p.dtype == DT_F16 || p.dtype == DT_BF16) && small_supported(p);
    if (variant > kNumVariants) return mfma16dma_supported(p, variant - kNumVariants);
    if (p.dtype != DT_F16 && p.dtype != DT_BF16) return false;
    if (variant < 1) return false;
    if (p.m < 1 || p.n < 1 || p.k < 1) return false;
    if (p.m > (1 << 30) || p.n > (1 << 30) || p.k > (1 << 30)) return false;
    if (p.c_cs != 1 && p.n != 1) return false;
    if (p.n > 1 && p.m > 1 && p.c_rs < p.n) return false;
    const OperandLayout la = classify(p.m, p.k, p.a_rs, p.a_cs);
    const OperandLayout lb = classify(p.n, p.k, p.b_cs, p.b_rs);
    if (!la.ok || !lb.ok) return false;
    const Variant &v = kVariants[variant - 1];
    // 32-bit offsets inside one tile
    if (la.ld * (la.kc ? v.bm : v.bk) >= (1ll << 30) || lb.ld * (lb.kc ? v.bn : v.bk) >= (1ll << 30)) return false;
    if (((uintptr_t)p.a | (uintptr_t)p.b) & 1u) return false;  // elements sit on 2 B boundaries at least
    if (p.nb1 * p.nb2 > 1 && (p.a_b1 < 0 || p.a_b2 < 0 || p.b_b1 < 0 || p.b_b2 < 0)) return false;
    const int64_t tiles = ((p.m + v.bm - 1) / v.bm) * ((p.n + v.bn - 1) / v.bn);
    const int64_t blocks = tiles * (p.reduce ? 1 : p.nb1 * p.nb2);
    if (blocks >= (1ll << 31) || p.nb1 * p.nb2 >= (1ll << 31)) return false;
    if (p.k * (p.reduce ? p.nb1 * p.nb2 : 1) >= (1ll << 31)) return false;
    return true;
}

int mfma16_dma_first_variant() { return kNumVariants + 1; }

static int pick_staged(const GemmProblem &p, int compute_units, bool check_support);

int mfma16_pick_variant(const GemmProblem &p, int compute_units) {
    if (const int d = mfma16dma_pick_variant(p, compute_units)) return kNumVariants + d;
    // Least estimated time among the BK = 64 tiles: the work of the padded tiles over the tile's rate (measured at
    // 4096^3 relative to 256x256: 821 TFLOP/s down to 377 for 64x64) and over the share of the chip its workgroups
    // fill.  Per-image convolution GEMMs with 64 or 96 rows run 1.5-1.8x faster on the small tiles than on the
    // largest tile that fills the chip.
    return pick_staged(p, compute_units, true);
}

static int pick_staged(const GemmProblem &p, int compute_units, bool check_support) {
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int candidates[] = {1, 3, 4, 5, 6};
    const double rate[] = {1.0, 0.60, 0.73, 0.54, 0.46};
    int best = 0;
    double best_time = 1e300;
    for (int i = 0; i < 5; i++) {
        const int v = candidates[i];
        if (check_support && !mfma16_supported(p, v)) continue;
        const Variant &t = kVariants[v - 1];
        const double blocks = (double)((p.m + t.bm - 1) / t.bm) * (double)((p.n + t.bn - 1) / t.bn) * (double)nbatch;
        const int s = mfma16_plan_splits(p, v, compute_units, 0);
        const double fill = std::min(1.0, blocks * s / std::max(1, compute_units));
        // a split adds the f32 round trip of its partial tiles: s * 8 bytes per padded C element against 2 * k flops
        const double round_trip = s > 1 ? 1.0 + (double)s * 8.0 * 250.0 / (2.0 * (double)std::max<int64_t>(p.k, 1)) : 1.0;
        const double time = blocks * t.bm * t.bn / (rate[i] * fill) * round_trip;
        if (time < best_time) {
            best_time = time;
            best = v;
        }
    }
    return best;
}

// Split-k of the register-staged family: for products whose tiles leave most of the chip idle while the contraction is
// long (an LM head's dX off the 16-byte grid: 32 tiles of 256 x 256, k = 50257).  Pieces of at least 4 k tiles, at most
// 16 of them (up to 64 while a piece keeps 16 k tiles), no more than fill the chip once; none may be empty.
int mfma16_plan_splits(const GemmProblem &p, int variant, int compute_units, int forced_splits) {
    if (variant < 1 || variant > kNumVariants) return 1;
    const Variant &t = kVariants[variant - 1];
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t total_iters = ((p.k + t.bk - 1) / t.bk) * (p.reduce ? p.nb1 * p.nb2 : 1);
    if (nbatch != 1 || p.c_cs != 1 || total_iters < 2) return 1;
    auto valid = [&](int64_t s) { return s == 1 || (s - 1) * ((total_iters + s - 1) / s) < total_iters; };
    int64_t s;
    if (forced_splits > 0) {
        s = std::min<int64_t>(forced_splits, total_iters);
    } else {
        const int64_t blocks = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn);
        // (a long contraction -- a filter gradient summed over a batch of images -- may take up to 64 pieces of 16+ k tiles)
        const int64_t pieces = std::max<int64_t>(std::min<int64_t>(16, total_iters / 4), std::min<int64_t>(64, total_iters / 16));
        s = std::min<int64_t>(pieces, std::max<int64_t>(1, compute_units / blocks));
        if (s < 2) return 1;
    }
    while (!valid(s)) s--;
    return (int)s;
}

// Estimated seconds of a register-staged variant, for the comparison with the small-product kernel: a lone workgroup's
// k tile takes 1.1 us (load -> LDS -> MFMA chain: 64 x 64 x 64 tiles measure 3.0 / 5.5 / 7.5 us for 1 / 3 / 5 k tiles),
// a full chip runs at the variant's rate; a split adds its second launch.
double mfma16_staged_time(const GemmProblem &p, int variant, int splits, int compute_units) {
    if (variant < 1 || variant > kNumVariants) return 1e300;
    const Variant &t = kVariants[variant - 1];
    const int cus = std::max(1, compute_units);
    const double rate[kNumVariants] = {1.0, 0.8, 0.60, 0.73, 0.54, 0.46};
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t total_iters = ((p.k + t.bk - 1) / t.bk) * (p.reduce ? p.nb1 * p.nb2 : 1);
    const double blocks = (double)((p.m + t.bm - 1) / t.bm) * (double)((p.n + t.bn - 1) / t.bn) * (double)nbatch * splits;
    const double step = std::max(1.1e-6, 2.0 * t.bm * t.bn * t.bk / (rate[variant - 1] * 821e12 / 256));
    return 2.5e-6 + std::max(1.0, blocks / cus) * (double)((total_iters + splits - 1) / splits) * step + (splits > 1 ? 4e-6 : 0.0);
}

// A few rows (or columns) against a large matrix, streamed by the 64 x 64 tile with the contraction split: the tile wastes
// the least of its rows on such a product and its small LDS footprint puts several workgroups on a compute unit, which
// is what streaming at the rate of HBM takes (16 x 8192 x 8192 A.B^T: 26.7 us where the 128-row LDS-DMA tiles take 30.6
// and the k-sliced small kernel 33.5; 8 x 4096 x 4096 A.B: 13.7 us against 15.8).  Returns the variant and its split
// count with an estimate in seconds, or 0 where the candidate does not apply.
int mfma16_skinny_plan(const GemmProblem &p, int compute_units, int forced_splits, int *splits, double *seconds) {
    constexpr int V = 6;  // 64x64x64_w2x2
    static_assert(kNumVariants >= V, "variant table");
    *splits = 1;
    *seconds = 1e300;
    if (std::min(p.m, p.n) > 64 || forced_splits == 1 || !mfma16_supported(p, V)) return 0;
    const Variant &t = kVariants[V - 1];
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t total_iters = ((p.k + t.bk - 1) / t.bk) * (p.reduce ? p.nb1 * p.nb2 : 1);
    if (nbatch != 1 || p.c_cs != 1 || total_iters < 8) return 0;
    const int64_t blocks = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn);
    int64_t s = forced_splits > 0 ? forced_splits
                                  : std::min<int64_t>(std::max<int64_t>(std::min<int64_t>(16, total_iters / 4), std::min<int64_t>(64, total_iters / 16)),
                                                      std::max<int64_t>(1, 2 * (int64_t)compute_units / blocks));
    s = std::min<int64_t>(s, total_iters);
    while (s > 1 && (s - 1) * ((total_iters + s - 1) / s) >= total_iters) s--;  // no empty piece
    if (s < 2) return 0;
    const double bytes = ((double)p.m * (double)p.k + (double)p.k * (double)p.n) * 2.0;
    if (bytes < 8e6) return 0;  // below that the k-sliced small kernel or an unsplit tile is the plan
    *splits = (int)s;
    // two launches, then the operands and the f32 partial tiles (written and read back) at the rate of HBM; an operand that
    // is not stored along k passes through the register transposes of this family
    const bool along_k = p.a_cs == 1 && p.b_rs == 1;
    const double partials = (double)s * (double)blocks * t.bm * t.bn * 4.0 * 2.0;
    *seconds = 6.0e-6 + (bytes * (along_k ? 1.0 : 1.08) + partials) / 6.3e12;
    return V;
}

static void ws_layout16(const GemmProblem &p, int variant, int64_t *ld, int64_t *split_stride) {
    const Variant &v = kVariants[variant - 1];
    *ld = ((p.n + v.bn - 1) / v.bn) * v.bn;
    *split_stride = *ld * (((p.m + v.bm - 1) / v.bm) * v.bm);
}

size_t mfma16_workspace_bytes(const GemmProblem &p, int variant, int splits) {
    if (splits <= 1 || variant < 1 || variant > kNumVariants) return 0;
    int64_t ld, stride;
    ws_layout16(p, variant, &ld, &stride);
    return (size_t)stride * splits * sizeof(float);
}

hipError_t launch_mfma16(const GemmProblem &g, int variant, hipStream_t stream) {
    if (variant == mfma16_small_variant()) return mfma16_supported(g, variant) ? launch_small(g, stream) : hipErrorInvalidValue;
    if (variant > kNumVariants) return launch_mfma16dma(g, variant - kNumVariants, stream);
    if (!mfma16_supported(g, variant)) return hipErrorInvalidValue;
    const Variant &v = kVariants[variant - 1];
    const OperandLayout la = classify(g.m, g.k, g.a_rs, g.a_cs);
    const OperandLayout lb = classify(g.n, g.k, g.b_cs, g.b_rs);
    Params p;
    p.a = (const uint16_t *)g.a; p.b = (const uint16_t *)g.b; p.c = (uint16_t *)g.c; p.bias = (const uint16_t *)g.bias;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.lda = (int)la.ld; p.ldb = (int)lb.ld;
    p.ldc = g.m == 1 ? g.n : g.c_rs;
    p.a_b1 = g.a_b1; p.a_b2 = g.a_b2; p.b_b1 = g.b_b1; p.b_b2 = g.b_b2; p.c_b1 = g.c_b1; p.c_b2 = g.c_b2;
    p.nb2 = (int)g.nb2;
    const int nbatch = (int)(g.nb1 * g.nb2);
    p.kbatches = g.reduce ? nbatch : 1;
    p.tiles_m = (int)((g.m + v.bm - 1) / v.bm);
    p.tiles_n = (int)((g.n + v.bn - 1) / v.bn);
    p.tiles_per_batch = p.tiles_m * p.tiles_n;
    p.total_blocks = p.tiles_per_batch * (g.reduce ? 1 : nbatch);
    p.accumulate = g.accumulate; p.bias_mode = g.bias ? g.bias_mode : BIAS_NONE;
    p.c_vec = (g.n % 4 == 0) && (p.ldc % 4 == 0) && (((uintptr_t)g.c & 7u) == 0) &&
              (g.c_b1 % 4 == 0) && (g.c_b2 % 4 == 0) && (!g.bias || ((uintptr_t)g.bias & 7u) == 0);
    p.window = needs_window(g, la, lb);
    p.group_m = 4;
    p.conv = ConvPatches{};
    const int total_iters = (int)(((g.k + v.bk - 1) / v.bk) * p.kbatches);
    p.splits = 1; p.chunk = total_iters; p.ws = nullptr; p.ws_ld = 0; p.ws_split_stride = 0;
    if (g.splits > 1) {
        if (!g.workspace || p.total_blocks != p.tiles_per_batch) return hipErrorInvalidValue;
        p.splits = g.splits;
        p.chunk = (total_iters + g.splits - 1) / g.splits;
        if ((int64_t)(g.splits - 1) * p.chunk >= total_iters) return hipErrorInvalidValue;
        p.ws = g.workspace;
        ws_layout16(g, variant, &p.ws_ld, &p.ws_split_stride);
        p.total_blocks = p.tiles_per_batch * g.splits;
    }
    const hipError_t e = (g.dtype == DT_F16) ? launch_variant<_Float16>(variant, p, la.kc, lb.kc, stream)
                                             : launch_variant<__bf16>(variant, p, la.kc, lb.kc, stream);
    if (e != hipSuccess || g.splits <= 1) return e;
    return launch_splitk_reduce(g, p.ws_ld, p.ws_split_stride, stream);
}

hipError_t launch_mfma16_conv(const GemmProblem &g, const ConvPatches &conv, int compute_units, hipStream_t stream) {
    if (g.dtype != DT_F16 && g.dtype != DT_BF16) return hipErrorNotSupported;
    if (g.reduce || g.bias || g.m < 1 || g.n < 8 || g.k < 8) return hipErrorNotSupported;
    if (g.m >= (1 << 30) || g.n >= (1 << 30) || g.k >= (1 << 30) || g.nb1 * g.nb2 >= (1ll << 31)) return hipErrorNotSupported;
    const OperandLayout la = classify(g.m, g.k, g.a_rs, g.a_cs);
    if (!la.ok || !la.kc || la.window || !aligned16(g.a) || g.a_b1 % 8 || g.a_b2 % 8 || g.a_b1 < 0 || g.a_b2 < 0) return hipErrorNotSupported;
    if (g.c_cs != 1 || g.n % 4 || g.c_rs % 4 || g.c_rs < g.n || ((uintptr_t)g.c & 7u) || g.c_b1 % 4 || g.c_b2 % 4) return hipErrorNotSupported;
    if (conv.w_dst < 8 || g.n % conv.w_dst || conv.w_src < 8 || conv.taps != conv.ksize * conv.ksize ||
        g.k % conv.taps || g.b_b1 < 0 || g.b_b2 < 0 || ((uintptr_t)g.b & 1u))
        return hipErrorNotSupported;
    if ((int64_t)(g.k / conv.taps) * conv.plane >= (1ll << 31)) return hipErrorNotSupported;
    const int variant = pick_staged(g, compute_units, false);
    const Variant &v = kVariants[variant - 1];
    if (la.ld * v.bm >= (1ll << 30)) return hipErrorNotSupported;
    Params p;
    p.a = (const uint16_t *)g.a; p.b = (const uint16_t *)g.b; p.c = (uint16_t *)g.c; p.bias = nullptr;
    p.m = (int)g.m; p.n = (int)g.n; p.k = (int)g.k;
    p.lda = (int)la.ld; p.ldb = 0;
    p.ldc = g.c_rs;
    p.a_b1 = g.a_b1; p.a_b2 = g.a_b2; p.b_b1 = g.b_b1; p.b_b2 = g.b_b2; p.c_b1 = g.c_b1; p.c_b2 = g.c_b2;
    p.nb2 = (int)g.nb2;
    p.kbatches = 1;
    p.tiles_m = (int)((g.m + v.bm - 1) / v.bm);
    p.tiles_n = (int)((g.n + v.bn - 1) / v.bn);
    p.tiles_per_batch = p.tiles_m * p.tiles_n;
    const int64_t blocks = (int64_t)p.tiles_per_batch * g.nb1 * g.nb2;
    if (blocks >= (1ll << 31)) return hipErrorNotSupported;
    p.total_blocks = (int)blocks;
    p.accumulate = g.accumulate; p.bias_mode = BIAS_NONE;
    p.c_vec = 1;
    p.window = 0;
    p.group_m = 4;
    p.splits = 1; p.chunk = (int)((g.k + v.bk - 1) / v.bk); p.ws = nullptr; p.ws_ld = 0; p.ws_split_stride = 0;
    p.conv = conv;
    if (g.dtype == DT_F16) return launch_conv_variant<_Float16>(variant, p, stream);
    return launch_conv_variant<__bf16>(variant, p, stream);
}

}  // namespace dfdx_rocm
