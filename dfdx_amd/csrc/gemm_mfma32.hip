// MFMA GEMM for f32 on gfx950 (CDNA4): v_mfma_f32_32x32x2_f32, f32 accumulate.
//
// Same skeleton as the 16-bit kernel: BM x BN tile per workgroup, LDS double buffer,
// global loads for step k+1 in flight while the matrix cores work on step k, one
// barrier per step.  An f32 MFMA lane supplies ONE k value per instruction, so no
// transpose is ever needed: a k-contiguous operand is kept in LDS as [row][k] and
// read 16 B at a time (4 k values feeding 4 MFMAs), an m/n-contiguous operand is
// kept as [k][row] and read 4 B at a time.  Which k a lane feeds to which MFMA is
// the same for both operands (k = 8*s + 4*(lane/32) + e for MFMA e of sub-step s),
// which is all the instruction needs.
//
// Preconditions (mfma32_supported): C unit column stride; A and B each have a unit
// stride.  Operands on the 16-byte grid (pointers, leading and batch strides, the
// contiguous extent multiples of 4 elements) take aligned vector loads -- or, for the
// 256 x 256 tile with K % 32 == 0, the LDS-DMA form further down, where the loads write
// LDS themselves; anything else runs the WINDOW instantiation.
#include "gemm_internal.h"
#include "elem.h"

namespace dfdx_rocm {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct Params {
    const float *a;
    const float *b;
    float *c;
    const float *bias;
    int m, n, k;
    int lda, ldb;
    int64_t ldc;
    int64_t a_b1, a_b2, b_b1, b_b2, c_b1, c_b2;
    int nb2, kbatches;
    int tiles_m, tiles_n, tiles_per_batch, total_blocks;
    int accumulate, bias_mode, c_vec;
    int window;  // operands that 16 B-aligned vector loads cannot walk (odd leading dimension, extent or address): window loads
    int group_m;
    // split-k: k-loop steps [split * chunk, +chunk) per workgroup, f32 partial tiles to ws[split][row][col]
    int splits, chunk;
    float *ws;
    int64_t ws_ld, ws_split_stride;
};

__device__ __forceinline__ f32x4 ldg4(const float *p, bool pred) {
    f32x4 z = {0.f, 0.f, 0.f, 0.f};
    return pred ? *(const f32x4 *)p : z;
}

template <int ROWS, int BK, int NT, bool KC> struct Loader {
    static constexpr int LOADS = ROWS * BK / 4 / NT;
    static_assert(LOADS >= 1 && (ROWS * BK / 4) % NT == 0, "tile does not divide over the threads");
    static constexpr int CPR = KC ? BK / 4 : ROWS / 4;               // 16 B chunks per LDS row
    static constexpr int LDS_ROW = KC ? BK + 4 : ROWS + 8;            // floats
    static constexpr int LDS_SIZE = KC ? ROWS * LDS_ROW : BK * LDS_ROW;
    f32x4 regs[LOADS];

    __device__ __forceinline__ void load(const float *g, int ld, int rows_left, int k_left, int tid) {
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            const int cid = i * NT + tid;
            const int r = cid / CPR, ch = cid % CPR;
            if constexpr (KC) regs[i] = ldg4(g + r * ld + ch * 4, r < rows_left && ch * 4 < k_left);
            else regs[i] = ldg4(g + r * ld + ch * 4, ch * 4 < rows_left && r < k_left);
        }
    }
    // The same tile for an operand whose rows do not start on 16 B boundaries, or whose contiguous extent is not a
    // multiple of 4: every 4-element piece is one unaligned 16 B load from the nearest window inside the matrix,
    // shifted into place, zeros beyond the extent (row_window_bytes).  `g` = tile origin: first row r0 of rows_total,
    // first k k0 of k_total; the contiguous extent is at least 4.
    __device__ __forceinline__ void load_window(const float *g, int ld, int r0, int rows_total, int k0, int k_total, int tid) {
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            const int cid = i * NT + tid;
            const int r = cid / CPR, ch = cid % CPR;
            u32x4 w;
            if constexpr (KC) w = row_window_bytes<4>(g + (int64_t)min(r, rows_total - r0 - 1) * ld - k0, true, k0 + ch * 4, k_total);
            else w = row_window_bytes<4>(g + (int64_t)r * ld - r0, k0 + r < k_total, r0 + ch * 4, rows_total);
            regs[i] = __builtin_bit_cast(f32x4, w);
        }
    }
    __device__ __forceinline__ void store_piece(float *lds, int tid, int i) const {
        const int cid = i * NT + tid;
        const int r = cid / CPR, ch = cid % CPR;
        *(f32x4 *)(lds + r * LDS_ROW + ch * 4) = regs[i];
    }
    __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            const int cid = i * NT + tid;
            const int r = cid / CPR, ch = cid % CPR;
            *(f32x4 *)(lds + r * LDS_ROW + ch * 4) = regs[i];
        }
    }
};

// Epilogue shared by the kernels of this file: lane holds m = l32 (per 32 x 32 tile), n = 8g + 4*lh + 0..3.
template <int TM, int TN>
__device__ __forceinline__ void store_tiles32(const Params &p, f32x16 (&acc)[TM][TN], int bm0, int bn0, int wm0, int wn0, int l32, int lh,
                                              int batch, int split) {
    if (p.splits > 1) {  // f32 partial tile into the workspace (padded to whole tiles: no bounds checks)
        float *wbase = p.ws + split * p.ws_split_stride;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            float *wrow = wbase + (int64_t)(bm0 + wm0 + i * 32 + l32) * p.ws_ld + bn0 + wn0 + lh * 4;
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][g * 4 + e];
                    *(f32x4 *)(wrow + j * 32 + g * 8) = v;
                }
        }
        return;
    }
    const int cb = p.kbatches > 1 ? 0 : batch;
    float *cbase = p.c + (int64_t)(cb / p.nb2) * p.c_b1 + (int64_t)(cb % p.nb2) * p.c_b2;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int gm_row = bm0 + wm0 + i * 32 + l32;
        if (gm_row >= p.m) continue;
        float *crow = cbase + (int64_t)gm_row * p.ldc;
        const float rbias = (p.bias_mode == BIAS_PER_ROW) ? p.bias[gm_row] : 0.0f;
        // beta = 1: the old values of this row block are all requested before its first store (clamped addresses);
        // a load issued behind a store can only be waited for together with every outstanding store
        f32x4 old[TN][4];
        if (p.c_vec && p.accumulate) {
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) old[j][g] = *(const f32x4 *)(crow + min(bn0 + wn0 + j * 32 + g * 8 + lh * 4, p.n - 4));
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int gn = bn0 + wn0 + j * 32 + g * 8 + lh * 4;
                if (gn >= p.n) continue;
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[i][j][g * 4 + e] + rbias;
                if (p.c_vec) {
                    if (p.bias_mode == BIAS_PER_COL) v += *(const f32x4 *)(p.bias + gn);
                    if (p.accumulate) v += old[j][g];
                    *(f32x4 *)(crow + gn) = v;
                } else if (gn + 4 <= p.n) {
                    // off the 16-byte grid, all four columns in range: one access from an address that is only
                    // element-aligned (global memory allows it) instead of four, a row per lane
                    typedef f32x4 f32x4_unaligned __attribute__((aligned(4)));
                    if (p.bias_mode == BIAS_PER_COL) v += *(const f32x4_unaligned *)(p.bias + gn);
                    if (p.accumulate) v += *(const f32x4_unaligned *)(crow + gn);
                    *(f32x4_unaligned *)(crow + gn) = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (gn + e >= p.n) break;
                        float x = v[e];
                        if (p.bias_mode == BIAS_PER_COL) x += p.bias[gn + e];
                        if (p.accumulate) x += crow[gn + e];
                        crow[gn + e] = x;
                    }
                }
            }
        }
    }
}

// WINDOW: operands off the 16-byte grid, fetched with window loads (an instantiation of its own: the aligned kernels
// keep their register allocation).
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool WINDOW>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_mfma32_kernel(const Params p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    using LA = Loader<BM, BK, NT, A_KC>;
    using LB = Loader<BN, BK, NT, B_KC>;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 8 == 0, "bad tile");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *As = (float *)smem;             // [2][LA::LDS_SIZE]
    float *Bs = As + 2 * LA::LDS_SIZE;     // [2][LB::LDS_SIZE]

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = tid / 64;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    const int l32 = lane % 32, lh = lane / 32;

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
    const int it0 = split * p.chunk;
    const int iters = min(ktiles * p.kbatches - it0, p.chunk);

    auto a_tile = [&](int it) -> const float * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch;
        const int kt = p.kbatches > 1 ? it % ktiles : it;
        const float *base = p.a + (int64_t)(kb / p.nb2) * p.a_b1 + (int64_t)(kb % p.nb2) * p.a_b2;
        return A_KC ? base + (int64_t)bm0 * p.lda + kt * BK : base + (int64_t)kt * BK * p.lda + bm0;
    };
    auto b_tile = [&](int it) -> const float * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch;
        const int kt = p.kbatches > 1 ? it % ktiles : it;
        const float *base = p.b + (int64_t)(kb / p.nb2) * p.b_b1 + (int64_t)(kb % p.nb2) * p.b_b2;
        return B_KC ? base + (int64_t)bn0 * p.ldb + kt * BK : base + (int64_t)kt * BK * p.ldb + bn0;
    };
    auto k_left = [&](int it) -> int {
        const int kt = p.kbatches > 1 ? it % ktiles : it;
        return p.k - kt * BK;
    };
    auto fetch = [&](LA &la_, LB &lb_, int it) {
        if constexpr (WINDOW) {
            const int k0 = p.k - k_left(it);
            la_.load_window(a_tile(it), p.lda, bm0, p.m, k0, p.k, tid);
            lb_.load_window(b_tile(it), p.ldb, bn0, p.n, k0, p.k, tid);
        } else {
            la_.load(a_tile(it), p.lda, p.m - bm0, k_left(it), tid);
            lb_.load(b_tile(it), p.ldb, p.n - bn0, k_left(it), tid);
        }
    };

    LA la;
    LB lb;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    if (iters > 0) {
        fetch(la, lb, it0);
        la.store(As, tid);
        lb.store(Bs, tid);
    }
    __syncthreads();

    // per-lane fragment origins
    const float *a_frag0 = A_KC ? As + (wm0 + l32) * LA::LDS_ROW + lh * 4 : As + (lh * 4) * LA::LDS_ROW + wm0 + l32;
    const float *b_frag0 = B_KC ? Bs + (wn0 + l32) * LB::LDS_ROW + lh * 4 : Bs + (lh * 4) * LB::LDS_ROW + wn0 + l32;

    // One k step of 8 = 4 MFMA k pairs per tile; a lane's fragment values of a k step: 4 floats per 32-row tile.
    constexpr int KS = BK / 8;
    static_assert(KS >= 2, "the loop below keeps the first and the last k step of a tile in registers");
    auto read_frags = [&](const float *af_base, const float *bf_base, int ks, float(&af)[TM][4], float(&bf)[TN][4]) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            if constexpr (A_KC) {
                const f32x4 v = *(const f32x4 *)(af_base + i * 32 * LA::LDS_ROW + ks * 8);
#pragma unroll
                for (int e = 0; e < 4; e++) af[i][e] = v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) af[i][e] = af_base[(ks * 8 + e) * LA::LDS_ROW + i * 32];
            }
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (B_KC) {
                const f32x4 v = *(const f32x4 *)(bf_base + j * 32 * LB::LDS_ROW + ks * 8);
#pragma unroll
                for (int e = 0; e < 4; e++) bf[j][e] = v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) bf[j][e] = bf_base[(ks * 8 + e) * LB::LDS_ROW + j * 32];
            }
        }
    };
    auto mma = [&](const float(&af)[TM][4], const float(&bf)[TN][4]) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j][e], af[i][e], acc[i][j], 0, 0, 0);
    };

    // The barrier that hands a stage over sits in FRONT of the tile's last k step: its fragments are already in
    // registers, so every wave crosses the barrier with a full group of MFMAs still to issue, and the first fragments
    // of the next tile are requested from LDS before that group -- neither the barrier skew nor the LDS latency
    // leaves the matrix core idle.
    float af_first[TM][4], bf_first[TN][4];
    if (iters > 0) read_frags(a_frag0, b_frag0, 0, af_first, bf_first);
    if (iters > 1) {   // the second tile waits in registers while the first is computed
        fetch(la, lb, it0 + 1);
    }
    for (int it = 0; it < iters; it++) {
        const int cur = it & 1;
        const bool more = it + 1 < iters;
        const float *af_base = a_frag0 + cur * LA::LDS_SIZE;
        const float *bf_base = b_frag0 + cur * LB::LDS_SIZE;
        float af_last[TM][4], bf_last[TN][4];
        {
            // The next tile's registers (requested during the previous tile) go to LDS one 16 B piece at a time
            // BETWEEN the MFMAs of the first k step: every store issues in the shadow of an MFMA instead of in a
            // block in front of the barrier, where the matrix core would sit idle; the registers are then free for the
            // tile after next, which has the rest of this tile to arrive.  Only the stores are conditional: accumulators
            // written under a branch make the register allocator copy them.
            float *an = As + (cur ^ 1) * LA::LDS_SIZE, *bn = Bs + (cur ^ 1) * LB::LDS_SIZE;
            constexpr int M = 4 * TM * TN, S = LA::LOADS + LB::LOADS;
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf_first[j][e], af_first[i][e], acc[i][j], 0, 0, 0);
                        const int n = (e * TM + i) * TN + j;
                        const int before = n * S / M, after = (n + 1) * S / M;
#pragma unroll
                        for (int q = 0; q < S; q++)
                            if (q >= before && q < after && more) {
                                if (q < LA::LOADS) la.store_piece(an, tid, q);
                                else lb.store_piece(bn, tid, q - LA::LOADS);
                            }
                    }
        }
        if (it + 2 < iters) {
            fetch(la, lb, it0 + it + 2);
        }
#pragma unroll
        for (int ks = 1; ks < KS; ks++) {
            if (ks < KS - 1) {
                float af[TM][4], bf[TN][4];
                read_frags(af_base, bf_base, ks, af, bf);
                mma(af, bf);
            } else {
                read_frags(af_base, bf_base, ks, af_last, bf_last);
            }
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (more) read_frags(a_frag0 + (cur ^ 1) * LA::LDS_SIZE, b_frag0 + (cur ^ 1) * LB::LDS_SIZE, 0, af_first, bf_first);
        __builtin_amdgcn_sched_barrier(0);
        mma(af_last, bf_last);
    }

    store_tiles32<TM, TN>(p, acc, bm0, bn0, wm0, wn0, l32, lh, batch, split);
}

// ---- LDS-DMA form -----------------------------------------------------------------------------------------------
// The same product with the operand tiles written into LDS by the load itself (global_load_lds_dwordx4: 16 B per lane,
// 1 KB contiguous per wave instruction) instead of passing through registers: no staging registers, no LDS store
// instructions, no wait for the loads inside the k loop.  Needs whole 16 B pieces (no window mode) and K % 32 == 0.
// LDS layouts (unpadded -- the DMA writes 1 KB runs -- and swizzled on the GLOBAL side: a lane fetches the piece that
// belongs into the slot it writes):
//   k-contiguous operand   [row][32 k]: 16 B piece c of row r sits in slot c ^ ((r >> 1) & 7); a fragment read takes
//                          rows r .. r+31 of one piece: conflict-free;
//   m/n-contiguous operand [k][ROWS]:   piece g of k-row kk sits in slot g ^ (8 * ((kk >> 2) & 1)): the two halves of a
//                          wave read k and k + 4 and land on different banks.
#define DFDX_LDS __attribute__((address_space(3)))
#define DFDX_GLB __attribute__((address_space(1)))

template <int ROWS, int NWAVES, bool KC> struct DmaTile32 {
    static constexpr int BK = 32;
    static constexpr int BYTES = ROWS * BK * 4;
    static constexpr int IPW = BYTES / 1024 / NWAVES;  // 1 KB instructions per wave
    static_assert(BYTES % (1024 * NWAVES) == 0 && IPW >= 1, "tile does not divide over the waves");
    static_assert(ROWS % 64 == 0, "the bank swizzle of an m/n-contiguous tile pairs 32-row groups");
    static constexpr int CPR = KC ? BK / 4 : ROWS / 4;  // 16 B pieces per LDS row
    uint32_t goff[IPW];                                 // byte offset of this lane's piece from the tile origin

    __device__ __forceinline__ void init(int ld, int rows_left, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < IPW; i++) {
            const int slot = (wave * IPW + i) * 64 + lane;
            const int r = slot / CPR, cp = slot % CPR;
            if constexpr (KC) {
                const int c = cp ^ ((r >> 1) & 7);
                goff[i] = (uint32_t)(min(r, rows_left - 1) * ld + c * 4) * 4u;  // rows past the edge repeat the last one
            } else {
                const int g = cp ^ (8 * ((r >> 2) & 1));
                goff[i] = (uint32_t)(r * ld + min(g * 4, rows_left - 4)) * 4u;  // r is a k index here
            }
        }
    }
    // `lds`: byte address of the tile inside the LDS allocation (wave-uniform)
    __device__ __forceinline__ void issue(const float *g, uint32_t lds, int wave) const {
#pragma unroll
        for (int i = 0; i < IPW; i++)
            __builtin_amdgcn_global_load_lds((const DFDX_GLB void *)((const char *)g + goff[i]),
                                             (DFDX_LDS void *)(uintptr_t)(lds + (uint32_t)(wave * IPW + i) * 1024u), 16, 0, 0);
    }
};

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_mfma32_dma_kernel(const Params p) {
    constexpr int BK = 32, NW = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    using TA = DmaTile32<BM, NW, A_KC>;
    using TB = DmaTile32<BN, NW, B_KC>;
    constexpr int STAGE = TA::BYTES + TB::BYTES;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    const int l32 = lane % 32, lh = lane / 32;

    const int work = xcd_remap(blockIdx.x, p.total_blocks);
    const int bidx = work / p.tiles_per_batch;
    const int batch = p.splits > 1 ? 0 : bidx;
    const int split = p.splits > 1 ? bidx : 0;
    const int tile = work % p.tiles_per_batch;
    const int gsize = p.group_m * p.tiles_n;
    const int group = tile / gsize;
    const int first_m = group * p.group_m;
    const int gm = min(p.tiles_m - first_m, p.group_m);
    const int bm0 = (first_m + (tile % gsize) % gm) * BM, bn0 = ((tile % gsize) / gm) * BN;

    const int ktiles = p.k / BK;
    const int it0 = split * p.chunk;
    const int iters = min(ktiles * p.kbatches - it0, p.chunk);

    auto a_tile = [&](int it) -> const float * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch;
        const int kt = p.kbatches > 1 ? it % ktiles : it;
        const float *base = p.a + (int64_t)(kb / p.nb2) * p.a_b1 + (int64_t)(kb % p.nb2) * p.a_b2;
        return A_KC ? base + (int64_t)bm0 * p.lda + kt * BK : base + (int64_t)kt * BK * p.lda + bm0;
    };
    auto b_tile = [&](int it) -> const float * {
        const int kb = p.kbatches > 1 ? it / ktiles : batch;
        const int kt = p.kbatches > 1 ? it % ktiles : it;
        const float *base = p.b + (int64_t)(kb / p.nb2) * p.b_b1 + (int64_t)(kb % p.nb2) * p.b_b2;
        return B_KC ? base + (int64_t)bn0 * p.ldb + kt * BK : base + (int64_t)kt * BK * p.ldb + bn0;
    };
    TA ta;
    TB tb;
    ta.init(p.lda, p.m - bm0, wave, lane);
    tb.init(p.ldb, p.n - bn0, wave, lane);
    const uint32_t smem_addr = (uint32_t)(uintptr_t)(DFDX_LDS const uint8_t *)smem;
    auto request = [&](int it) {  // tile `it` of this work item into stage it & 1
        const uint32_t st = smem_addr + (uint32_t)((it - it0) & 1) * STAGE;
        ta.issue(a_tile(it), st, wave);
        tb.issue(b_tile(it), st + TA::BYTES, wave);
    };

    // per-lane fragment offsets (floats) inside an operand tile, k step ks = 0..3 (8 k each: lane half lh takes 4 of them)
    int a_off[4], b_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        a_off[ks] = A_KC ? (wm0 + l32) * BK + (((ks * 2 + lh) ^ ((l32 >> 1) & 7)) * 4) : (ks * 8 + lh * 4) * BM + wm0 + l32;
        b_off[ks] = B_KC ? (wn0 + l32) * BK + (((ks * 2 + lh) ^ ((l32 >> 1) & 7)) * 4) : (ks * 8 + lh * 4) * BN + wn0 + l32;
    }
    auto read_frags = [&](const uint8_t *stage, auto ks_tag, float(&af)[TM][4], float(&bf)[TN][4]) {
        constexpr int ks = decltype(ks_tag)::value;
        const float *as = (const float *)stage, *bs = (const float *)(stage + TA::BYTES);
#pragma unroll
        for (int i = 0; i < TM; i++) {
            if constexpr (A_KC) {
                const f32x4 v = *(const f32x4 *)(as + a_off[ks] + i * 32 * BK);
#pragma unroll
                for (int e = 0; e < 4; e++) af[i][e] = v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) af[i][e] = as[a_off[ks] + e * BM + ((i ^ lh) * 32)];  // rows ^ 32 for the upper lane half
            }
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (B_KC) {
                const f32x4 v = *(const f32x4 *)(bs + b_off[ks] + j * 32 * BK);
#pragma unroll
                for (int e = 0; e < 4; e++) bf[j][e] = v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) bf[j][e] = bs[b_off[ks] + e * BN + ((j ^ lh) * 32)];
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
    auto mma = [&](const float(&af)[TM][4], const float(&bf)[TN][4]) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j][e], af[i][e], acc[i][j], 0, 0, 0);
    };
    constexpr std::integral_constant<int, 0> K0{};
    constexpr std::integral_constant<int, 1> K1{};
    constexpr std::integral_constant<int, 2> K2{};
    constexpr std::integral_constant<int, 3> K3{};

    // Two tiles are requested ahead.  A tile's fragments are read one k step ahead of their MFMAs, into two register
    // sets in turn; the hand-over (wait for the next tile, barrier, first fragments of the next tile, request for the
    // tile after next into the stage just vacated) sits in front of the LAST k step's MFMAs, whose fragments are in
    // registers by then: every wave crosses the barrier with 4 * TM * TN MFMAs still to issue.
    float fa0[TM][4], fb0[TN][4], fa1[TM][4], fb1[TN][4];
    if (iters > 0) request(it0);
    if (iters > 1) request(it0 + 1);
    if (iters > 0) {
        if (iters > 1) __builtin_amdgcn_s_waitcnt(0x0F70 | ((TA::IPW + TB::IPW) & 15) | (((TA::IPW + TB::IPW) >> 4) << 14));  // first tile in
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        read_frags(smem, K0, fa0, fb0);
    }
    for (int it = 0; it < iters; it++) {
        const uint8_t *cur = smem + (it & 1) * STAGE, *nxt = smem + ((it & 1) ^ 1) * STAGE;
        const bool more = it + 1 < iters;
        // the scheduling fences keep every block of fragment reads IN FRONT of the MFMAs of the step before (left alone,
        // the compiler sinks the reads to their first use and every k step waits for LDS)
        read_frags(cur, K1, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, K2, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, K3, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) & lgkmcnt(0): the next tile has landed, this one has been read
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (more) read_frags(nxt, K0, fa0, fb0);
        if (it + 2 < iters) request(it0 + it + 2);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa1, fb1);
    }
    store_tiles32<TM, TN>(p, acc, bm0, bn0, wm0, wn0, l32, lh, batch, split);
}

struct Variant {
    const char *name;
    int bm, bn, bk, waves_m, waves_n;
    bool dma;    // the LDS-DMA form: aligned operands, K % 32 == 0
    bool small;  // the 16 x 16 tile with the contraction cut over the waves (gemm_small.hip: any strides, no batch)
};
constexpr Variant kVariants[] = {
    {"256x256x32_w2x4", 256, 256, 32, 2, 4, false},
    {"256x256x32_w2x2", 256, 256, 32, 2, 2, false},
    {"256x128x32_w2x2", 256, 128, 32, 2, 2, false},
    {"128x128x32_w2x2", 128, 128, 32, 2, 2, false},
    {"128x64x32_w4x1", 128, 64, 32, 4, 1, false},
    {"64x64x32_w2x2", 64, 64, 32, 2, 2, false},
    {"dma_256x256x32_w2x4", 256, 256, 32, 2, 4, true},
    {"dma_128x128x32_w2x2", 128, 128, 32, 2, 2, true},
    {"small_16x16_ksliced", 16, 16, 16, 1, 1, false, true},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <int BM, int BN, int WM, int WN>
hipError_t launch_dma_layout(const Params &p, bool a_kc, bool b_kc, hipStream_t stream) {
    constexpr int NT = WM * WN * 64;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 32 * 4;
    dim3 grid((unsigned)p.total_blocks), block(NT);
#define DFDX_LAUNCH(AKC, BKC)                                                                                   \
    do {                                                                                                        \
        auto kern = gemm_mfma32_dma_kernel<BM, BN, WM, WN, AKC, BKC>;                                           \
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

template <int BM, int BN, int BK, int WM, int WN, bool WINDOW>
hipError_t launch_layout(const Params &p, bool a_kc, bool b_kc, hipStream_t stream) {
    constexpr int NT = WM * WN * 64;
    dim3 grid((unsigned)p.total_blocks), block(NT);
#define DFDX_LAUNCH(AKC, BKC)                                                                                   \
    do {                                                                                                        \
        constexpr size_t lds = (size_t)2 * 4 * (Loader<BM, BK, NT, AKC>::LDS_SIZE + Loader<BN, BK, NT, BKC>::LDS_SIZE); \
        auto kern = gemm_mfma32_kernel<BM, BN, BK, WM, WN, AKC, BKC, WINDOW>;                                   \
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

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

struct OperandLayout {
    bool ok, kc;
    bool window;  // walkable, but not by 16 B-aligned loads: odd leading dimension or extent (the kernel's window loads)
    int64_t ld;
};
inline OperandLayout classify(int64_t rows, int64_t kdim, int64_t row_stride, int64_t k_stride) {
    OperandLayout r{false, false, false, 0};
    if (k_stride == 1 && kdim % 4 == 0 && (rows == 1 || (row_stride % 4 == 0 && row_stride >= kdim))) {
        r.ok = true; r.kc = true; r.ld = rows == 1 ? kdim : row_stride;
    } else if (row_stride == 1 && rows % 4 == 0 && (kdim == 1 || (k_stride % 4 == 0 && k_stride >= rows))) {
        r.ok = true; r.kc = false; r.ld = kdim == 1 ? rows : k_stride;
    } else if (k_stride == 1 && kdim >= 4 && (rows == 1 || row_stride >= kdim)) {
        r.ok = true; r.kc = true; r.window = true; r.ld = rows == 1 ? kdim : row_stride;
    } else if (row_stride == 1 && rows >= 4 && (kdim == 1 || k_stride >= rows)) {
        r.ok = true; r.kc = false; r.window = true; r.ld = kdim == 1 ? rows : k_stride;
    }
    return r;
}
// Window loads for the whole launch when either operand needs them, or an address / batch stride is not 16 B-aligned.
inline bool needs_window(const GemmProblem &p, const OperandLayout &la, const OperandLayout &lb) {
    if (la.window || lb.window || !aligned16(p.a) || !aligned16(p.b)) return true;
    return p.nb1 * p.nb2 > 1 && (p.a_b1 % 4 || p.a_b2 % 4 || p.b_b1 % 4 || p.b_b2 % 4);
}

}  // namespace

int mfma32_variant_count() { return kNumVariants; }
bool mfma32_ksum_supported(const GemmProblem &p, int variant) {
    return variant >= 1 && variant <= kNumVariants && kVariants[variant - 1].small && p.dtype == DT_F32 && small_ksum_supported(p);
}
const char *mfma32_variant_name(int v) { return (v >= 1 && v <= kNumVariants) ? kVariants[v - 1].name : "?"; }

bool mfma32_supported(const GemmProblem &p, int variant) {
    if (p.dtype != DT_F32) return false;
    if (variant < 1 || variant > kNumVariants) return false;
    if (p.m < 1 || p.n < 1 || p.k < 1) return false;
    if (p.m > (1 << 30) || p.n > (1 << 30) || p.k > (1 << 30)) return false;
    if (p.c_cs != 1 && p.n != 1) return false;
    if (p.n > 1 && p.m > 1 && p.c_rs < p.n) return false;
    if (kVariants[variant - 1].small) return small_supported(p);
    const OperandLayout la = classify(p.m, p.k, p.a_rs, p.a_cs);
    const OperandLayout lb = classify(p.n, p.k, p.b_cs, p.b_rs);
    if (!la.ok || !lb.ok) return false;
    const Variant &v = kVariants[variant - 1];
    if (la.ld * (la.kc ? v.bm : v.bk) >= (1ll << 31) || lb.ld * (lb.kc ? v.bn : v.bk) >= (1ll << 31)) return false;
    if (((uintptr_t)p.a | (uintptr_t)p.b) & 3u) return false;  // elements sit on 4 B boundaries at least
    if (p.nb1 * p.nb2 > 1 && (p.a_b1 < 0 || p.a_b2 < 0 || p.b_b1 < 0 || p.b_b2 < 0)) return false;
    const int64_t tiles = ((p.m + v.bm - 1) / v.bm) * ((p.n + v.bn - 1) / v.bn);
    const int64_t blocks = tiles * (p.reduce ? 1 : p.nb1 * p.nb2);
    if (blocks >= (1ll << 31) || p.nb1 * p.nb2 >= (1ll << 31)) return false;
    if (p.k * (p.reduce ? p.nb1 * p.nb2 : 1) >= (1ll << 31)) return false;
    if (v.dma && (p.k % 32 != 0 || needs_window(p, la, lb))) return false;
    return true;
}

// Split-k for small outputs with a long reduction (weight gradients): when the chosen tile shape leaves most of
// the chip idle, the k loop is cut into up to 16 slices of at least 4 steps each.
// Planner of the f32 family: estimated time of (tile variant, k pieces) = rounds of workgroups x k steps x the time of
// one step at the variant's measured rate (relative to 256x256 at 4096^3: 128 / 130 TFLOP/s down to 101 for 64x64,
// shared by the workgroups a compute unit holds), plus, for a split, the second launch and the workspace round trip.
// Measured against forced sweeps: a per-image convolution GEMM with 64 output channels runs 3.4x faster on 64-row
// tiles than on the largest tile that fills the chip; long-k weight gradients want the big tile cut 16 ways.
namespace {
constexpr double kRate32[kNumVariants] = {1.0, 0.97, 0.90, 0.91, 0.80, 0.78, 1.055, 0.96, 0.0};  // LDS-DMA form: 139-140 against 132 TFLOP/s
constexpr int kPerCu32[kNumVariants] = {1, 1, 1, 2, 2, 4, 1, 2, 1};  // workgroups a compute unit holds (LDS)
constexpr double kCuFlops32 = 130e12 / 256, kSplitLaunch32 = 2.5e-6, kWorkspaceBw32 = 4.5e12;
constexpr double kStepLatency32 = 1.0e-6;  // a k step of a lone small workgroup is bound by its load -> LDS -> MFMA chain

double plan_time32(const GemmProblem &p, int v, int64_t s, int compute_units) {
    const Variant &t = kVariants[v - 1];
    if (t.small) return small_time(p, compute_units);
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t total_iters = ((p.k + t.bk - 1) / t.bk) * (p.reduce ? p.nb1 * p.nb2 : 1);
    const int64_t items = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn) * nbatch * s;
    const int64_t slots = (int64_t)std::max(1, compute_units) * kPerCu32[v - 1];
    const double rounds = std::max(1.0, (double)items / (double)slots);  // workgroups are handed out as others finish
    const int64_t conc = std::min<int64_t>(kPerCu32[v - 1], (items + compute_units - 1) / std::max(1, compute_units));
    const double step = std::max(kStepLatency32, 2.0 * t.bm * t.bn * t.bk / (kRate32[v - 1] * kCuFlops32 / (double)conc));
    double time = rounds * (double)((total_iters + s - 1) / s) * step + 4e-6;
    if (s > 1) time += kSplitLaunch32 + (double)s * (double)p.m * (double)p.n * 4.0 * 2.0 / kWorkspaceBw32;
    return time;
}

// best number of pieces for one variant (1 when it may not be split)
int64_t plan_pieces32(const GemmProblem &p, int v, int compute_units, int forced_splits, double *time) {
    const Variant &t = kVariants[v - 1];
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int64_t total_iters = ((p.k + t.bk - 1) / t.bk) * (p.reduce ? p.nb1 * p.nb2 : 1);
    const bool may_split = nbatch == 1 && p.c_cs == 1 && total_iters >= 2 && !t.small;
    auto valid = [&](int64_t s) { return s == 1 || (s - 1) * ((total_iters + s - 1) / s) < total_iters; };  // no empty piece
    if (forced_splits > 0) {
        int64_t s = may_split ? std::min<int64_t>(forced_splits, total_iters) : 1;
        while (!valid(s)) s--;
        if (time) *time = plan_time32(p, v, s, compute_units);
        return s;
    }
    int64_t best = 1;
    double best_time = plan_time32(p, v, 1, compute_units);
    // (up to 256 pieces: the filter gradient of a first convolution layer is a 32 x 27 result over k = 131 072, and a lone
    // workgroup walks its k tiles at 1.1 us each)
    constexpr int kCandidates[] = {2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256};
    for (int s : kCandidates) {
        if (!may_split || total_iters / s < 4) break;
        if (!valid(s)) continue;
        const double tm = plan_time32(p, v, s, compute_units);
        if (tm < best_time) {
            best_time = tm;
            best = s;
        }
    }
    if (time) *time = best_time;
    return best;
}
}  // namespace

int mfma32_plan_splits(const GemmProblem &p, int variant, int compute_units, int forced_splits) {
    if (variant < 1 || variant > kNumVariants) return 1;
    return (int)plan_pieces32(p, variant, compute_units, forced_splits, nullptr);
}

static void ws_layout32(const GemmProblem &p, int variant, int64_t *ld, int64_t *split_stride) {
    const Variant &v = kVariants[variant - 1];
    *ld = ((p.n + v.bn - 1) / v.bn) * v.bn;
    *split_stride = *ld * (((p.m + v.bm - 1) / v.bm) * v.bm);
}

size_t mfma32_workspace_bytes(const GemmProblem &p, int variant, int splits) {
    if (splits <= 1) return 0;
    int64_t ld, stride;
    ws_layout32(p, variant, &ld, &stride);
    return (size_t)stride * splits * sizeof(float);
}

int mfma32_pick_variant(const GemmProblem &p, int compute_units, int forced_splits, double *seconds) {
    int best = 0;
    double best_time = 1e300;
    for (int v = 1; v <= kNumVariants; v++) {
        if (!mfma32_supported(p, v)) continue;
        // the small kernel adds its k slices in an order of its own: not where the caller asked for the plain k order
        // (nor for large products, except those of a few rows or columns: one row of 16 x 16 tiles streams the large
        // operand once, 16 x 8192 x 8192: 67 us against 103 us on the split 64 x 64 tiles)
        if (kVariants[v - 1].small && (forced_splits == 1 || ((double)p.m * (double)p.n * (double)p.k > 536870912.0 && std::min(p.m, p.n) > 16))) continue;
        double tm;
        plan_pieces32(p, v, compute_units, forced_splits, &tm);
        if (tm < best_time) {
            best_time = tm;
            best = v;
        }
    }
    if (seconds) *seconds = best_time;
    return best;
}

static hipError_t launch_tiles(const Params &p, int variant, bool a_kc, bool b_kc, hipStream_t stream);

hipError_t launch_mfma32(const GemmProblem &g, int variant, hipStream_t stream) {
    if (!mfma32_supported(g, variant)) return hipErrorInvalidValue;
    const Variant &v = kVariants[variant - 1];
    if (v.small) return g.splits > 1 ? hipErrorInvalidValue : launch_small(g, stream);
    const OperandLayout la = classify(g.m, g.k, g.a_rs, g.a_cs);
    const OperandLayout lb = classify(g.n, g.k, g.b_cs, g.b_rs);
    Params p;
    p.a = (const float *)g.a; p.b = (const float *)g.b; p.c = (float *)g.c; p.bias = (const float *)g.bias;
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
    p.c_vec = (g.n % 4 == 0) && (p.ldc % 4 == 0) && (((uintptr_t)g.c & 15u) == 0) &&
              (g.c_b1 % 4 == 0) && (g.c_b2 % 4 == 0) && (!g.bias || ((uintptr_t)g.bias & 15u) == 0);
    p.window = needs_window(g, la, lb);
    p.group_m = 4;
    const int total_iters = (int)(((g.k + v.bk - 1) / v.bk) * p.kbatches);
    p.splits = 1; p.chunk = total_iters; p.ws = nullptr; p.ws_ld = 0; p.ws_split_stride = 0;
    if (g.splits > 1) {
        if (!g.workspace || p.total_blocks != p.tiles_per_batch) return hipErrorInvalidValue;
        p.splits = g.splits;
        p.chunk = (total_iters + g.splits - 1) / g.splits;
        if ((int64_t)(g.splits - 1) * p.chunk >= total_iters) return hipErrorInvalidValue;
        p.ws = g.workspace;
        ws_layout32(g, variant, &p.ws_ld, &p.ws_split_stride);
        p.total_blocks = p.tiles_per_batch * g.splits;
    }
    hipError_t e = launch_tiles(p, variant, la.kc, lb.kc, stream);
    if (e != hipSuccess || g.splits <= 1) return e;
    return launch_splitk_reduce(g, p.ws_ld, p.ws_split_stride, stream);
}

static hipError_t launch_tiles(const Params &p, int variant, bool a_kc, bool b_kc, hipStream_t stream) {
    struct { bool kc; } la{a_kc}, lb{b_kc};
#define DFDX_TILE(BM, BN, WM, WN)                                                                    \
    return p.window ? launch_layout<BM, BN, 32, WM, WN, true>(p, la.kc, lb.kc, stream)               \
                    : launch_layout<BM, BN, 32, WM, WN, false>(p, la.kc, lb.kc, stream)
    switch (variant) {
    case 1: DFDX_TILE(256, 256, 2, 4);
    case 2: DFDX_TILE(256, 256, 2, 2);
    case 3: DFDX_TILE(256, 128, 2, 2);
    case 4: DFDX_TILE(128, 128, 2, 2);
    case 5: DFDX_TILE(128, 64, 4, 1);
    case 6: DFDX_TILE(64, 64, 2, 2);
    case 7: return launch_dma_layout<256, 256, 2, 4>(p, la.kc, lb.kc, stream);
    case 8: return launch_dma_layout<128, 128, 2, 2>(p, la.kc, lb.kc, stream);
    default: return hipErrorInvalidValue;
    }
#undef DFDX_TILE
}

}  // namespace dfdx_rocm
