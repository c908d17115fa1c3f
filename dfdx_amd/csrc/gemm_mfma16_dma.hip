// MFMA GEMM for 16-bit inputs (f16 / bf16), f32 accumulate, gfx950 (CDNA4): the fast path for
// K % 64 == 0.  v_mfma_f32_16x16x32_{f16,bf16}; BM x BN x 64 tile per workgroup of 8 waves.
//
// Data movement
//   * A and B tiles go from global memory straight into LDS with 16 B-per-lane LDS-DMA loads
//     (global_load_lds_dwordx4): no VGPR staging, no ds_write.  One wave instruction fills 1 KB of
//     LDS contiguously; WHICH 16 B chunk of the tile a lane fetches is chosen so that the tile lands
//     XOR-swizzled and every fragment read is bank-conflict free (measured: SQ_LDS_BANK_CONFLICT = 0).
//   * k-contiguous operand (A row-major, or B stored [N][K]): LDS holds [row][64 k], chunk c of row r at
//     position c ^ ((r >> 1) & 7); fragments are read with ds_read_b128.
//   * m/n-contiguous operand (A stored [K][M], or B row-major [K][N]): LDS holds [k][rows] exactly as in
//     memory (no transpose anywhere); fragments are read with the transposing ds_read_b64_tr_b16, two per
//     fragment.  Chunk c of k-row k sits at c ^ swz(k) (see mc_swizzle).
//   * Two LDS stages.  Tile t+1 is requested right after the barrier that retires tile t-1 and has one
//     full k step of MFMAs to arrive.
// Schedule per k step (32 wide, two per tile): the A fragments are single buffered in two halves, the B
// fragments double buffered; the reads for the next step are issued in the middle of the MFMAs of the
// current one, into registers that are already free, so each read has >= a quarter step of MFMAs to land.
// One s_barrier per tile.  Stage hand-over uses explicit s_waitcnt vmcnt/lgkmcnt + s_barrier.
//
// Rows/columns past the matrix edge are clamped onto valid addresses (they only feed C entries that are
// never stored).  There is no k tail here: K % 64 != 0 is served by the register-staged kernel.
#include "gemm_internal.h"
#include <algorithm>
#include <type_traits>

namespace dfdx_rocm {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define DFDX_LDS __attribute__((address_space(3)))
#define DFDX_GLB __attribute__((address_space(1)))

constexpr int BK = 64;
constexpr int STAGES = 2;

struct Params {
    const uint16_t *a;
    const uint16_t *b;
    uint16_t *c;
    const uint16_t *bias;
    int m, n, k;
    int lda, ldb;
    int64_t ldc;
    int64_t a_b1, a_b2, b_b1, b_b2, c_b1, c_b2;
    int nb2, kbatches;
    int tiles_m, tiles_n, tiles_per_batch, total_blocks;
    int accumulate, bias_mode;
    int group_m;
    // split-k: `splits` workgroups per C tile, each covering `chunk` k-loop steps, f32 partials in `ws`
    int splits, chunk;
    int grid;  // workgroups launched (<= total_blocks: each walks blockIdx.x, blockIdx.x + grid, ...)
    float *ws;
    int64_t ws_ld, ws_split_stride;
    // sums of A's rows over the contraction as a second result (KSUM instances, split-k only): f32 partial sums in
    // ws_ksum[(split * (BM / 64) + tile column) * 8 + wave][tiles_m * BM], combined by the reduce kernel
    float *ws_ksum;
    int ws_ksum_stride;
};

// A 16-byte store of C in the non-temporal form (`global_store_dwordx4 ... nt`): the lines are not kept in the caches on
// their way to memory.  For C that is written once and not read back by this launch.  Measured on MI355X against the
// cached form, over buffer sets that defeat the 256 MB last-level cache: 128 x (1024 x 64 x 1024), 268 MB of C, 71 -> 57 us
// (the output stops evicting the operand tiles); 8192 x 1024 x 1024 24.7 -> 18.8 us; 4096^3 109 -> 105 us; one encoder
// block, forward + backward, 1288 -> 1268 us.  Launch after launch on ONE buffer set whose output fits that cache the
// cached form is up to 6 % faster (256 x (512 x 64 x 512): 29.1 vs 30.9 us) -- a state no training step is in.
__device__ __forceinline__ void stream16(void *p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4 *)p); }

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // v_cvt_pk_f16_f32: RNE, lo in bits 15:0
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, h2));
    }
};
template <> struct Mma<__bf16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }  // RNE, quiet NaNs
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // v_cvt_pk_bf16_f32: RNE, quiet NaNs
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, b2));
    }
};

// DPP row rotation by 8 lanes: the lanes of the 4-lane banks selected by BANK_MASK (bit b = lanes 4b..4b+3 of every
// 16-lane row) receive `src` of the lane 8 places away in their row, the other lanes keep `keep`.
template <int BANK_MASK> __device__ __forceinline__ uint32_t lane8_trade(uint32_t keep, uint32_t src) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)src, 0x128 /* row_ror:8 */, 0xF, BANK_MASK, false);
}

// Swizzle of an m/n-contiguous tile ([k][ROWS] in LDS, ROWS*2 bytes per k-row): XOR applied to the 16 B
// chunk index of k-row k.  A 16-lane group of a transposing read touches 4 consecutive k-rows x 2 chunks,
// a second group the same chunks 8 k-rows further: the XOR spreads those over distinct banks.
template <int ROWS> __device__ __forceinline__ int mc_swizzle(int k) {
    if constexpr (ROWS >= 128) return (4 * (k & 3)) ^ (2 * ((k >> 3) & 1));
    else return (4 * ((k >> 1) & 1)) ^ (2 * ((k >> 3) & 1));  // ROWS == 64: bit 3 of the bank slot comes from k & 1
}

// One operand tile in LDS, filled by LDS-DMA loads (16 B per lane, 1 KB contiguous per wave instruction).
// PERM (k-contiguous B tiles of wave tiles that are at least 32 columns wide): the fragments of such a tile do not take
// 16 consecutive rows but the rows 8q + 4 * (fragment parity) + 0..3, q = 0..3, of a 32-row group (see the epilogue: a
// lane then owns 8 consecutive columns of C without any exchange between lanes).  The swizzle follows the lane that
// reads the row, (2 * (r / 8 % 4) + r % 4 / 2), so that the banks a fragment read touches are those of the plain order.
template <int ROWS, int NWAVES, bool KC, bool PERM = false> struct DmaTile {
    static constexpr int BYTES = ROWS * BK * 2;
    static constexpr int INSTRS = BYTES / 1024;
    static constexpr int IPW = INSTRS / NWAVES;
    static_assert(INSTRS % NWAVES == 0 && IPW >= 1, "tile does not divide over the waves");
    static constexpr int CPR = KC ? BK / 8 : ROWS / 8;  // 16 B chunks per LDS row
    // Byte offset from the tile origin in global memory, plus 1024 * (IPW - 1 - i): the wave's IPW instructions share
    // ONE LDS base, that of the last 1 KB piece (one M0 write instead of IPW), and reach their own piece through the
    // instruction offset -1024 * (IPW - 1 - i), which the hardware adds to the global address as well.
    static_assert((IPW - 1) * 1024 <= 4096, "instruction offsets are 13-bit signed");
    uint32_t goff[IPW];

    __device__ __forceinline__ void init(int ld, int rows_left, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < IPW; i++) {
            const int slot = (wave * IPW + i) * 64 + lane;  // 16 B slot index inside the tile
            const int r = slot / CPR, cp = slot % CPR;
            if constexpr (KC) {
                const int c = PERM ? cp ^ ((((r >> 3) & 3) << 1) | ((r >> 1) & 1)) : cp ^ ((r >> 1) & 7);
                goff[i] = (uint32_t)(min(r, rows_left - 1) * ld + c * 8) * 2u + (uint32_t)(1024 * (IPW - 1 - i));
            } else {
                const int c = cp ^ mc_swizzle<ROWS>(r);
                goff[i] = (uint32_t)(r * ld + min(c * 8, rows_left - 8)) * 2u + (uint32_t)(1024 * (IPW - 1 - i));
            }
        }
    }
    template <int I> __device__ __forceinline__ void issue_one(const char *origin, DFDX_LDS void *lds) const {
        if constexpr (I < IPW) {
            __builtin_amdgcn_global_load_lds((const DFDX_GLB void *)(origin + goff[I]), lds, 16, -1024 * (IPW - 1 - I), 0);
            issue_one<I + 1>(origin, lds);
        }
    }
    // LDS byte address of the wave's last 1 KB piece inside a tile that starts at byte `tile` of the LDS allocation
    static __device__ __forceinline__ uint32_t wave_base(uint32_t tile, int wave) { return tile + (uint32_t)(wave * IPW + IPW - 1) * 1024u; }
    // `lds_last`: wave_base of the destination tile, wave-uniform (a scalar register: it goes to M0 as it is)
    __device__ __forceinline__ void issue(const uint16_t *g, uint32_t lds_last) const {
        issue_one<0>((const char *)g, (DFDX_LDS void *)(uintptr_t)lds_last);
    }
};

// Waves per SIMD that the two LDS stages of a BM x BN x 64 tile let a CU hold (160 KB of LDS, 8-wave workgroups on 4
// SIMDs): the register budget the kernel is compiled for, so that a scalar-register spill into vector lanes cannot
// push the 128 x 128 tile past 128 VGPRs and halve its occupancy.
constexpr int dma_waves_per_simd(int bm, int bn, int waves) {
    const int wgs = 163840 / (2 * (bm + bn) * 64 * 2);
    const int w = (wgs < 1 ? 1 : wgs) * waves / 4;
    return w < 2 ? 2 : (w > 6 ? 6 : w);
}

// EDGE = false is the instance for problems made of whole tiles (no per-row bias, no bias together with beta = 1): its
// epilogue has only the two interior forms.  With the general form compiled in as well, the compiler guards the
// fragment registers against a load of that form it cannot prove complete, with a wait for ALL memory traffic in the
// middle of the k loop -- where every wave then stalls on the tile prefetched for the step after.
//
// KSUM = true (A stored [k][m] only, split-k only) adds a second result: the sums of A's rows over the contraction --
// the bias gradient of a Linear layer when A is grad_out^T and the product is the weight gradient.  The A tile sits in
// LDS as 64 k-rows of BM values; its column sums need no MFMA and no fragment: every thread reads ONE 16-byte piece
// (8 values of one k-row) per k tile and adds it to 8 f32 sums of its own.  The 512 threads cover 512 of the tile's
// 64 * BM / 8 pieces; the workgroups of a tile row all hold the same A tiles, so tile column q < BM / 64 takes the q-th
// 512 pieces and the others none.  At the end of a work item lanes that hold the same 8 columns are added up and each
// wave leaves its sums in a workspace slot of its own; the split-k reduce kernel adds the slots.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool EDGE, bool KSUM = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, dma_waves_per_simd(BM, BN, WAVES_M *WAVES_N)) void gemm_mfma16_dma_kernel(const Params p) {
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 16, TN = WTN / 16;
    static_assert(WTM % 64 == 0 && WTN % 16 == 0, "wave tile must be a multiple of 64 x 16");
    constexpr int Q = TM / 4;  // tile rows per quarter of a k step
    // B stored along k and a wave tile of whole fragment pairs: the rows (n) of B are dealt to the fragments so that the
    // two accumulators acc[i][2jp], acc[i][2jp + 1] of a lane hold 8 CONSECUTIVE columns of C, n = 32 jp + 8 lq + 0..7
    // (fragment 2jp + par, MFMA row 4 lq + v  <->  n = 32 jp + 8 lq + 4 par + v), instead of two runs of 4 that the lane
    // rows would have to trade.  Same products, same k order, same bits; the epilogue loses its cross-lane exchange.
    constexpr bool PERM = B_KC && TN % 2 == 0;
    using TA = DmaTile<BM, NW, A_KC>;
    using TB = DmaTile<BN, NW, B_KC, PERM>;
    constexpr int STAGE_BYTES = TA::BYTES + TB::BYTES;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = tid / 64;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    const int l16 = lane % 16, lq = lane / 16;

    // ---- work items ---------------------------------------------------------
    // A work item is one C tile (of one batch, or of one k split).  The workgroup is persistent: it walks the
    // work items blockIdx.x, blockIdx.x + gridDim.x, ... and keeps ONE load pipeline running across them, so
    // the stores of a finished tile overlap with the loads (already in flight) and MFMAs of the next one.
    struct Work {
        int batch, split, bm0, bn0, it0, iters;
    };
    const int ktiles = p.k / BK;
    auto decode = [&](int index) -> Work {
        Work w;
        const int work = xcd_remap(index, p.total_blocks);
        const int bidx = work / p.tiles_per_batch;  // batch, or k split
        const int tile = work % p.tiles_per_batch;
        const int gsize = p.group_m * p.tiles_n;
        const int group = tile / gsize;
        const int first_m = group * p.group_m;
        const int gm = min(p.tiles_m - first_m, p.group_m);
        w.bm0 = (first_m + (tile % gsize) % gm) * BM;
        w.bn0 = ((tile % gsize) / gm) * BN;
        w.split = p.splits > 1 ? bidx : 0;
        w.batch = p.splits > 1 ? 0 : bidx;
        // k-loop steps run over (batch, k-tile) pairs; with split-k this item owns steps [it0, it0 + iters)
        w.it0 = w.split * p.chunk;
        w.iters = min(ktiles * p.kbatches - w.it0, p.chunk);
        return w;
    };

    // ---- global side: the load pipeline ("fetch" state runs ahead of the compute state) ------------------
    const int64_t a_step = A_KC ? BK : (int64_t)BK * p.lda;
    const int64_t b_step = B_KC ? BK : (int64_t)BK * p.ldb;
    int f_index = blockIdx.x;   // work item whose tiles are being requested
    Work fw = decode(f_index);
    int f_left = 0, f_kb = 0, f_kt = 0, f_stage = 0;
    const uint16_t *a_next = nullptr, *b_next = nullptr;
    TA ta;
    TB tb;
    auto a_origin = [&](const Work &w, int kb) -> const uint16_t * {
        const uint16_t *base = p.a + (int64_t)(kb / p.nb2) * p.a_b1 + (int64_t)(kb % p.nb2) * p.a_b2;
        return A_KC ? base + (int64_t)w.bm0 * p.lda : base + w.bm0;
    };
    auto b_origin = [&](const Work &w, int kb) -> const uint16_t * {
        const uint16_t *base = p.b + (int64_t)(kb / p.nb2) * p.b_b1 + (int64_t)(kb % p.nb2) * p.b_b2;
        return B_KC ? base + (int64_t)w.bn0 * p.ldb : base + w.bn0;
    };
    auto begin_fetch = [&]() {  // position the pipeline on the first tile of work item fw
        f_left = fw.iters;
        f_kb = p.kbatches > 1 ? fw.it0 / ktiles : fw.batch;
        f_kt = p.kbatches > 1 ? fw.it0 % ktiles : fw.it0;
        a_next = a_origin(fw, f_kb) + f_kt * a_step;
        b_next = b_origin(fw, f_kb) + f_kt * b_step;
        // wave and lane as new values: the tile coordinates derived from them are needed once per work item only and
        // are recomputed here instead of being carried through the k loop
        int f_wave = wave, f_lane = lane;
        asm volatile("" : "+v"(f_wave), "+v"(f_lane));
        ta.init(p.lda, p.m - fw.bm0, f_wave, f_lane);
        tb.init(p.ldb, p.n - fw.bn0, f_wave, f_lane);
    };
    begin_fetch();
    bool fetching = true;
    const uint32_t smem_addr = (uint32_t)(uintptr_t)(DFDX_LDS const uint8_t *)smem;
    const uint32_t lds_last_a = __builtin_amdgcn_readfirstlane(TA::wave_base(smem_addr, wave));
    const uint32_t lds_last_b = __builtin_amdgcn_readfirstlane(TB::wave_base(smem_addr + TA::BYTES, wave));
    auto issue = [&]() {
        const uint32_t st = (uint32_t)f_stage * STAGE_BYTES;
        f_stage ^= 1;
        ta.issue(a_next, lds_last_a + st);
        tb.issue(b_next, lds_last_b + st);
        if (--f_left == 0) {  // next request belongs to the next work item (if any)
            f_index += gridDim.x;
            fetching = f_index < p.total_blocks;
            if (fetching) {
                fw = decode(f_index);
                begin_fetch();
            }
            return;
        }
        a_next += a_step;
        b_next += b_step;
        if (++f_kt == ktiles) {
            f_kt = 0;
            ++f_kb;
            a_next = a_origin(fw, f_kb);
            b_next = b_origin(fw, f_kb);
        }
    };

    // ---- LDS side: per-lane fragment addresses ------------------------------
    // k-contiguous: lane reads row w0 + 16*t + l16, logical chunk 4*ks + lq
    int a_off[2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        const int c = ks * 4 + lq;
        a_off[ks] = (wm0 + l16) * BK * 2 + ((c ^ ((l16 >> 1) & 7)) * 16);
        b_off[ks] = (wn0 + (PERM ? 8 * (l16 / 4) + l16 % 4 : l16)) * BK * 2 + ((c ^ ((l16 >> 1) & 7)) * 16);
    }
    // m/n-contiguous: lane 16*g + L supplies the address of X[k = 8*g + L/4 (+32*ks, +4)][col = w0 + 16*t + 4*(L%4)];
    // the transposing read hands lane L the 4 k-values of column w0 + 16*t + L.  k + 4 and k + 32 leave the
    // swizzle bits of k alone, so the four reads of one 16-column tile (two k steps x two halves) differ only by
    // immediate offsets from one per-lane address.
    //
    // These reads are issued from inline asm: the compiler puts a vmcnt(0) in front of every transposing-read
    // builtin while an LDS-DMA load is outstanding (it cannot see that the load targets the other stage), which
    // would make the prefetched tile arrive half a tile early.  The price is that the compiler does not track
    // their completion either: every consumer sits behind an explicit `fence` (see below).
    const int tr_k = lq * 8 + l16 / 4;
    const int tr_col = 4 * (l16 % 4);
    auto tr_base = [&](auto rows_tag, int col0) -> uint32_t {  // byte offset inside the operand tile, k step 0, low half
        constexpr int ROWS = decltype(rows_tag)::value;
        const int col = col0 + tr_col;
        const int c = col / 8, half = (col / 4) % 2;
        return (uint32_t)(tr_k * ROWS * 2 + ((c ^ mc_swizzle<ROWS>(tr_k)) * 16) + half * 8);
    };
    uint32_t a_tr[A_KC ? 1 : TM], b_tr[B_KC ? 1 : TN];
    if constexpr (!A_KC) {
#pragma unroll
        for (int i = 0; i < TM; i++) a_tr[i] = tr_base(std::integral_constant<int, BM>{}, wm0 + i * 16);
    }
    if constexpr (!B_KC) {
#pragma unroll
        for (int j = 0; j < TN; j++) b_tr[j] = TA::BYTES + tr_base(std::integral_constant<int, BN>{}, wn0 + j * 16);
    }
    auto lds_addr = [](const uint8_t *p) -> uint32_t { return (uint32_t)(uintptr_t)(DFDX_LDS const uint8_t *)p; };
    auto tr_frag = [&](uint32_t addr, auto rows_tag, auto ks_tag) -> u32x4 {
        constexpr int OFF = decltype(ks_tag)::value * 32 * decltype(rows_tag)::value * 2;
        constexpr int HI = 4 * decltype(rows_tag)::value * 2;
        u32x2 l, h;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(l) : "v"(addr), "i"(OFF));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(h) : "v"(addr), "i"(OFF + HI));
        return u32x4{l[0], l[1], h[0], h[1]};
    };
    // `fence<N>(x...)`: at most N LDS operations issued by this wave may still be outstanding (they complete in
    // order); the fragments passed in are re-defined by the asm so that nothing that uses them can move above it.
    auto tie = [](u32x4 &x) { asm volatile("" : "+v"(x)); };
    constexpr int OPS_A = A_KC ? 1 : 2, OPS_B = B_KC ? 1 : 2;  // LDS instructions per fragment

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc[i][j][v] = 0.0f;

    u32x4 fa[TM], fb[2][TN];
    // KSUM: the thread's piece of every A tile is chunk ks_chunk = tid % CH (8 columns) of one k-row, at byte ks_off of
    // the tile (the swizzle depends on the k-row only, so the same place in every tile).
    constexpr int CH = BM / 8, KS_SHARE = BM / 64;  // pieces per k-row; tile columns that share a tile's pieces
    static_assert(!KSUM || (!A_KC && NW == 8 && (CH == 32 || CH == 16)), "row sums: [k][m] tiles of 8-wave workgroups");
    [[maybe_unused]] float ks_sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    [[maybe_unused]] u32x4 ks_piece;
    [[maybe_unused]] uint32_t ks_off = 0;
    [[maybe_unused]] int ks_chunk = 0;
    [[maybe_unused]] bool ks_on = false;
    [[maybe_unused]] auto ks_begin = [&](int bn0) {
        const int tn = bn0 / BN;
        ks_on = tn < KS_SHARE;
        const int cell = (ks_on ? tn : 0) * 512 + tid;
        const int krow = cell / CH;
        ks_chunk = cell % CH;  // lanes CH apart hold the same chunk of neighbouring k-rows
        ks_off = (uint32_t)(krow * BM * 2 + (ks_chunk ^ mc_swizzle<BM>(krow)) * 16);
    };
    [[maybe_unused]] auto ks_read = [&](const uint8_t *sa) {  // asm: see the note on the transposing reads above
        if constexpr (KSUM) asm volatile("ds_read_b128 %0, %1" : "=v"(ks_piece) : "v"(lds_addr(sa) + ks_off));
    };
    [[maybe_unused]] auto ks_add = [&]() {  // after a wait for every LDS read of the wave
        if constexpr (KSUM) {
            tie(ks_piece);
            if (ks_on) {
#pragma unroll
                for (int e = 0; e < 8; e++) ks_sum[e] += Mma<T>::to_f32((uint16_t)(ks_piece[e / 2] >> ((e & 1) * 16)));
            }
        }
    };
    auto read_a = [&](const uint8_t *sa, auto ks_tag, int i0, int i1) {
        constexpr int ks = decltype(ks_tag)::value;
        [[maybe_unused]] const uint32_t base = lds_addr(sa);
#pragma unroll
        for (int i = 0; i < TM; i++)
            if (i >= i0 && i < i1) {
                if constexpr (A_KC) fa[i] = *(const u32x4 *)(sa + a_off[ks] + i * 16 * BK * 2);
                else fa[i] = tr_frag(base + a_tr[i], std::integral_constant<int, BM>{}, ks_tag);
            }
    };
    auto read_b = [&](const uint8_t *sa, auto ks_tag, u32x4(&bf)[TN]) {
        constexpr int ks = decltype(ks_tag)::value;
        const uint8_t *sb = sa + TA::BYTES;
        [[maybe_unused]] const uint32_t base = lds_addr(sa);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (B_KC) bf[j] = *(const u32x4 *)(sb + b_off[ks] + (PERM ? (j / 2) * 32 + (j % 2) * 4 : j * 16) * BK * 2);
            else bf[j] = tr_frag(base + b_tr[j], std::integral_constant<int, BN>{}, ks_tag);
        }
    };
    // Completion of the asm-issued (transposing) reads.  `left` = LDS instructions issued after the youngest one
    // that must be complete; the hardware counter saturates the wait at 15.
    auto fence_a = [&](auto left_tag, int i0, int i1) {
        if constexpr (!A_KC) {
            constexpr int LEFT = decltype(left_tag)::value > 15 ? 15 : decltype(left_tag)::value;
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"i"(LEFT));
#pragma unroll
            for (int i = 0; i < TM; i++)
                if (i >= i0 && i < i1) tie(fa[i]);
        }
    };
    auto fence_b = [&](auto left_tag, u32x4(&bf)[TN]) {
        if constexpr (!B_KC) {
            constexpr int LEFT = decltype(left_tag)::value > 15 ? 15 : decltype(left_tag)::value;
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"i"(LEFT));
#pragma unroll
            for (int j = 0; j < TN; j++) tie(bf[j]);
        }
    };
    // swapped operands: the lane ends up with m = l16 and 4 consecutive n = 4*lq + 0..3 per 16x16 tile
    auto mma = [&](const u32x4(&bf)[TN], int i0, int i1) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
            for (int i = 0; i < TM; i++)
                if (i >= i0 && i < i1) acc[i][j] = Mma<T>::mfma(bf[j], fa[i], acc[i][j]);
        }
    };
    // Make the oldest requested tile visible to every wave, then request the next one into the stage that the
    // previously computed tile occupied.  Callers guarantee that this wave has issued all its LDS reads of
    // that previous tile; lgkmcnt(0) makes sure they are done.  (vmcnt(0) also covers the stores of a finished
    // C tile: they had a whole k step to drain.)
    // `behind`: how many memory instructions this wave issued AFTER its last tile request -- the stores of the C tile
    // finished before this one (one of the compile-time counts below, else 0).  The counter retires in issue order, so
    // waiting until that many are left means: the requested tile has landed, the stores may still be draining.  With
    // one k tile per work item (attention scores) a wait for everything would stop every workgroup until its previous
    // C tile is in memory, and the chip would alternate between storing and computing.
    constexpr int ST_PLAIN = TM * TN / 2, ST_ACC = (TM * (TN / 2) > 8 ? TM / 2 : TM) * TN / 2, ST_SPLIT = TM * TN;
    static_assert(ST_SPLIT < 64, "vmcnt is a 6-bit count");
    constexpr auto wait_vm_lgkm0 = [](int vm) { return (vm & 15) | ((vm >> 4) << 14) | 0x0070; };  // vmcnt(vm) & lgkmcnt(0)
    auto sync_tile = [&](int behind = 0) {
        if (behind == ST_PLAIN) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(ST_PLAIN));
        else if (behind == ST_ACC) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(ST_ACC));
        else if (behind == ST_SPLIT) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(ST_SPLIT));
        else __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) & lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (fetching) issue();
    };

    // one 64-wide k tile from stage `cs`; HAS_NEXT: the next tile belongs to the same work item (hand the stage
    // over and prefetch its first fragments while the last MFMAs of this tile run)
    // LDS instructions per group of reads, as issued below: half of the A fragments, all B fragments of a k step
    constexpr int RA = 2 * Q * OPS_A, RB = TN * OPS_B, KS_READS = KSUM ? 1 : 0;
    constexpr std::integral_constant<int, 0> K0{};
    constexpr std::integral_constant<int, 1> K1{};
#define DFDX_LEFT(n) std::integral_constant<int, (n)> {}
    // First fragments of a tile, in the order the fences of tile_body assume: A rows [0, 2Q), B, A rows [2Q, TM).
    auto read_first = [&](const uint8_t *st) {
        read_a(st, K0, 0, 2 * Q);
        read_b(st, K0, fb[0]);
        read_a(st, K0, 2 * Q, TM);
    };
    auto tile_body = [&](int cs, auto has_next_tag) {
        constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
        const uint8_t *sa = smem + cs * STAGE_BYTES;
        const uint8_t *sn = smem + (cs ^ 1) * STAGE_BYTES;
        // ---- k step 0 (B buffer 0); prefetch k step 1 of this tile.  Outstanding on entry, oldest first:
        //      A[0,2Q), B, A[2Q,TM) of this k step.
        fence_b(DFDX_LEFT(RA), fb[0]);
        fence_a(DFDX_LEFT(RA / 2 + RB + RA), 0, Q);
        mma(fb[0], 0, Q);
        __builtin_amdgcn_sched_barrier(0);
        fence_a(DFDX_LEFT(RB + RA), Q, 2 * Q);
        mma(fb[0], Q, 2 * Q);
        __builtin_amdgcn_sched_barrier(0);
        fence_a(DFDX_LEFT(RA / 2), 2 * Q, 3 * Q);
        mma(fb[0], 2 * Q, 3 * Q);
        __builtin_amdgcn_sched_barrier(0);
        read_a(sa, K1, 0, 2 * Q);
        read_b(sa, K1, fb[1]);
        __builtin_amdgcn_sched_barrier(0);
        fence_a(DFDX_LEFT(RA + RB), 3 * Q, TM);
        mma(fb[0], 3 * Q, TM);
        __builtin_amdgcn_sched_barrier(0);
        // ---- k step 1 (B buffer 1); prefetch k step 0 of the next tile
        fence_b(DFDX_LEFT(0), fb[1]);
        fence_a(DFDX_LEFT(RA / 2 + RB), 0, Q);
        mma(fb[1], 0, Q);
        __builtin_amdgcn_sched_barrier(0);
        read_a(sa, K1, 2 * Q, TM);
        ks_read(sa);  // KSUM: the last (youngest) LDS read of this tile, consumed behind a wait for all of them
        __builtin_amdgcn_sched_barrier(0);
        fence_a(DFDX_LEFT(RB + RA + KS_READS), Q, 2 * Q);
        mma(fb[1], Q, 2 * Q);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (HAS_NEXT) {
            // Every LDS read of this tile has been issued: wait for them and hand the stage over TWO MFMA groups before
            // the end of the tile, so that the requests for the tile after next and the first fragment reads of the
            // next one are issued under MFMAs instead of in front of an idle matrix core.  The two waves that share a
            // SIMD (w and w + NW/2) take opposite orders: one issues its MFMA group while the other issues requests.
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) & lgkmcnt(0)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            fence_a(DFDX_LEFT(0), 2 * Q, TM);
            ks_add();
            const bool mfma_first = __builtin_amdgcn_readfirstlane(wave) >= NW / 2;
            if (mfma_first) {
                mma(fb[1], 2 * Q, 3 * Q);
                mma(fb[1], 3 * Q, TM);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (fetching) issue();
            __builtin_amdgcn_sched_barrier(0);
            read_a(sn, K0, 0, 2 * Q);
            read_b(sn, K0, fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            if (!mfma_first) {
                mma(fb[1], 2 * Q, 3 * Q);
                mma(fb[1], 3 * Q, TM);
            }
            __builtin_amdgcn_sched_barrier(0);
            read_a(sn, K0, 2 * Q, TM);
        } else {
            fence_a(DFDX_LEFT(RA / 2 + KS_READS), 2 * Q, 3 * Q);
            mma(fb[1], 2 * Q, 3 * Q);
            __builtin_amdgcn_sched_barrier(0);
            fence_a(DFDX_LEFT(0), 3 * Q, TM);
            mma(fb[1], 3 * Q, TM);
            ks_add();
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- epilogue of one work item: lane holds m = l16 (per tile), n = 4*lq + 0..3 -------------
    // Returns the number of stores it issued after its last load (see sync_tile), 0 when that is not a fixed count.
    auto store_tile = [&](const Work &w) -> int {
        const int bm0 = w.bm0, bn0 = w.bn0, split = w.split, batch = w.batch;
        if constexpr (KSUM) {
            // Lanes that hold the same 8 columns (they differ in the k-row) are added up; the first CH lanes of each wave
            // store.  These stores come before the C tile's: the count returned below stays a lower bound of what was
            // issued after the last load.
            if (ks_on) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
#pragma unroll
                    for (int d = CH; d < 64; d *= 2) ks_sum[e] += __shfl_xor(ks_sum[e], d, 64);
                }
                if (lane < CH) {
                    float *slot = p.ws_ksum + (int64_t)((split * KS_SHARE + bn0 / BN) * 8 + wave) * p.ws_ksum_stride + bm0 + ks_chunk * 8;
                    *(f32x4 *)slot = f32x4{ks_sum[0], ks_sum[1], ks_sum[2], ks_sum[3]};  // rows padded to whole tiles
                    *(f32x4 *)(slot + 4) = f32x4{ks_sum[4], ks_sum[5], ks_sum[6], ks_sum[7]};
                }
#pragma unroll
                for (int e = 0; e < 8; e++) ks_sum[e] = 0.0f;
            }
        }
    if (p.splits > 1) {  // f32 partial tile into the workspace (padded to whole tiles: no bounds checks)
        float *wbase = p.ws + split * p.ws_split_stride;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            float *wrow = wbase + (int64_t)(bm0 + wm0 + i * 16 + l16) * p.ws_ld + bn0 + wn0 + lq * (PERM ? 8 : 4);
#pragma unroll
            for (int j = 0; j < TN; j++) *(f32x4 *)(wrow + (PERM ? (j / 2) * 32 + (j % 2) * 4 : j * 16)) = acc[i][j];
        }
        return ST_SPLIT;
    }
    const int cb = p.kbatches > 1 ? 0 : batch;
    uint16_t *cbase = p.c + (int64_t)(cb / p.nb2) * p.c_b1 + (int64_t)(cb % p.nb2) * p.c_b2;
    if constexpr (TN % 2 == 0) {
        // 16 B per lane: two neighbouring 16x16 tiles exchange halves between the lane rows (16-lane groups) so
        // that a lane ends up with 8 consecutive columns of one of them.  v_permlane16_swap(x, y) trades lane
        // rows 1 and 3 of x against lane rows 0 and 2 of y: afterwards lane row lq holds, in (x, y), columns
        // 8*(lq/2) .. +3 and +4 .. +7 of tile j + (lq & 1).  A wave instruction then writes 64 contiguous
        // bytes per matrix row instead of 32, which is what the memory system needs to reach its write rate.
        {
            // The general form: bounds checks, either bias, beta = 1 with the old value loaded where it is used (edge
            // tiles, per-row bias, very large ldc).
            auto rows = [&]() {
                u32x4 cbias[TN / 2];
                float rbias_all[TM];
                if (p.bias_mode == BIAS_PER_COL) {
#pragma unroll
                    for (int jp = 0; jp < TN / 2; jp++)
                        cbias[jp] = *(const u32x4 *)(p.bias + min(bn0 + wn0 + (PERM ? jp * 32 + lq * 8 : (2 * jp + (lq & 1)) * 16 + (lq >> 1) * 8), p.n - 8));
                }
                if (p.bias_mode == BIAS_PER_ROW) {
#pragma unroll
                    for (int i = 0; i < TM; i++) rbias_all[i] = Mma<T>::to_f32(p.bias[min(bm0 + wm0 + i * 16 + l16, p.m - 1)]);
                }
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    const int gm_row = bm0 + wm0 + i * 16 + l16;
                    const bool row_ok = gm_row < p.m;
                    uint16_t *crow = cbase + (int64_t)gm_row * p.ldc;
#pragma unroll
                    for (int jp = 0; jp < TN / 2; jp++) {
                        float v[8];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            if constexpr (PERM) {
                                v[e] = acc[i][2 * jp][e];
                                v[4 + e] = acc[i][2 * jp + 1][e];
                            } else {
                                const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(acc[i][2 * jp][e]),
                                                                                __float_as_uint(acc[i][2 * jp + 1][e]), false, false);
                                v[e] = __uint_as_float(r[0]);
                                v[4 + e] = __uint_as_float(r[1]);
                            }
                        }
                        const int gn = bn0 + wn0 + (PERM ? jp * 32 + lq * 8 : (2 * jp + (lq & 1)) * 16 + (lq >> 1) * 8);
                        if (!row_ok || gn >= p.n) continue;  // n % 8 == 0 here: all 8 columns are in range
                        if (p.bias_mode == BIAS_PER_ROW) {
#pragma unroll
                            for (int e = 0; e < 8; e++) v[e] += rbias_all[i];
                        }
                        if (p.bias_mode == BIAS_PER_COL) {
                            const u32x4 bv = cbias[jp];
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                v[2 * e] += Mma<T>::to_f32((uint16_t)(bv[e] & 0xffffu));
                                v[2 * e + 1] += Mma<T>::to_f32((uint16_t)(bv[e] >> 16));
                            }
                        }
                        if (p.accumulate) {
                            const u32x4 old = *(const u32x4 *)(crow + gn);
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                v[2 * e] += Mma<T>::to_f32((uint16_t)(old[e] & 0xffffu));
                                v[2 * e + 1] += Mma<T>::to_f32((uint16_t)(old[e] >> 16));
                            }
                        }
                        u32x4 o;
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = Mma<T>::pack2(v[2 * e], v[2 * e + 1]);
                        *(u32x4 *)(crow + gn) = o;
                    }
                }
            };
            // Interior tiles address C as wave-uniform base (scalar registers) + one 32-bit per-lane byte offset
            // + immediate: no address arithmetic in vector registers per access.
            const int wave_u = __builtin_amdgcn_readfirstlane(wave);
            char *const tile_base = (char *)(cbase + (int64_t)(bm0 + (wave_u / WAVES_N) * WTM) * p.ldc + bn0 + (wave_u % WAVES_N) * WTN);
            const uint32_t lane_off = (uint32_t)(l16 * (int)p.ldc + (PERM ? lq * 8 : (lq & 1) * 16 + (lq >> 1) * 8)) * 2u;
            const int64_t row_step = p.ldc * 32;  // 16 rows, bytes
            // A wave tile that is 64 columns wide (TN == 4) writes whole 128 B lines: after the 16-lane swaps a lane
            // row holds the left 64 B of matrix row l16 in one register set and the right 64 B in another; lanes
            // l16 < 8 and l16 >= 8 then trade one set each (DPP row rotation by 8), so that one store instruction
            // covers rows 0..7 x 128 B and a second one rows 8..15.  Measured on the device with plain store kernels,
            // a CU retires 134 GB/s of whole-line stores but only 38 GB/s when every line arrives as two 64 B
            // halves from different instructions (and 19 GB/s in 32 B pieces); with half lines the stores of a
            // K = 64 work item take longer to leave the CU than its MFMAs take to compute.
            [[maybe_unused]] const uint32_t line_off =
                (uint32_t)((l16 & 7) * (int)p.ldc * 2 + (l16 >> 3) * 64 + (PERM ? lq : (lq & 1) * 2 + (lq >> 1)) * 16);
            [[maybe_unused]] const int64_t half_step = p.ldc * 16;  // 8 rows, bytes
            // Pure overwrite of an interior tile, optionally with a per-column bias (every forward product of whole
            // tiles, Linear's fused bias included): no bounds checks, no read of C; the bias values are fetched and
            // widened once, before the first store.
            auto rows_plain = [&](auto bias_tag) {
                constexpr bool BIAS = decltype(bias_tag)::value;
                // Rounded to the 16-bit type first, the lane rows then trade PACKED pairs: half as many cross-lane
                // instructions as trading the f32 values (the conversions and trades of a K = 64 work item cost
                // the vector ALU more cycles than its MFMAs cost the matrix core).
                [[maybe_unused]] float cb[TN][4];  // bias of the columns the lane holds before the trade
                if constexpr (BIAS) {
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const u32x2 bv = *(const u32x2 *)(p.bias + bn0 + wn0 + (PERM ? (j / 2) * 32 + lq * 8 + (j % 2) * 4 : j * 16 + lq * 4));
                        cb[j][0] = Mma<T>::to_f32((uint16_t)(bv[0] & 0xffffu));
                        cb[j][1] = Mma<T>::to_f32((uint16_t)(bv[0] >> 16));
                        cb[j][2] = Mma<T>::to_f32((uint16_t)(bv[1] & 0xffffu));
                        cb[j][3] = Mma<T>::to_f32((uint16_t)(bv[1] >> 16));
                    }
                }
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    u32x4 o[TN / 2];
#pragma unroll
                    for (int jp = 0; jp < TN / 2; jp++) {
                        uint32_t pk[2][2];  // [tile 2jp / 2jp + 1][columns 4*lq + 0,1 / 2,3]
#pragma unroll
                        for (int t = 0; t < 2; t++)
#pragma unroll
                            for (int h = 0; h < 2; h++) {
                                float x = acc[i][2 * jp + t][2 * h], y = acc[i][2 * jp + t][2 * h + 1];
                                if constexpr (BIAS) {
                                    x += cb[2 * jp + t][2 * h];
                                    y += cb[2 * jp + t][2 * h + 1];
                                }
                                pk[t][h] = Mma<T>::pack2(x, y);
                            }
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            if constexpr (PERM) {  // the lane's own 8 consecutive columns, 32 jp + 8 lq + 0..7
                                o[jp][h] = pk[0][h];
                                o[jp][2 + h] = pk[1][h];
                            } else {
                                const auto r = __builtin_amdgcn_permlane16_swap(pk[0][h], pk[1][h], false, false);
                                o[jp][h] = r[0];      // columns 8*(lq/2) + 2h, + 1 of tile 2jp + (lq & 1)
                                o[jp][2 + h] = r[1];  // columns 8*(lq/2) + 4 + 2h, + 1
                            }
                        }
                    }
                    if constexpr (TN == 4) {
                        u32x4 lo, hi;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            hi[e] = lane8_trade<0x3>(o[1][e], o[0][e]);  // rows 8..15: left halves come from lanes + 8
                            lo[e] = lane8_trade<0xC>(o[0][e], o[1][e]);  // rows 0..7: right halves come from lanes - 8
                        }
                        stream16(tile_base + i * row_step + line_off, lo);
                        stream16(tile_base + i * row_step + half_step + line_off, hi);
                    } else {
#pragma unroll
                        for (int jp = 0; jp < TN / 2; jp++) stream16(tile_base + i * row_step + jp * 64 + lane_off, o[jp]);
                    }
                }
            };
            // beta = 1 on an interior tile without bias (every gradient product of whole tiles): all old values are
            // requested before the first store goes out.  The memory counter retires in issue order, so waiting for a
            // load also waits for every store issued before it: the interleaved form of `rows` drains the stores of
            // the tile sixteen times; here the loads overlap each other and are waited for in issue order.
            auto rows_accumulate = [&]() {
                constexpr int IG = TM * (TN / 2) > 8 ? TM / 2 : TM;  // tile rows per batch: at most 8 vectors in flight
                char *const base = tile_base;
#pragma unroll
                for (int i0 = 0; i0 < TM; i0 += IG) {
                    u32x4 old[IG][TN / 2];
#pragma unroll
                    for (int i = 0; i < IG; i++)
#pragma unroll
                        for (int jp = 0; jp < TN / 2; jp++) {
                            if constexpr (TN == 4) old[i][jp] = *(const u32x4 *)(base + (i0 + i) * row_step + jp * half_step + line_off);
                            else old[i][jp] = *(const u32x4 *)(base + (i0 + i) * row_step + jp * 64 + lane_off);
                        }
#pragma unroll
                    for (int i = 0; i < IG; i++) {
                        float v[TN / 2][8];
#pragma unroll
                        for (int jp = 0; jp < TN / 2; jp++)
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                if constexpr (PERM) {
                                    v[jp][e] = acc[i0 + i][2 * jp][e];
                                    v[jp][4 + e] = acc[i0 + i][2 * jp + 1][e];
                                } else {
                                    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(acc[i0 + i][2 * jp][e]),
                                                                                    __float_as_uint(acc[i0 + i][2 * jp + 1][e]), false, false);
                                    v[jp][e] = __uint_as_float(r[0]);
                                    v[jp][4 + e] = __uint_as_float(r[1]);
                                }
                            }
                        if constexpr (TN == 4) {  // whole lines: v[0] becomes rows 0..7, v[1] rows 8..15 (see line_off)
#pragma unroll
                            for (int e = 0; e < 8; e++) {
                                const uint32_t left = __float_as_uint(v[0][e]), right = __float_as_uint(v[1][e]);
                                v[1][e] = __uint_as_float(lane8_trade<0x3>(right, left));
                                v[0][e] = __uint_as_float(lane8_trade<0xC>(left, right));
                            }
                        }
#pragma unroll
                        for (int jp = 0; jp < TN / 2; jp++) {
                            u32x4 o;
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                o[e] = Mma<T>::pack2(v[jp][2 * e] + Mma<T>::to_f32((uint16_t)(old[i][jp][e] & 0xffffu)),
                                                     v[jp][2 * e + 1] + Mma<T>::to_f32((uint16_t)(old[i][jp][e] >> 16)));
                            if constexpr (TN == 4) *(u32x4 *)(base + (i0 + i) * row_step + jp * half_step + line_off) = o;
                            else *(u32x4 *)(base + (i0 + i) * row_step + jp * 64 + lane_off) = o;
                        }
                    }
                }
            };
            // Every form ends by telling the compiler, with a wait that costs nothing, that the loads it issued are
            // complete: "at most as many memory instructions outstanding as the stores issued after the last load" (the
            // counter retires in issue order, and every loaded value has been consumed by then).  The general form
            // cannot count its stores and waits for them (edge tiles).
            constexpr auto vmcnt_only = [](int vm) { return (vm & 15) | ((vm >> 4) << 14) | 0x0F70; };
            const bool interior = !EDGE || (bm0 + BM <= p.m && bn0 + BN <= p.n && p.bias_mode != BIAS_PER_ROW && p.ldc < (1 << 26));
            if (interior && !p.accumulate) {
                if (p.bias_mode == BIAS_PER_COL) rows_plain(std::true_type{});
                else rows_plain(std::false_type{});
                __builtin_amdgcn_s_waitcnt(vmcnt_only(ST_PLAIN));
                return ST_PLAIN;
            } else if (!EDGE || (interior && p.bias_mode == BIAS_NONE)) {
                rows_accumulate();
                __builtin_amdgcn_s_waitcnt(vmcnt_only(ST_ACC));
                return ST_ACC;
            } else if constexpr (EDGE) {
                rows();
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
            }
            return 0;
        }
    }
    if constexpr (TN % 2 != 0) {  // a single 16-column tile per wave: 8 B per lane (the host guarantees n % 4 == 0 etc.)
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int gm_row = bm0 + wm0 + i * 16 + l16;
            if (gm_row >= p.m) continue;
            uint16_t *crow = cbase + (int64_t)gm_row * p.ldc;
            const float rbias = (p.bias_mode == BIAS_PER_ROW) ? Mma<T>::to_f32(p.bias[gm_row]) : 0.0f;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int gn = bn0 + wn0 + j * 16 + lq * 4;
                if (gn >= p.n) continue;  // n % 4 == 0: the 4 columns are all in range
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[i][j][e] + rbias;
                if (p.bias_mode == BIAS_PER_COL) {
                    const u32x2 bv = *(const u32x2 *)(p.bias + gn);
                    v[0] += Mma<T>::to_f32((uint16_t)(bv[0] & 0xffffu));
                    v[1] += Mma<T>::to_f32((uint16_t)(bv[0] >> 16));
                    v[2] += Mma<T>::to_f32((uint16_t)(bv[1] & 0xffffu));
                    v[3] += Mma<T>::to_f32((uint16_t)(bv[1] >> 16));
                }
                if (p.accumulate) {
                    const u32x2 old = *(const u32x2 *)(crow + gn);
                    v[0] += Mma<T>::to_f32((uint16_t)(old[0] & 0xffffu));
                    v[1] += Mma<T>::to_f32((uint16_t)(old[0] >> 16));
                    v[2] += Mma<T>::to_f32((uint16_t)(old[1] & 0xffffu));
                    v[3] += Mma<T>::to_f32((uint16_t)(old[1] >> 16));
                }
                *(u32x2 *)(crow + gn) = u32x2{Mma<T>::pack2(v[0], v[1]), Mma<T>::pack2(v[2], v[3])};
            }
        }
    }
    return 0;
    };

    // ---- compute state ---------------------------------------------------------------------------------------
    int c_index = blockIdx.x;
    Work cw = decode(c_index);
    int c_left = cw.iters, c_stage = 0;
    int behind = 0;  // stores of the previous work item that may still be in flight
    if constexpr (KSUM) ks_begin(cw.bn0);
    issue();
    sync_tile();
    read_first(smem);
    for (;;) {
        for (; c_left > 1; --c_left) {
            tile_body(c_stage, std::true_type{});  // waits for everything outstanding and requests a tile
            behind = 0;
            c_stage ^= 1;
        }
        tile_body(c_stage, std::false_type{});
        c_stage ^= 1;
        // Work item finished.  Hand the stage over BEFORE the stores are issued: the wait inside sync_tile then
        // covers the next tile's loads and the stores of the PREVIOUS item only, and this item's stores drain while
        // the next tile is computed.  (Converting the accumulators before that wait was tried: it costs registers
        // inside the k loop and lost.)
        const bool more = c_index + (int)gridDim.x < p.total_blocks;
        if (more) sync_tile(behind);
        behind = __builtin_amdgcn_readfirstlane(store_tile(cw));
        if (!more) break;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[i][j][v] = 0.0f;
        c_index += gridDim.x;
        cw = decode(c_index);
        c_left = cw.iters;
        if constexpr (KSUM) ks_begin(cw.bn0);
        read_first(smem + c_stage * STAGE_BYTES);
    }
}


#undef DFDX_LEFT

// ------------------------------------------------------------------ host side --

struct Variant {
    const char *name;
    int bm, bn, waves_m, waves_n;
};

// X(id, BM, BN, WAVES_M, WAVES_N); ids are 1-based inside this family.
#define DFDX_MFMA16_DMA_VARIANTS(X) \
    X(1, 256, 256, 2, 4)            \
    X(2, 256, 128, 4, 2)            \
    X(3, 128, 128, 2, 4)            \
    X(4, 256, 64, 4, 2)             \
    X(5, 128, 64, 2, 4)

constexpr Variant kVariants[] = {
#define X(id, bm, bn, wm, wn) {"dma_" #bm "x" #bn "x64_w" #wm "x" #wn, bm, bn, wm, wn},
    DFDX_MFMA16_DMA_VARIANTS(X)
#undef X
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

// Persistent launch: as many workgroups as the chip holds at once (what LDS and registers allow per compute
// unit, rounded to a multiple of the 8 XCDs so that work item i and i + grid land on the same XCD), or one per
// work item when there are fewer.
template <typename T, int BM, int BN, int WM, int WN>
hipError_t launch_layout(Params p, int compute_units, bool a_kc, bool b_kc, hipStream_t stream) {
    constexpr int NT = WM * WN * 64;
    constexpr size_t lds = (size_t)STAGES * (BM + BN) * BK * 2;
#define DFDX_LAUNCH(AKC, BKC, EDGE, ...)                                                                       \
    do {                                                                                                       \
        auto kern = gemm_mfma16_dma_kernel<T, BM, BN, WM, WN, AKC, BKC, EDGE, ##__VA_ARGS__>;                  \
        static PerDevice occupancy_on;                                                                         \
        std::atomic<int> &known = occupancy_on.here();                                                         \
        int per_cu = known.load(std::memory_order_acquire);                                                    \
        if (per_cu == 0) {                                                                                     \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                               (int)lds);                                                      \
            if (e != hipSuccess) return e;                                                                     \
            int occ = 0;                                                                                       \
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void *)kern, NT, lds);               \
            if (e != hipSuccess) return e;                                                                     \
            per_cu = occ < 1 ? 1 : occ;                                                                        \
            known.store(per_cu, std::memory_order_release);                                                    \
        }                                                                                                      \
        const int resident = (compute_units < 8 ? 8 : compute_units) * per_cu / 8 * 8;                         \
        p.grid = p.total_blocks <= resident ? p.total_blocks : resident;                                       \
        kern<<<dim3((unsigned)p.grid), dim3(NT), lds, stream>>>(p);                                            \
    } while (0)
    // whole tiles only, and nothing but the two interior epilogue forms: the instance without the general form
    const bool edge = p.m % BM != 0 || p.n % BN != 0 || p.bias_mode == BIAS_PER_ROW || p.ldc >= (1 << 26) ||
                      (p.accumulate && p.bias_mode != BIAS_NONE);
    if (p.ws_ksum) {  // row sums of A: compiled for the layout of weight gradients only (ksum_supported)
        if (a_kc || b_kc) return hipErrorInvalidValue;
        if (edge) DFDX_LAUNCH(false, false, true, true);
        else DFDX_LAUNCH(false, false, false, true);
    } else if (edge) {
        if (a_kc && b_kc) DFDX_LAUNCH(true, true, true);
        else if (a_kc && !b_kc) DFDX_LAUNCH(true, false, true);
        else if (!a_kc && b_kc) DFDX_LAUNCH(false, true, true);
        else DFDX_LAUNCH(false, false, true);
    } else {
        if (a_kc && b_kc) DFDX_LAUNCH(true, true, false);
        else if (a_kc && !b_kc) DFDX_LAUNCH(true, false, false);
        else if (!a_kc && b_kc) DFDX_LAUNCH(false, true, false);
        else DFDX_LAUNCH(false, false, false);
    }
#undef DFDX_LAUNCH
    return hipGetLastError();
}

template <typename T>
hipError_t launch_variant(int variant, const Params &p, int compute_units, bool a_kc, bool b_kc, hipStream_t s) {
    switch (variant) {
#define X(id, bm, bn, wm, wn) \
    case id: return launch_layout<T, bm, bn, wm, wn>(p, compute_units, a_kc, b_kc, s);
        DFDX_MFMA16_DMA_VARIANTS(X)
#undef X
    default: return hipErrorInvalidValue;
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

struct OperandLayout {
    bool ok, kc;
    int64_t ld;
};
inline OperandLayout classify(int64_t rows, int64_t kdim, int64_t row_stride, int64_t k_stride) {
    OperandLayout r{false, false, 0};
    if (k_stride == 1 && kdim % 8 == 0 && (rows == 1 || (row_stride % 8 == 0 && row_stride >= kdim))) {
        r.ok = true; r.kc = true; r.ld = rows == 1 ? kdim : row_stride;
    } else if (row_stride == 1 && rows % 8 == 0 && (kdim == 1 || (k_stride % 8 == 0 && k_stride >= rows))) {
        r.ok = true; r.kc = false; r.ld = kdim == 1 ? rows : k_stride;
    }
    return r;
}

}  // namespace

int mfma16dma_variant_count() { return kNumVariants; }
const char *mfma16dma_variant_name(int v) { return (v >= 1 && v <= kNumVariants) ? kVariants[v - 1].name : "?"; }

bool mfma16dma_supported(const GemmProblem &p, int variant) {
    if (p.dtype != DT_F16 && p.dtype != DT_BF16) return false;
    if (variant < 1 || variant > kNumVariants) return false;
    if (p.m < 1 || p.n < 1 || p.k < BK || p.k % BK != 0) return false;
    if (p.m > (1 << 30) || p.n > (1 << 30) || p.k > (1 << 30)) return false;
    if (p.c_cs != 1 && p.n != 1) return false;
    if (p.n > 1 && p.m > 1 && p.c_rs < p.n) return false;
    const OperandLayout la = classify(p.m, p.k, p.a_rs, p.a_cs);
    const OperandLayout lb = classify(p.n, p.k, p.b_cs, p.b_rs);
    if (!la.ok || !lb.ok) return false;
    const Variant &v = kVariants[variant - 1];
    if (la.ld * (la.kc ? v.bm : BK) >= (1ll << 30) || lb.ld * (lb.kc ? v.bn : BK) >= (1ll << 30)) return false;
    if (!aligned16(p.a) || !aligned16(p.b)) return false;
    {   // the epilogue stores whole 16 B (8 B for the 16-column wave tile) pieces of C rows and nothing narrower
        const int vecw = (v.bn / v.waves_n) % 32 == 0 ? 8 : 4;
        const int64_t ldc = p.m == 1 ? p.n : p.c_rs;
        const uintptr_t mask = (uintptr_t)vecw * 2 - 1;
        if (p.n % vecw || ldc % vecw || ((uintptr_t)p.c & mask) || p.c_b1 % vecw || p.c_b2 % vecw) return false;
        if (p.bias && ((uintptr_t)p.bias & mask)) return false;
    }
    if (p.nb1 * p.nb2 > 1) {
        if (p.a_b1 % 8 || p.a_b2 % 8 || p.b_b1 % 8 || p.b_b2 % 8) return false;
        if (p.a_b1 < 0 || p.a_b2 < 0 || p.b_b1 < 0 || p.b_b2 < 0) return false;
    }
    const int64_t tiles = ((p.m + v.bm - 1) / v.bm) * ((p.n + v.bn - 1) / v.bn);
    const int64_t blocks = tiles * (p.reduce ? 1 : p.nb1 * p.nb2);
    if (blocks >= (1ll << 31) || p.nb1 * p.nb2 >= (1ll << 31)) return false;
    if (p.k * (p.reduce ? p.nb1 * p.nb2 : 1) >= (1ll << 31)) return false;
    return true;
}

int mfma16dma_pick_variant(const GemmProblem &p, int compute_units) {
    // Largest tile that still gives every compute unit a workgroup; BN = 64 tiles only for narrow outputs.
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const int wide[] = {1, 2, 3}, narrow[] = {4, 5};
    if (p.n <= 64) {
        for (int v : narrow) {
            if (!mfma16dma_supported(p, v)) continue;
            const Variant &t = kVariants[v - 1];
            const int64_t blocks = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn) * nbatch;
            if (blocks >= compute_units || v == 5) return v;
        }
        return 0;
    }
    for (int v : wide) {
        if (!mfma16dma_supported(p, v)) continue;
        const Variant &t = kVariants[v - 1];
        const int64_t blocks = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn) * nbatch;
        if (blocks >= compute_units || v == 3) return v;
    }
    return 0;
}

// Cost model of the planner (seconds), fitted to timings of this kernel family on a 256-CU MI355X.
//   * a compute unit sustains rate1 / rate2 flop/s on a variant's k tiles when the chip is full; the 128-row tiles
//     only get there with two workgroups resident per compute unit, and lightly loaded chips clock higher;
//   * a work item also moves (operands mostly from L2) + (C tile) bytes at the compute unit's share of HBM;
//   * every work item pays a fixed hand-over cost, every launch a first-load latency and a last C tile;
//   * split-k adds the workspace round trip, which stays in the last-level cache while it is small.
namespace {
struct VariantModel {
    int per_cu;           // workgroups resident per compute unit (LDS and register limits)
    double rate1, rate2;  // flop/s of a compute unit with 1 / with >= 2 resident workgroups
};
constexpr VariantModel kModel[] = {
    {1, 5.50e12, 5.50e12},  // 256x256
    {1, 4.40e12, 4.40e12},  // 256x128
    {2, 3.00e12, 4.25e12},  // 128x128
    {1, 3.60e12, 3.60e12},  // 256x64
    {2, 2.20e12, 2.90e12},  // 128x64
};
constexpr double kItemOverhead = 2.0e-6, kLaunchLatency = 2e-6, kCuBandwidth = 24e9, kOperandWeight = 0.32;
constexpr double kIdleBoost = 0.146, kWsBandwidthCached = 9.5e12, kWsBandwidthHbm = 6.1e12, kWsCached = 128e6;
constexpr double kSplitLaunch = 7e-6, kSplitPerPiece = 0.25e-6;  // 1024^3: 12.4 us unsplit, 15.9 / 18.0 us in 2 / 4 pieces
}  // namespace

void mfma16dma_plan_split(const GemmProblem &p, int compute_units, int forced_variant, int forced_splits, int *variant,
                          int *splits, double *seconds) {
    *variant = 0;
    *splits = 1;
    const int cus = std::max(1, compute_units);
    const int64_t nbatch = p.reduce ? 1 : p.nb1 * p.nb2;
    const bool may_split = nbatch == 1 && p.c_cs == 1;
    const int64_t total_iters = (p.k / BK) * (p.reduce ? p.nb1 * p.nb2 : 1);
    const bool a_kc = classify(p.m, p.k, p.a_rs, p.a_cs).kc, b_kc = classify(p.n, p.k, p.b_cs, p.b_rs).kc;
    const double elem = 2.0, out_elems = (double)p.m * p.n * nbatch;
    double best = 1e300;
    for (int v = 1; v <= kNumVariants; v++) {
        if (forced_variant > 0 && v != forced_variant) continue;
        if (!mfma16dma_supported(p, v)) continue;
        const Variant &t = kVariants[v - 1];
        const VariantModel &vm = kModel[v - 1];
        // narrow outputs take the BN = 64 tiles; wide ones may take the small 128 x 64 tile (more workgroups for a
        // problem of a few tiles), never the 256 x 64 one
        if (forced_variant == 0 && (p.n <= 64 ? t.bn > 64 : (t.bn <= 64 && t.bm > 128))) continue;
        const int64_t tiles = ((p.m + t.bm - 1) / t.bm) * ((p.n + t.bn - 1) / t.bn) * nbatch;
        const double layout = (a_kc && b_kc) ? 1.0 : (!a_kc && !b_kc) ? 0.98 : 0.99;  // transposing LDS reads cost a little
        // candidates 1..16, 20..32, 40..64 (filter gradients of convolutions: a handful of tiles, thousands of k steps)
        int forced_s = forced_splits > 0 ? (int)std::min<int64_t>(forced_splits, total_iters) : 0;
        while (forced_s > 1 && (forced_s - 1) * ((total_iters + forced_s - 1) / forced_s) >= total_iters) forced_s--;  // no empty split
        for (int s = forced_s ? forced_s : 1; s <= (forced_s ? forced_s : 64); s += (s < 16 ? 1 : s < 32 ? 4 : 8)) {
            if (s > 1 && (!may_split || (forced_splits == 0 && total_iters / s < 4))) break;
            const int64_t chunk = (total_iters + s - 1) / s;
            if ((s - 1) * chunk >= total_iters) continue;  // an empty split
            const int64_t items = tiles * s;
            const int64_t grid = std::min<int64_t>(items, (int64_t)cus * vm.per_cu);
            const int64_t conc = (grid + cus - 1) / cus, items_per_wg = (items + grid - 1) / grid;
            const double active = (double)std::min<int64_t>(grid, cus) / cus;
            const double cu_rate = (conc >= 2 ? vm.rate2 : vm.rate1) * layout * (1.0 + kIdleBoost * (1.0 - active));
            const double t_mma = chunk * (2.0 * t.bm * t.bn * BK) / (cu_rate / conc);
            const double out_bytes = (double)t.bm * t.bn * (s > 1 ? 4.0 : elem * (1 + p.accumulate));
            const double t_mem = (kOperandWeight * (t.bm + t.bn) * BK * elem * chunk + out_bytes) / (kCuBandwidth / conc);
            double time = items_per_wg * (std::max(t_mma, t_mem) + kItemOverhead) + kLaunchLatency +
                          out_bytes / (kCuBandwidth / conc);
            if (s > 1) {
                const double ws = s * out_elems * 4.0;
                // second launch + the reduce kernel's chain of s dependent partial-tile reads, then the workspace round trip
                time += kSplitLaunch + kSplitPerPiece * s +
                        (ws + out_elems * elem * (1 + p.accumulate)) / (ws <= kWsCached ? kWsBandwidthCached : kWsBandwidthHbm);
            }
            if (time < best) {
                best = time;
                *variant = v;
                *splits = s;
            }
        }
    }
    if (seconds) *seconds = best;
}

// layout of the split-k workspace: [splits][tiles_m * BM][tiles_n * BN] f32, then -- row sums of A asked for --
// [splits * (BM / 64) * 8][tiles_m * BM] f32
static void ws_layout(const GemmProblem &p, int variant, int64_t *ld, int64_t *split_stride, int64_t *ksum_stride = nullptr) {
    const Variant &v = kVariants[variant - 1];
    *ld = ((p.n + v.bn - 1) / v.bn) * v.bn;
    *split_stride = *ld * (((p.m + v.bm - 1) / v.bm) * v.bm);
    if (ksum_stride) *ksum_stride = ((p.m + v.bm - 1) / v.bm) * v.bm;
}
// Workspace slots of the row sums: one per split, sharing tile column and wave.
static int ksum_slots(int variant, int splits) { return splits * (kVariants[variant - 1].bm / 64) * 8; }

size_t mfma16dma_workspace_bytes(const GemmProblem &p, int variant, int splits) {
    if (splits <= 1) return 0;
    int64_t ld, stride, ks;
    ws_layout(p, variant, &ld, &stride, &ks);
    const int64_t slots = p.ksum ? ksum_slots(variant, splits) : 0;
    return (size_t)(stride * splits + ks * slots) * sizeof(float);
}

// The sums of A's rows ride along only where A and B are both stored contraction-major (m- and n-contiguous: the
// weight gradient grad_out^T . x after the output transposition) and the contraction is split (the partial sums are
// combined by the reduce kernel that runs then anyway).
bool mfma16dma_ksum_supported(const GemmProblem &p, int variant, int splits) {
    if (!p.ksum || p.ksum_of != KSUM_OF_A || splits <= 1 || !mfma16dma_supported(p, variant)) return false;
    if (!p.reduce && p.nb1 * p.nb2 != 1) return false;
    if ((uintptr_t)p.ksum & 1u) return false;
    const Variant &v = kVariants[variant - 1];
    if ((p.n + v.bn - 1) / v.bn < v.bm / 64) return false;  // too few tile columns to share a tile's pieces
    return !classify(p.m, p.k, p.a_rs, p.a_cs).kc && !classify(p.n, p.k, p.b_cs, p.b_rs).kc;
}

hipError_t launch_mfma16dma(const GemmProblem &g, int variant, hipStream_t stream) {
    if (!mfma16dma_supported(g, variant)) return hipErrorInvalidValue;
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
    p.group_m = 4;
    const int total_iters = (p.k / BK) * p.kbatches;
    p.splits = 1; p.chunk = total_iters; p.ws = nullptr; p.ws_ld = 0; p.ws_split_stride = 0;
    p.ws_ksum = nullptr; p.ws_ksum_stride = 0;
    if (g.ksum && !mfma16dma_ksum_supported(g, variant, g.splits)) return hipErrorInvalidValue;
    if (g.splits > 1) {
        if (!g.workspace || p.total_blocks != p.tiles_per_batch) return hipErrorInvalidValue;
        p.splits = g.splits;
        p.chunk = (total_iters + g.splits - 1) / g.splits;
        if ((int64_t)(g.splits - 1) * p.chunk >= total_iters) return hipErrorInvalidValue;
        p.ws = g.workspace;
        int64_t ks_stride = 0;
        ws_layout(g, variant, &p.ws_ld, &p.ws_split_stride, &ks_stride);
        if (g.ksum) {
            p.ws_ksum = g.workspace + p.ws_split_stride * g.splits;
            p.ws_ksum_stride = (int)ks_stride;
        }
        p.total_blocks = p.tiles_per_batch * g.splits;
    }
    p.grid = 0;  // set per kernel instantiation at launch
    hipError_t e = (g.dtype == DT_F16) ? launch_variant<_Float16>(variant, p, g.compute_units, la.kc, lb.kc, stream)
                                       : launch_variant<__bf16>(variant, p, g.compute_units, la.kc, lb.kc, stream);
    if (e != hipSuccess || g.splits <= 1) return e;
    return launch_splitk_reduce(g, p.ws_ld, p.ws_split_stride, stream, p.ws_ksum, p.ws_ksum_stride, ksum_slots(variant, g.splits));
}

}  // namespace dfdx_rocm
