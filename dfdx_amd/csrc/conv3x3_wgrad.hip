// Filter gradient of a 3 x 3 convolution at unit stride with padding 1 (f16 / bf16, f32 accumulate, gfx950) without a patch
// matrix: the `weight_g^T += img * unfold(grad_out)^T` product of `Conv2DKernel::backward` (dfdx-core/src/tensor_ops/
// conv2d/cpu_kernel.rs:152-170) for the shapes the band kernel of conv3x3.hip takes.
//
//   grad_filters[o][c][ky][kx] += sum over (b, y, x) of  grad_out[b][o][y][x] * img[b][c][y + ky - 1][x + kx - 1]
//
// as nine GEMMs (one per tap) with M = output channels, N = input channels and K = pixels.  Both operands are kept in LDS
// pixel-major -- a record per pixel with its 64 channels next to each other, rows of W + 2 records whose first and last are
// zeros (the padding columns) -- exactly as the band kernel keeps the image; the MFMA fragments (8 consecutive pixels of
// one channel per lane) come out of them through the transposing LDS read ds_read_b64_tr_b16.  In that padded pixel
// numbering a tap is ONE shift of the image band against the grad_out band, (ky - 1) (W + 2) + (kx - 1) records, for every
// pixel; the zero columns and rows take care of the borders.
//
// A workgroup (12 waves) owns one block of 64 output x 64 input channels and walks a share of the (image, band of rows)
// work items, all 9 x 64 x 64 sums staying in its accumulators (wave w: the three (tap, 16-channel tile) pairs 3w .. 3w + 2
// times the four 16-row tiles of output channels: 12 MFMAs per 32 pixels against 4 + 3 fragments).  At the end every
// workgroup leaves its sums as f32 in a workspace and a second kernel adds the shares in a fixed order into grad_filters
// (one rounding): deterministic.
//
// f32 has a kernel of its own further down (conv3x3_wgrad_f32_kernel): v_mfma_f32_16x16x4_f32 takes ONE k per lane, so no
// operand needs transposing -- both bands stay channel-major, as they lie in memory, and are written into LDS by the loads
// themselves.
#include "gemm_internal.h"
#include "conv3x3.h"
#include <algorithm>

namespace dfdx_rocm {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define DFDX_LDS __attribute__((address_space(3)))

constexpr int NTH = 768;    // 12 waves
constexpr int REC = 144;    // bytes of a pixel record: 64 channels + 16 of padding (the transposing reads take any pitch at the same rate;
                            // the deposits, two records apart from lane to lane, collide 2-way on an odd multiple of 16 bytes, 4-way on 160)
constexpr int KMAX = 256;   // records of a grad_out band at most (a multiple of the 32-pixel k step)
constexpr int UMAX = 2;     // pixel-pair units of a band a thread may own

template <typename T> struct MmaW;
template <> struct MmaW<_Float16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};
template <> struct MmaW<__bf16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
};

template <> struct MmaW<float> {
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <typename T> struct StoredAs { typedef uint16_t type; };
template <> struct StoredAs<float> { typedef float type; };

struct Params {
    const uint16_t *img;  // [B][C][H][W]
    const uint16_t *go;   // [B][O][H][W]
    float *partial;       // [slices][combos][9][64][64]
    int C, O, H, W, HW;
    int R, bands;          // rows per band, bands per image
    int items;             // batch x bands
    int slices, cblocks;   // workgroups per channel-block pair; blocks of 64 input channels
    int kp;                // records of the grad_out band, rounded up to the k step
    int xrecs;             // records of the image band that are ever read (zeroed once)
    uint32_t magic_pairs;  // ceil(2^32 / (W / 2))
};

// Fragment of an operand stored [pixel record][channel]: 16 channels (from `chan0`) x 32 pixels (from record `rec0`).
// Lane 16 g + L supplies the addresses of 4 channels of record rec0 + 8 g + L / 4 (and of the record 4 further); the
// hardware hands lane L the 8 pixels of channel chan0 + L: the layout the MFMA wants for 8 consecutive k.
__device__ __forceinline__ u32x4 tr_fragment(const uint8_t *band, int rec0, int chan0, int l16, int lq) {
    const uint8_t *p = band + (rec0 + lq * 8 + l16 / 4) * REC + (chan0 + 4 * (l16 % 4)) * 2;
    const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DFDX_LDS v4i16 *)(DFDX_LDS uint8_t *)p);
    const v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DFDX_LDS v4i16 *)(DFDX_LDS uint8_t *)(p + 4 * REC));
    const u32x2 l = __builtin_bit_cast(u32x2, lo), h = __builtin_bit_cast(u32x2, hi);
    return u32x4{l[0], l[1], h[0], h[1]};
}

template <typename T>
__global__ __launch_bounds__(NTH, 3) void conv3x3_wgrad_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t *const gband = smem;                    // grad_out band: kp records
    uint8_t *const xband = smem + KMAX * REC;       // image band: xrecs records, its row 0 = the row above the band
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int l16 = lane % 16, lq = lane / 16;
    const int W = p.W, WP = W + 2, H = p.H, pairs = W / 2;

    // everything the deposits never write stays zero for the whole launch: padding columns, the records behind the
    // last band row that the k steps and the tap shifts still touch
    for (int i = tid; i < (KMAX + p.xrecs) * (REC / 16); i += NTH) *(u32x4 *)(smem + i * 16) = u32x4{0, 0, 0, 0};

    const int combos = gridDim.x / p.slices;
    const int combo = blockIdx.x % combos, slice = blockIdx.x / combos;
    const int cb = combo % p.cblocks, ob = combo / p.cblocks;

    f32x4 acc[4][3];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 3; e++) acc[i][e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // the wave's three (tap, input-channel tile) pairs: pair q = tap * 4 + tile
    int b_rec[3], b_chan[3];
#pragma unroll
    for (int e = 0; e < 3; e++) {
        const int q = wave * 3 + e, tap = q / 4, j = q % 4;
        b_rec[e] = WP + (tap / 3 - 1) * WP + (tap % 3 - 1);  // image record that meets grad_out record 0 at this tap
        b_chan[e] = 16 * j;
    }

    // ---- what a thread moves per work item: UMAX pixel-pair units of each band (8 channels x 2 neighbouring pixels)
    const int x_rows = p.R + 2, g_rows = p.R;
    const int x_units = 8 * x_rows * pairs, g_units = 8 * g_rows * pairs;
    int xs_off[UMAX], xs_row[UMAX], xs_dst[UMAX], gs_off[UMAX], gs_row[UMAX], gs_dst[UMAX];
#pragma unroll
    for (int s = 0; s < UMAX; s++) {
        const int u = tid + s * NTH;
        const int t = (int)__umulhi((uint32_t)u, p.magic_pairs), xp = u - t * pairs;  // t = group * rows + row
        {
            const int cg = t / x_rows, r = t - cg * x_rows;
            xs_row[s] = u < x_units ? r : -1000000;
            xs_off[s] = (8 * cg * H) * W + 2 * xp;  // + row * W: element offset of the unit's first channel in its block
            xs_dst[s] = (r * WP + 1 + 2 * xp) * REC + cg * 16;
        }
        {
            const int cg = t / g_rows, r = t - cg * g_rows;
            gs_row[s] = u < g_units ? r : -1000000;
            gs_off[s] = (8 * cg * H) * W + 2 * xp;
            gs_dst[s] = (r * WP + 1 + 2 * xp) * REC + cg * 16;
        }
    }
    __syncthreads();

    uint32_t dx[UMAX][8], dg[UMAX][8];
    auto request = [&](int item) {  // the global loads of one work item: 8 channels x 2 pixels per unit and band
        const int b = item / p.bands, y0 = (item - b * p.bands) * p.R;
        const __amdgpu_buffer_rsrc_t xsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.img + ((int64_t)b * p.C + cb * 64) * p.HW), 0, 64 * p.HW * 2, 0x00020000);
        const __amdgpu_buffer_rsrc_t gsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.go + ((int64_t)b * p.O + ob * 64) * p.HW), 0, 64 * p.HW * 2, 0x00020000);
#pragma unroll
        for (int s = 0; s < UMAX; s++) {
            const int yx = y0 - 1 + xs_row[s], yg = y0 + gs_row[s];
            // (a unit outside the image, or none at all, points past the end of the resource and receives zeros)
            const uint32_t ox = (xs_row[s] >= 0 && yx >= 0 && yx < H) ? (uint32_t)(xs_off[s] + yx * W) * 2u : 0xFFFFFFF0u;
            const uint32_t og = (gs_row[s] >= 0 && yg < H) ? (uint32_t)(gs_off[s] + yg * W) * 2u : 0xFFFFFFF0u;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                dx[s][e] = __builtin_amdgcn_raw_buffer_load_b32(xsrc, (int)ox, e * p.HW * 2, 0);
                dg[s][e] = __builtin_amdgcn_raw_buffer_load_b32(gsrc, (int)og, e * p.HW * 2, 0);
            }
        }
    };
    if (slice < p.items) request(slice);
    for (int item = slice; item < p.items; item += p.slices) {
        __syncthreads();  // the previous item's fragments have been read
#pragma unroll
        for (int s = 0; s < UMAX; s++) {
            u32x4 a0, a1, g0, g1;
#pragma unroll
            for (int h = 0; h < 4; h++) {
                a0[h] = __builtin_amdgcn_perm(dx[s][2 * h + 1], dx[s][2 * h], 0x05040100u);  // low halves: pixel 2 xp
                a1[h] = __builtin_amdgcn_perm(dx[s][2 * h + 1], dx[s][2 * h], 0x07060302u);  // high halves: pixel 2 xp + 1
                g0[h] = __builtin_amdgcn_perm(dg[s][2 * h + 1], dg[s][2 * h], 0x05040100u);
                g1[h] = __builtin_amdgcn_perm(dg[s][2 * h + 1], dg[s][2 * h], 0x07060302u);
            }
            if (xs_row[s] >= 0) {
                *(u32x4 *)(xband + xs_dst[s]) = a0;
                *(u32x4 *)(xband + xs_dst[s] + REC) = a1;
            }
            if (gs_row[s] >= 0) {
                *(u32x4 *)(gband + gs_dst[s]) = g0;
                *(u32x4 *)(gband + gs_dst[s] + REC) = g1;
            }
        }
        __syncthreads();
        if (item + p.slices < p.items) request(item + p.slices);  // the next item travels while this one is multiplied
        // k steps of 32 pixels in a software pipeline: the fragments of step k + 1 are requested from LDS in front of
        // the 12 MFMAs of step k (two register sets, the loop unrolled by two)
        u32x4 fa[2][4], fb[2][3];
        auto read_step = [&](int k0, u32x4(&a)[4], u32x4(&bf)[3]) {
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = tr_fragment(gband, k0, 16 * i, l16, lq);
#pragma unroll
            for (int e = 0; e < 3; e++) bf[e] = tr_fragment(xband, k0 + b_rec[e], b_chan[e], l16, lq);
        };
        auto mma_step = [&](const u32x4(&a)[4], const u32x4(&bf)[3]) {
#pragma unroll
            for (int e = 0; e < 3; e++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[i][e] = MmaW<T>::mfma(bf[e], a[i], acc[i][e]);
        };
        read_step(0, fa[0], fb[0]);
        for (int k0 = 0; k0 < p.kp; k0 += 64) {  // kp is a multiple of 32: the second half may be missing
            const bool second = k0 + 32 < p.kp;
            if (second) read_step(k0 + 32, fa[1], fb[1]);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            if (second) {
                if (k0 + 64 < p.kp) read_step(k0 + 64, fa[0], fb[0]);
                __builtin_amdgcn_sched_barrier(0);
                mma_step(fa[1], fb[1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- this workgroup's share of the sums: lane holds output channel 16 i + l16 and input channels 16 j + 4 lq + 0..3
    float *const share = p.partial + ((int64_t)slice * combos + combo) * (9 * 64 * 64);
#pragma unroll
    for (int e = 0; e < 3; e++) {
        const int q = wave * 3 + e, tap = q / 4, j = q % 4;
#pragma unroll
        for (int i = 0; i < 4; i++) *(f32x4 *)(share + (tap * 64 + 16 * i + l16) * 64 + 16 * j + 4 * lq) = acc[i][e];
    }
}

// grad_filters[o][c][tap] += sum over the slices of their shares (f32), rounded once.  A workgroup owns 128 consecutive
// sums (32 lanes x 4 sums: 512 contiguous bytes of every share per load); its 8 thread groups add an eighth of the slices
// each, in slice order, and the eight subtotals meet in LDS in group order: one fixed summation order, whatever the timing.
template <typename T>
__global__ __launch_bounds__(256) void conv3x3_wgrad_reduce_kernel(const float *__restrict__ partial,
                                                                   typename StoredAs<T>::type *__restrict__ grad_filters, int C,
                                                                   int cblocks, int combos, int slices, int total) {
    __shared__ f32x4 subtotal[8][32];
    const int lane_elem = threadIdx.x % 32, group = threadIdx.x / 32;
    const int i = blockIdx.x * 128 + lane_elem * 4;  // (combo, tap, o, c), c fastest; total is a multiple of 128
    const int combo = i / (9 * 4096), within = i - combo * (9 * 4096);
    const int per = (slices + 7) / 8, s0 = group * per, s1 = min(slices, s0 + per);
    const float *src = partial + (int64_t)combo * (9 * 4096) + within;
    const int64_t step = (int64_t)combos * (9 * 4096);
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    int s = s0;
    for (; s + 8 <= s1; s += 8) {
        f32x4 v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = *(const f32x4 *)(src + (s + e) * step);
#pragma unroll
        for (int e = 0; e < 8; e++) sum += v[e];
    }
    for (; s < s1; s++) sum += *(const f32x4 *)(src + s * step);
    subtotal[group][lane_elem] = sum;
    __syncthreads();
    if (group == 0 && i < total) {
        f32x4 all = subtotal[0][lane_elem];
#pragma unroll
        for (int g = 1; g < 8; g++) all += subtotal[g][lane_elem];
        const int c = within % 64, o = (within / 64) % 64, tap = within / 4096;
        const int cb = combo % cblocks, ob = combo / cblocks;
        typename StoredAs<T>::type *dst = grad_filters + ((int64_t)(ob * 64 + o) * C + cb * 64 + c) * 9 + tap;
#pragma unroll
        for (int e = 0; e < 4; e++) dst[9 * e] = MmaW<T>::from_f32(MmaW<T>::to_f32(dst[9 * e]) + all[e]);
    }
}

// ---- f32 ----------------------------------------------------------------------------------------------------------------
// The same nine GEMMs with v_mfma_f32_16x16x4_f32: a lane supplies ONE value, (channel l16, pixel lq) of a 16-channel x
// 4-pixel fragment, so a fragment is one ds_read_b32 from a CHANNEL-major band -- the layout of the tensors in memory.
// A band row of a channel is RP = 4 + W rounded up to 4 slots: four zeros, the W pixels, zeros up to the pitch; the zeros
// in front of a row are the padding column of its first pixel and of the previous row's last one.  k steps are the
// 4-aligned slot groups that hold pixels (the group of zeros in front of every row is skipped); a tap shifts the image
// slot by ky RP + kx - 1 against the grad_out slot.  Channel pitches are odd multiples of 2 dwords: the 16 channels x 4
// consecutive slots of a fragment read then count no bank conflict (odd multiples of 4 counted 2-way conflicts).
// Both bands of a work item (RS grad_out rows, RS + 2 image rows, 64 channels each) are written into LDS by the loads
// themselves (buffer_load_dword ... lds: 64 consecutive slots of one channel per wave instruction; a lane whose slot is a
// zero -- padding, a row outside the image -- points past the end of the buffer resource and the hardware writes the
// zero; a lane past the end of the channel's band is switched off): no staging registers, no deposit phase, two stages,
// one barrier per item.  A wave requests the next item's bands one channel per k step of the current item: requested in
// one block behind the barrier, the 250 instructions of an item fill the queue of the address unit and every wave waits
// there instead of multiplying.
constexpr int SEGS = 5;          // 64-slot runs of one channel's band at most
constexpr int PITCH_MAX = 320;   // G pitch + X pitch (dwords per channel): two stages of 64 channels in 160 KB
constexpr uint32_t UNIT_ZERO = 0xFFFFFFFFu, UNIT_NONE = 0xFFFFFFFEu;

struct ParamsF {
    const float *img, *go;
    float *partial;
    int C, O, H, W, HW;
    int RS, bands, items, slices, cblocks;
    int RP, Q;       // slots per band row; k steps per band row
    int GP, XP;      // dwords per channel of the grad_out / image band
    uint32_t magic_rp;
};

__global__ __launch_bounds__(NTH, 1) void conv3x3_wgrad_f32_kernel(const ParamsF p) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int l16 = lane % 16, lq = lane / 16;
    const uint32_t stage_bytes = (uint32_t)(p.GP + p.XP) * 256u;  // 64 channels of both bands
    const uint32_t smem_addr = (uint32_t)(uintptr_t)(DFDX_LDS const uint8_t *)smem;

    const int combos = gridDim.x / p.slices;
    const int combo = blockIdx.x % combos, slice = blockIdx.x / combos;
    const int cb = combo % p.cblocks, ob = combo / p.cblocks;

    // what this lane fetches for slot 64 seg + lane of any channel: element offset inside the channel's plane, counted
    // from image row y0 - 1, in the low 24 bits and the band row above them
    uint32_t g_unit[SEGS], x_unit[SEGS];
#pragma unroll
    for (int seg = 0; seg < SEGS; seg++) {
        const int s = 64 * seg + lane;
        const int r = (int)__umulhi((uint32_t)s, p.magic_rp), x = s - r * p.RP - 4;
        const bool pixel = x >= 0 && x < p.W;
        // grad_out row r lies beside image band row r + 1; its slots behind the last row are never read
        g_unit[seg] = s >= p.RS * p.RP ? UNIT_NONE : pixel ? (uint32_t)((r + 1) * p.W + x) | ((uint32_t)(r + 1) << 24) : UNIT_ZERO;
        x_unit[seg] = s >= p.XP ? UNIT_NONE : (pixel && r < p.RS + 2) ? (uint32_t)(r * p.W + x) | ((uint32_t)r << 24) : UNIT_ZERO;
    }
    const int g_segs = (p.RS * p.RP + 63) / 64, x_segs = (p.XP + 63) / 64;

    // the item being requested: its image, rows and destination stage; dma_ch = the next channel this wave requests
    __amdgpu_buffer_rsrc_t xsrc, gsrc;
    int dma_ybase = 0, dma_ch = 64;
    uint32_t dma_dst = 0;
    auto begin_request = [&](int item, int stage) {
        const int b = item / p.bands;
        dma_ybase = (item - b * p.bands) * p.RS - 1;
        xsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.img + ((int64_t)b * p.C + cb * 64) * p.HW), 0, 64 * p.HW * 4, 0x00020000);
        gsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.go + ((int64_t)b * p.O + ob * 64) * p.HW), 0, 64 * p.HW * 4, 0x00020000);
        dma_dst = smem_addr + (uint32_t)stage * stage_bytes;
        dma_ch = wave;
    };
    auto request_channel = [&]() {  // both bands of channel dma_ch
        if (dma_ch >= 64) return;
        const int plane = dma_ch * p.HW * 4;
        const int row0 = dma_ybase * p.W;
        auto offset_of = [&](uint32_t u) -> int {
            const int y = dma_ybase + (int)(u >> 24);
            return (u != UNIT_ZERO && (unsigned)y < (unsigned)p.H) ? ((int)(u & 0xFFFFFFu) + row0) * 4 : (int)0x80000000u;
        };
#pragma unroll
        for (int seg = 0; seg < SEGS; seg++)
            if (seg < g_segs && g_unit[seg] != UNIT_NONE)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(gsrc, (DFDX_LDS void *)(uintptr_t)(dma_dst + (uint32_t)(dma_ch * p.GP + 64 * seg) * 4u), 4,
                                                         offset_of(g_unit[seg]), plane, 0, 0);
#pragma unroll
        for (int seg = 0; seg < SEGS; seg++)
            if (seg < x_segs && x_unit[seg] != UNIT_NONE)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xsrc, (DFDX_LDS void *)(uintptr_t)(dma_dst + (uint32_t)(64 * p.GP + dma_ch * p.XP + 64 * seg) * 4u), 4,
                                                         offset_of(x_unit[seg]), plane, 0, 0);
        dma_ch += 12;
    };

    f32x4 acc[4][3];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 3; e++) acc[i][e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // fragment addresses (dwords from the start of a stage) at slot 0; the wave's three (tap, input-channel tile) pairs
    const int g_at = l16 * p.GP + lq;
    int x_at[3];
#pragma unroll
    for (int e = 0; e < 3; e++) {
        const int q = wave * 3 + e, tap = q / 4, j = q % 4;
        x_at[e] = p.GP * 64 + (16 * j + l16) * p.XP + lq + (tap / 3) * p.RP + (tap % 3) - 1;
    }

    int stage = 0;
    if (slice < p.items) {
        begin_request(slice, 0);
        while (dma_ch < 64) request_channel();
    }
    for (int item = slice; item < p.items; item += p.slices) {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the item has landed
        __syncthreads();                     // ... and everybody's; the other stage is no longer being read
        if (item + p.slices < p.items) begin_request(item + p.slices, stage ^ 1);
        const float *const st = (const float *)(smem + (uint32_t)stage * stage_bytes);
        const int y0 = (item % p.bands) * p.RS;
        const int steps = min(p.RS, p.H - y0) * p.Q;
        // k steps of 4 slots in a software pipeline: the 7 fragments of step t + 1 are requested from LDS in front of
        // the 12 MFMAs of step t (no conditional read inside the loop: with one, the compiler's wait in front of a step's
        // MFMAs also covers the reads just issued for the next step)
        float fa[2][4], fb[2][3];
        int slot = 4, q = 0;
        auto read_step = [&](float(&a)[4], float(&bf)[3]) {
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = st[g_at + 16 * i * p.GP + slot];
#pragma unroll
            for (int e = 0; e < 3; e++) bf[e] = st[x_at[e] + slot];
            slot += 4;
            if (++q == p.Q) {  // over the zeros in front of the next row
                q = 0;
                slot += 4;
            }
            request_channel();
        };
        auto mma_step = [&](const float(&a)[4], const float(&bf)[3]) {
#pragma unroll
            for (int e = 0; e < 3; e++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[i][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[e], a[i], acc[i][e], 0, 0, 0);
        };
        read_step(fa[0], fb[0]);
        int t = 0;
        for (; t + 2 < steps; t += 2) {
            read_step(fa[1], fb[1]);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            read_step(fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(fa[1], fb[1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (t + 1 < steps) {  // one or two steps are left
            read_step(fa[1], fb[1]);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(fa[1], fb[1]);
        } else {
            mma_step(fa[0], fb[0]);
        }
        while (dma_ch < 64) request_channel();  // (an item of few k steps)
        stage ^= 1;
    }

    float *const share = p.partial + ((int64_t)slice * combos + combo) * (9 * 64 * 64);
#pragma unroll
    for (int e = 0; e < 3; e++) {
        const int q = wave * 3 + e, tap = q / 4, j = q % 4;
#pragma unroll
        for (int i = 0; i < 4; i++) *(f32x4 *)(share + (tap * 64 + 16 * i + l16) * 64 + 16 * j + 4 * lq) = acc[i][e];
    }
}

struct PlanF {
    int RS, bands, RP, Q, GP, XP, slices, combos;
    size_t lds;
};
int bank_free_pitch(int n) {  // the smallest odd multiple of 2 that is >= n
    int p = (n + 1) / 2 * 2;
    return p % 4 == 2 ? p : p + 2;
}
bool make_plan_f32(const Conv3x3Problem &c, int compute_units, PlanF *out) {
    if (c.dtype != DT_F32) return false;
    if (c.batch < 1 || c.chan_in < 64 || c.chan_in % 64 || c.chan_out < 64 || c.chan_out % 64) return false;
    if (c.w < 2 || c.h < 1) return false;
    const int64_t hw = (int64_t)c.h * c.w;
    if (hw >= (1 << 22)) return false;  // byte offsets inside a block of 64 planes are 32-bit integers
    if (((uintptr_t)c.img & 3u) || ((uintptr_t)c.out & 3u) || ((uintptr_t)c.filters & 3u)) return false;
    PlanF pl;
    pl.Q = (c.w + 3) / 4;
    pl.RP = 4 * pl.Q + 4;
    pl.RS = 0;
    for (int rs = 1; rs <= std::min(c.h, 64); rs++) {  // as many rows per item as two stages leave room for
        const int gp = bank_free_pitch(rs * pl.RP), xp = bank_free_pitch((rs + 2) * pl.RP + 1);
        if (gp + xp > PITCH_MAX) break;
        pl.RS = rs; pl.GP = gp; pl.XP = xp;
    }
    if (pl.RS < 1) return false;
    pl.bands = (c.h + pl.RS - 1) / pl.RS;
    pl.lds = (size_t)2 * (pl.GP + pl.XP) * 256;
    pl.combos = (c.chan_in / 64) * (c.chan_out / 64);
    const int64_t items = (int64_t)c.batch * pl.bands;
    if (items >= (1ll << 31) || pl.combos > 65536) return false;
    pl.slices = (int)std::max<int64_t>(1, std::min<int64_t>(items, std::max(1, compute_units) / pl.combos));
    *out = pl;
    return true;
}

struct Plan {
    int R, bands, kp, xrecs, slices, combos;
    size_t lds;
};
bool make_plan(const Conv3x3Problem &c, int compute_units, Plan *out) {
    if (c.dtype != DT_F16 && c.dtype != DT_BF16) return false;
    if (c.batch < 1 || c.chan_in < 64 || c.chan_in % 64 || c.chan_out < 64 || c.chan_out % 64) return false;
    if (c.w < 4 || c.w > 254 || c.w % 2 || c.h < 1) return false;
    const int64_t hw = (int64_t)c.h * c.w;
    if (hw >= (1 << 24) || 64 * hw >= (1ll << 30)) return false;
    if (((uintptr_t)c.img & 3u) || ((uintptr_t)c.out & 3u) || ((uintptr_t)c.filters & 1u)) return false;
    const int wp = c.w + 2;
    Plan pl;
    pl.R = std::min(c.h, KMAX / wp);
    while (pl.R > 1 && 8 * (pl.R + 2) * (c.w / 2) > UMAX * NTH) pl.R--;  // wide rows: fewer of them per item
    if (pl.R < 1) return false;
    pl.bands = (c.h + pl.R - 1) / pl.R;
    pl.kp = (pl.R * wp + 31) / 32 * 32;
    pl.xrecs = pl.kp + 2 * wp + 8;  // the last k step under the largest tap shift
    if (8 * (pl.R + 2) * (c.w / 2) > UMAX * NTH) return false;
    pl.lds = (size_t)(KMAX + pl.xrecs) * REC;
    if (pl.lds > 160 * 1024) return false;
    pl.combos = (c.chan_in / 64) * (c.chan_out / 64);
    const int64_t items = (int64_t)c.batch * pl.bands;
    if (items >= (1ll << 31) || pl.combos > 65536) return false;
    pl.slices = (int)std::max<int64_t>(1, std::min<int64_t>(items, std::max(1, compute_units) / pl.combos));
    *out = pl;
    return true;
}

}  // namespace

// `c` as for the forward kernel, with `out` = grad_out [batch][chan_out][h][w] and `filters` = grad_filters (accumulated into).
bool conv3x3_wgrad_supported(const Conv3x3Problem &c, int compute_units) {
    Plan pl;
    PlanF plf;
    return make_plan(c, compute_units, &pl) || make_plan_f32(c, compute_units, &plf);
}

size_t conv3x3_wgrad_workspace_bytes(const Conv3x3Problem &c, int compute_units) {
    Plan pl;
    PlanF plf;
    if (make_plan_f32(c, compute_units, &plf)) return (size_t)plf.slices * plf.combos * 9 * 64 * 64 * sizeof(float);
    if (!make_plan(c, compute_units, &pl)) return 0;
    return (size_t)pl.slices * pl.combos * 9 * 64 * 64 * sizeof(float);
}

hipError_t launch_conv3x3_wgrad_f32(const Conv3x3Problem &c, const PlanF &pl, void *workspace, hipStream_t stream) {
    ParamsF p;
    p.img = (const float *)c.img; p.go = (const float *)c.out; p.partial = (float *)workspace;
    p.C = c.chan_in; p.O = c.chan_out; p.H = c.h; p.W = c.w; p.HW = c.h * c.w;
    p.RS = pl.RS; p.bands = pl.bands; p.items = c.batch * pl.bands;
    p.slices = pl.slices; p.cblocks = c.chan_in / 64;
    p.RP = pl.RP; p.Q = pl.Q; p.GP = pl.GP; p.XP = pl.XP;
    p.magic_rp = (uint32_t)(((1ull << 32) + pl.RP - 1) / pl.RP);
    static PerDevice attr_on;
    std::atomic<int> &known = attr_on.here();
    if (known.load(std::memory_order_acquire) == 0) {
        hipError_t e = hipFuncSetAttribute((const void *)conv3x3_wgrad_f32_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        known.store(1, std::memory_order_release);
    }
    conv3x3_wgrad_f32_kernel<<<(unsigned)(pl.combos * pl.slices), NTH, pl.lds, stream>>>(p);
    const int total = pl.combos * 9 * 4096;
    conv3x3_wgrad_reduce_kernel<float><<<total / 128, 256, 0, stream>>>((const float *)workspace, (float *)c.filters, c.chan_in, p.cblocks,
                                                                        pl.combos, pl.slices, total);
    return hipGetLastError();
}

hipError_t launch_conv3x3_wgrad(const Conv3x3Problem &c, int compute_units, void *workspace, hipStream_t stream) {
    PlanF plf;
    if (make_plan_f32(c, compute_units, &plf)) {
        if ((uintptr_t)workspace & 15u) return hipErrorNotSupported;
        return launch_conv3x3_wgrad_f32(c, plf, workspace, stream);
    }
    Plan pl;
    if (!make_plan(c, compute_units, &pl) || ((uintptr_t)workspace & 15u)) return hipErrorNotSupported;
    Params p;
    p.img = (const uint16_t *)c.img; p.go = (const uint16_t *)c.out; p.partial = (float *)workspace;
    p.C = c.chan_in; p.O = c.chan_out; p.H = c.h; p.W = c.w; p.HW = c.h * c.w;
    p.R = pl.R; p.bands = pl.bands; p.items = c.batch * pl.bands;
    p.slices = pl.slices; p.cblocks = c.chan_in / 64;
    p.kp = pl.kp; p.xrecs = pl.xrecs;
    p.magic_pairs = (uint32_t)(((1ull << 32) + c.w / 2 - 1) / (c.w / 2));
    const unsigned grid = (unsigned)(pl.combos * pl.slices);
#define DFDX_WGRAD(T)                                                                                                  \
    do {                                                                                                               \
        static PerDevice attr_on;                                                                                      \
        std::atomic<int> &known = attr_on.here();                                                                      \
        if (known.load(std::memory_order_acquire) == 0) {                                                              \
            hipError_t e = hipFuncSetAttribute((const void *)conv3x3_wgrad_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return e;                                                                             \
            known.store(1, std::memory_order_release);                                                                 \
        }                                                                                                              \
        conv3x3_wgrad_kernel<T><<<grid, NTH, pl.lds, stream>>>(p);                                                     \
        const int total = pl.combos * 9 * 4096;                                                                        \
        conv3x3_wgrad_reduce_kernel<T><<<total / 128, 256, 0, stream>>>((const float *)workspace, (uint16_t *)c.filters, c.chan_in, \
                                                                               p.cblocks, pl.combos, pl.slices, total); \
    } while (0)
    if (c.dtype == DT_F16) DFDX_WGRAD(_Float16);
    else DFDX_WGRAD(__bf16);
#undef DFDX_WGRAD
    return hipGetLastError();
}

}  // namespace dfdx_rocm
