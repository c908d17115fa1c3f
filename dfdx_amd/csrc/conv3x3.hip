// 3 x 3 convolution at unit stride with padding 1 (f16 / bf16, f32 accumulate, gfx950) without a patch matrix, in
// global memory or in any other form: the product of `Conv2DKernel::forward` (dfdx-core/src/tensor_ops/conv2d/
// cpu_kernel.rs:52-98: unfold, then filters . patches per image and group) for the shapes of a residual network's 3 x 3
// layers.
//
//   out[b][o][y][x] = sum over (ky, kx, c) of  filters[o][c][ky][kx] * img[b][c][y + ky - 1][x + kx - 1]
//
// as a GEMM per image with M = output channels, N = pixels, K ordered (tap, channel) -- channel fastest.  With that
// order the 8 consecutive k a lane feeds to one v_mfma_f32_16x16x32 are 8 CHANNELS of ONE pixel at ONE tap, so the B
// operand of every tap is read from one copy of the image in LDS, stored pixel-major with the channels of a pixel next
// to each other; the tap only shifts the pixel a lane reads.  The K*K-fold patch matrix never exists.
//
// A workgroup (8 waves as 2 x 4, wave tile 32 channels x 64 pixels) owns 64 output channels x 256 consecutive pixels of
// one image.  Per chunk of 32 input channels it fills
//   * A: filters[64][9 taps][32 ch] from the re-laid copy wt[o][tap][c] (conv3x3_filters_kernel), the four 16-byte
//     pieces of a tap XOR-swizzled by the row so that the 16 rows of a fragment read fall on distinct banks;
//   * the band of the image its pixels and their neighbours lie in: rows (first row - 1 .. last row + 1) x columns
//     (-1 .. W) x 32 channels, 96 bytes per pixel (64 + 32 of padding: 16 consecutive pixels x 4 pieces read without a
//     bank conflict), zeros outside the image.  The image is stored channel-major in memory, so a thread takes two
//     neighbouring pixels of 8 channels (eight 4-byte loads: any even width is aligned), interleaves them with byte
//     permutes and writes two 16-byte pieces of pixel records;
// then runs 9 taps x 8 MFMAs per wave, the loads of the next chunk in flight meanwhile.  One LDS stage (80 KB at a width
// of 56): two workgroups share a compute unit.
#include "gemm_internal.h"
#include "conv3x3.h"
#include <algorithm>

namespace dfdx_rocm {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int NT = 256;        // pixels per workgroup
constexpr int MT = 64;         // output channels per workgroup
// LDS layouts, both measured free of bank conflicts for the fragment reads (16 rows or pixels x four 16-byte pieces per
// wave instruction; records of 64 or 80 bytes, or unswizzled 576-byte rows, read at half the rate):
constexpr int PIX = 96;        // bytes of a pixel record: 32 channels + 32 of padding (an odd multiple of 32 bytes)
constexpr int AROW = 36 * 16;  // bytes of a filter row: 9 taps x four pieces, piece g of a tap in slot g ^ (row / 2 % 4)
constexpr int A_BYTES = MT * AROW;

template <typename T> struct Mma16;
template <> struct Mma16<_Float16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, h2));
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
};
template <> struct Mma16<__bf16> {
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, b2));
    }
    static __device__ __forceinline__ float to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
};

// f32: the same kernel with 16-channel chunks (a pixel record is still 64 bytes of data), v_mfma_f32_16x16x4_f32 -- a lane's
// 16-byte fragment read feeds four of them, one channel each -- and a thread moving one pixel of 4 channels per unit.
template <> struct Mma16<float> {};

struct Params {
    const void *img;  // [B][C][H][W]
    const void *wt;   // [O][9][C]
    void *out;        // [B][O][H][W]
    int C, O, H, W, HW;
    int nblocks, mblocks;  // pixel blocks per image, blocks of 64 output channels
    int band_rows;         // image rows (with the two halo rows) the LDS band holds
    uint32_t magic_w, magic_pairs;  // ceil(2^32 / W), ceil(2^32 / (W / 2)) (f32: / W again): n / W = umulhi(n, magic_w) for n < 2^24
};

// wt[o][tap][c] = filters[o][c][tap] -- or, `transposed` (the image gradient: a convolution of grad_out with the filters
// turned by 180 degrees, input and output channels trading places), wt[c][tap][o] = filters[o][c][8 - tap].
// `inner` = the extent of wt's last axis, `outer` = that of its first.
template <typename E>
__global__ __launch_bounds__(256) void conv3x3_filters_kernel(const E *__restrict__ f, E *__restrict__ wt, int inner, int outer,
                                                              int transposed, int total) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int c = i % inner, tap = (i / inner) % 9, o = i / (9 * inner);
    wt[i] = transposed ? f[((int64_t)c * outer + o) * 9 + (8 - tap)] : f[((int64_t)o * inner + c) * 9 + tap];
}

// UMAX: pixel-pair units of the band a thread may own per chunk (2: four waves per SIMD, 128 registers; 4: two)
// ACC: the result is added to `out` (one rounding: old value and sum meet in f32).
template <typename T, int UMAX, bool ACC>
__global__ __launch_bounds__(512, (UMAX * (sizeof(T) == 2 ? 8 : 4) <= 16) ? 4 : 2) void conv3x3_kernel(const Params p) {
    constexpr int ES = sizeof(T), CKT = 64 / ES, PPU = 4 / ES;  // element bytes, channels per chunk, pixels per unit
    constexpr int UL = 16 / ES;                                  // channels (= 4-byte loads) per unit: 8 or 4
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t *const sin = smem + A_BYTES;
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int l16 = lane % 16, lq = lane / 16;
    const int wm0 = (wave / 4) * 32, wn0 = (wave % 4) * 64;
    const int W = p.W, WP = W + 2, H = p.H;

    const int mb = blockIdx.x, nb = blockIdx.y, b = blockIdx.z;
    const int n0 = nb * NT;
    // (divisions by W and W / 2 as multiplications: the quotients are exact for every n < 2^24 >= H * W)
    auto div_w = [&](int n) { return (int)__umulhi((uint32_t)n, p.magic_w); };
    const int ytop = div_w(n0);                           // first image row with a pixel of this block
    const int ylast = div_w(min(n0 + NT - 1, p.HW - 1));  // last one
    const int rows = ylast - ytop + 3;                    // band rows: ytop - 1 .. ylast + 1

    // halo columns (x = -1 and x = W) of every band row: zero for the whole launch
    for (int u = tid; u < rows * 2 * 4; u += 512) {
        const int r = u / 8, side = (u / 4) % 2, q = u % 4;
        *(u32x4 *)(sin + (r * WP + side * (W + 1)) * PIX + q * 16) = u32x4{0, 0, 0, 0};
    }

    // fragment addresses
    uint32_t a_addr[2], b_addr[4];
#pragma unroll
    for (int i = 0; i < 2; i++) a_addr[i] = (uint32_t)((wm0 + 16 * i + l16) * AROW + ((lq ^ ((l16 >> 1) & 3)) * 16));
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int n = min(n0 + wn0 + 16 * j + l16, p.HW - 1);
        const int y = div_w(n), x = n - y * W;
        b_addr[j] = (uint32_t)(A_BYTES + ((y - ytop) * WP + x) * PIX + lq * 16);  // tap (0, 0): band row y - ytop, column x
    }

    f32x4 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    const char *const image = (const char *)p.img + (int64_t)b * p.C * p.HW * ES;
    const __amdgpu_buffer_rsrc_t planes = __builtin_amdgcn_make_buffer_rsrc((void *)image, 0, p.C * p.HW * ES, 0x00020000);
    const char *const wrows = (const char *)p.wt + (int64_t)mb * MT * 9 * p.C * ES;
    const int pairs = W / PPU, units = 4 * rows * pairs;  // units of a band row: pixel pairs (16-bit) or pixels (f32)

    // What a thread moves per chunk, worked out once: UMAX pixel-pair units of the band (element offset of channel 0 of
    // the unit's 8 in chunk 0, -1 = the row lies outside the image and is written as zeros; LDS byte offset, -1 = no
    // such unit) (its five of the 64 x 36 filter pieces are worked out where they are used).
    int u_src[UMAX], u_dst[UMAX];
#pragma unroll
    for (int s = 0; s < UMAX; s++) {
        const int u = tid + s * 512;
        const int t = (int)__umulhi((uint32_t)u, p.magic_pairs), xp = u - t * pairs;  // t = cg * rows + r
        const int cg = (t >= rows) + (t >= 2 * rows) + (t >= 3 * rows), r = t - cg * rows;
        const int y = ytop - 1 + r;
        u_src[s] = (u < units && y >= 0 && y < H) ? (UL * cg * H + y) * W + PPU * xp : -1;
        u_dst[s] = u < units ? A_BYTES + (r * WP + 1 + PPU * xp) * PIX + cg * 16 : -1;
    }
    uint32_t d[UMAX][UL];
    u32x4 piece[5];
    auto request = [&](int c0) {  // the global loads of one chunk: the band first, then the filter pieces
        // buffer loads: the image of this batch entry as the resource, one 32-bit byte offset per lane shared by the eight
        // loads of a unit, the channel plane in the scalar offset; a lane with nothing to load points past the end of the
        // resource and receives zeros
#pragma unroll
        for (int s = 0; s < UMAX; s++) {
            const uint32_t off = u_src[s] >= 0 ? (uint32_t)u_src[s] * (uint32_t)ES : 0xFFFFFFF0u;
#pragma unroll
            for (int e = 0; e < UL; e++) d[s][e] = __builtin_amdgcn_raw_buffer_load_b32(planes, (int)off, (c0 + e) * p.HW * ES, 0);
        }
        const char *rowbase = wrows + c0 * ES;
#pragma unroll
        for (int s = 0; s < 5; s++) {
            const int q = tid + s * 512;  // 64 rows x 36 pieces, not kept in registers across the chunk
            const int o = min(q / 36, MT - 1), part = q % 36;
            piece[s] = *(const u32x4 *)(rowbase + (uint32_t)(((o * 9 + part / 4) * p.C + (part % 4) * (16 / ES)) * ES));
        }
    };
    auto deposit = [&]() {  // ... into LDS: pixel records of two neighbouring pixels x 8 channels, filter pieces as they are
#pragma unroll
        for (int s = 0; s < 5; s++) {
            const int q = tid + s * 512;
            const int o = q / 36, part = q % 36;
            if (q < MT * 36) *(u32x4 *)(smem + o * AROW + ((part & ~3) | ((part & 3) ^ ((o >> 1) & 3))) * 16) = piece[s];
        }
#pragma unroll
        for (int s = 0; s < UMAX; s++) {
            if (u_dst[s] >= 0) {
                if constexpr (ES == 2) {
                    u32x4 px0, px1;
#pragma unroll
                    for (int h = 0; h < 4; h++) {
                        px0[h] = __builtin_amdgcn_perm(d[s][2 * h + 1], d[s][2 * h], 0x05040100u);  // low halves: pixel 2 xp
                        px1[h] = __builtin_amdgcn_perm(d[s][2 * h + 1], d[s][2 * h], 0x07060302u);  // high halves: pixel 2 xp + 1
                    }
                    *(u32x4 *)(smem + u_dst[s]) = px0;
                    *(u32x4 *)(smem + u_dst[s] + PIX) = px1;
                } else {
                    *(u32x4 *)(smem + u_dst[s]) = u32x4{d[s][0], d[s][1], d[s][2], d[s][3]};  // one pixel, 4 channels
                }
            }
        }
    };

    request(0);
    for (int c0 = 0; c0 < p.C; c0 += CKT) {
        __syncthreads();  // the previous chunk's fragments have been read
        deposit();
        __syncthreads();
        if (c0 + CKT < p.C) request(c0 + CKT);  // the next chunk travels while this one is multiplied
        // ---- 9 taps x (2 x 4) MFMAs; operands swapped so that a lane ends up with 4 consecutive pixels of one channel.
        // Eighteen half taps (two pixel tiles each) in a software pipeline: the fragments of half tap h + 1 are requested
        // from LDS in front of the four MFMAs of half tap h, into the other register set.
        // (a wave whose 64 pixels all lie past the end of the image -- the last pixel block of an image -- has nothing to multiply)
        if (n0 + wn0 < p.HW) {
            u32x4 fa[2], fb[2][2];
            auto read_a = [&](int tap) {
#pragma unroll
                for (int i = 0; i < 2; i++) fa[i] = *(const u32x4 *)(smem + a_addr[i] + tap * 64);
            };
            auto read_b = [&](int tap, int jh, u32x4(&dst)[2]) {
                const uint32_t shift = (uint32_t)(((tap / 3) * WP + tap % 3) * PIX);
#pragma unroll
                for (int j = 0; j < 2; j++) dst[j] = *(const u32x4 *)(smem + b_addr[jh + j] + shift);
            };
            read_a(0);
            read_b(0, 0, fb[0]);
#pragma unroll
            for (int h = 0; h < 18; h++) {
                const int tap = h / 2, jh = (h % 2) * 2;
                if (h + 1 < 18) read_b((h + 1) / 2, ((h + 1) % 2) * 2, fb[(h + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        if constexpr (ES == 2) {
                            acc[i][jh + j] = Mma16<T>::mfma(fb[h & 1][j], fa[i], acc[i][jh + j]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)  // channel 4 lq + e of the chunk in both operands
                                acc[i][jh + j] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(fb[h & 1][j][e]), __uint_as_float(fa[i][e]),
                                                                                      acc[i][jh + j], 0, 0, 0);
                        }
                    }
                __builtin_amdgcn_sched_barrier(0);
                // (the filter fragments have one register set: the next tap's are requested behind this tap's last MFMAs)
                if (jh == 2 && tap + 1 < 9) read_a(tap + 1);
            }
        }
    }

    // ---- epilogue: lane holds channel o = l16 (per tile) and pixels 4 lq + 0..3 of each 16-pixel tile
    if constexpr (ES == 4) {
        // f32: a lane's four values are four consecutive pixels of a channel row, 16 bytes as they are (H * W % 4 == 0)
        float *const obase = (float *)p.out + ((int64_t)b * p.O + (int64_t)mb * MT) * p.HW;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            float *orow = obase + (int64_t)(wm0 + 16 * i + l16) * p.HW;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int n = n0 + wn0 + 16 * j + 4 * lq;
                if (n < p.HW) {
                    f32x4 v = acc[i][j];
                    if constexpr (ACC) v += *(const f32x4 *)(orow + n);
                    *(f32x4 *)(orow + n) = v;
                }
            }
        }
    } else {
        uint16_t *const obase = (uint16_t *)p.out + ((int64_t)b * p.O + (int64_t)mb * MT) * p.HW;
        if (p.HW % 8 == 0) {
            // 16 bytes per lane: two neighbouring pixel tiles trade halves between the lane rows (v_permlane16_swap), after
            // which lane row lq holds pixels 8 (lq / 2) + 0..7 of tile 2 jp + (lq & 1); a store instruction then writes 64
            // contiguous bytes of each of 16 channel rows instead of 32.  Overwriting, the packed pairs are traded (half as
            // many instructions); accumulating, the f32 values, which then meet the old ones before the one rounding.
#pragma unroll
            for (int i = 0; i < 2; i++) {
                uint16_t *orow = obase + (int64_t)(wm0 + 16 * i + l16) * p.HW;
#pragma unroll
                for (int jp = 0; jp < 2; jp++) {
                    const int n = n0 + wn0 + (2 * jp + (lq & 1)) * 16 + (lq >> 1) * 8;
                    u32x4 o;
                    if constexpr (ACC) {
                        float v[8];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(acc[i][2 * jp][e]), __float_as_uint(acc[i][2 * jp + 1][e]), false, false);
                            v[e] = __uint_as_float(r[0]);
                            v[4 + e] = __uint_as_float(r[1]);
                        }
                        if (n < p.HW) {
                            const u32x4 old = *(const u32x4 *)(orow + n);
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                o[e] = Mma16<T>::pack2(v[2 * e] + Mma16<T>::to_f32((uint16_t)(old[e] & 0xffffu)),
                                                       v[2 * e + 1] + Mma16<T>::to_f32((uint16_t)(old[e] >> 16)));
                        }
                    } else {
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const uint32_t lo = Mma16<T>::pack2(acc[i][2 * jp][2 * h], acc[i][2 * jp][2 * h + 1]);
                            const uint32_t hi = Mma16<T>::pack2(acc[i][2 * jp + 1][2 * h], acc[i][2 * jp + 1][2 * h + 1]);
                            const auto r = __builtin_amdgcn_permlane16_swap(lo, hi, false, false);
                            o[h] = r[0];
                            o[2 + h] = r[1];
                        }
                    }
                    if (n < p.HW) *(u32x4 *)(orow + n) = o;
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                uint16_t *orow = obase + (int64_t)(wm0 + 16 * i + l16) * p.HW;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int n = n0 + wn0 + 16 * j + 4 * lq;
                    if (n < p.HW) {  // HW % 4 == 0: all four pixels are in range
                        float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
                        if constexpr (ACC) {
                            const u32x2 old = *(const u32x2 *)(orow + n);
                            v[0] += Mma16<T>::to_f32((uint16_t)(old[0] & 0xffffu));
                            v[1] += Mma16<T>::to_f32((uint16_t)(old[0] >> 16));
                            v[2] += Mma16<T>::to_f32((uint16_t)(old[1] & 0xffffu));
                            v[3] += Mma16<T>::to_f32((uint16_t)(old[1] >> 16));
                        }
                        *(u32x2 *)(orow + n) = u32x2{Mma16<T>::pack2(v[0], v[1]), Mma16<T>::pack2(v[2], v[3])};
                    }
                }
            }
        }

    }
}

}  // namespace

bool conv3x3_supported(const Conv3x3Problem &c) {
    if (c.dtype != DT_F16 && c.dtype != DT_BF16 && c.dtype != DT_F32) return false;
    const int es = c.dtype == DT_F32 ? 4 : 2, ck = 64 / es;  // element bytes, channels per chunk
    if (c.batch < 1 || c.chan_in < ck || c.chan_in % ck || c.chan_out < MT || c.chan_out % MT) return false;
    if (c.w < 4 || c.w > 254 || c.w % 2 || c.h < 1 || ((int64_t)c.h * c.w) % 4) return false;
    const int64_t hw = (int64_t)c.h * c.w;
    if (hw < 128 || hw >= (1 << 24) || (int64_t)c.chan_in * hw * es >= (1ll << 31)) return false;  // byte offsets of an image fit 31 bits
    const uintptr_t out_mask = es == 4 ? 15u : 7u;
    if (((uintptr_t)c.img & 3u) || ((uintptr_t)c.out & out_mask) || ((uintptr_t)c.filters & (uintptr_t)(es - 1)) || ((uintptr_t)c.wt & 15u)) return false;
    const int band_rows = (int)std::min<int64_t>(c.h, (NT - 1) / c.w + 2) + 2;
    if ((size_t)A_BYTES + (size_t)band_rows * (c.w + 2) * PIX > 160 * 1024) return false;
    if (4 * band_rows * (c.w / 2) > 6 * 512) return false;  // units per chunk: at most six (f32: twelve) per thread
    return c.batch < 65536 && (hw + NT - 1) / NT < 65536;  // grid.z, grid.y
}

size_t conv3x3_filter_bytes(const Conv3x3Problem &c) { return (size_t)c.chan_out * 9 * c.chan_in * (c.dtype == DT_F32 ? 4 : 2); }

hipError_t launch_conv3x3(const Conv3x3Problem &c, hipStream_t stream) {
    if (!conv3x3_supported(c)) return hipErrorNotSupported;
    const int total = c.chan_out * 9 * c.chan_in;
    if (c.dtype == DT_F32)
        conv3x3_filters_kernel<uint32_t><<<(total + 255) / 256, 256, 0, stream>>>((const uint32_t *)c.filters, (uint32_t *)c.wt, c.chan_in, c.chan_out,
                                                                                 c.transposed_filters ? 1 : 0, total);
    else
        conv3x3_filters_kernel<uint16_t><<<(total + 255) / 256, 256, 0, stream>>>((const uint16_t *)c.filters, (uint16_t *)c.wt, c.chan_in, c.chan_out,
                                                                                 c.transposed_filters ? 1 : 0, total);
    Params p;
    p.img = c.img; p.wt = c.wt; p.out = c.out;
    p.C = c.chan_in; p.O = c.chan_out; p.H = c.h; p.W = c.w; p.HW = c.h * c.w;
    p.nblocks = (p.HW + NT - 1) / NT; p.mblocks = c.chan_out / MT;
    p.band_rows = (int)std::min<int64_t>(c.h, (NT - 1) / c.w + 2) + 2;
    const size_t lds = (size_t)A_BYTES + (size_t)p.band_rows * (c.w + 2) * PIX;
    const int per_row = c.dtype == DT_F32 ? c.w : c.w / 2;  // units of a band row
    p.magic_w = (uint32_t)(((1ull << 32) + c.w - 1) / c.w);
    p.magic_pairs = (uint32_t)(((1ull << 32) + per_row - 1) / per_row);
    const dim3 grid((unsigned)p.mblocks, (unsigned)p.nblocks, (unsigned)c.batch);
    const bool few = 4 * p.band_rows * (c.w / 2) <= 2 * 512, many = 4 * p.band_rows * (c.w / 2) > 4 * 512;  // (rows of 206+ pixels)
#define DFDX_CONV3(T, U, A)                                                                                            \
    do {                                                                                                               \
        static PerDevice attr_on;                                                                                      \
        std::atomic<int> &known = attr_on.here();                                                                      \
        if (known.load(std::memory_order_acquire) == 0) {                                                              \
            hipError_t e = hipFuncSetAttribute((const void *)conv3x3_kernel<T, U, A>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return e;                                                                             \
            known.store(1, std::memory_order_release);                                                                 \
        }                                                                                                              \
        conv3x3_kernel<T, U, A><<<grid, 512, lds, stream>>>(p);                                                        \
    } while (0)
#define DFDX_CONV3_U(T, A, UF, UM, UW)       \
    do {                                     \
        if (few) DFDX_CONV3(T, UF, A);       \
        else if (many) DFDX_CONV3(T, UW, A); \
        else DFDX_CONV3(T, UM, A);           \
    } while (0)
    if (c.dtype == DT_F16) {
        if (c.accumulate) DFDX_CONV3_U(_Float16, true, 2, 4, 6);
        else DFDX_CONV3_U(_Float16, false, 2, 4, 6);
    } else if (c.dtype == DT_BF16) {
        if (c.accumulate) DFDX_CONV3_U(__bf16, true, 2, 4, 6);
        else DFDX_CONV3_U(__bf16, false, 2, 4, 6);
    } else {
        if (c.accumulate) DFDX_CONV3_U(float, true, 4, 8, 12);
        else DFDX_CONV3_U(float, false, 4, 8, 12);
    }
#undef DFDX_CONV3_U
#undef DFDX_CONV3
    return hipGetLastError();
}

}  // namespace dfdx_rocm
