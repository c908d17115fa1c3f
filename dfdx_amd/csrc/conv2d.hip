// conv2d as unfold + batched GEMM: the images (forward) or the output gradients (backward) are unfolded into patch
// matrices by HBM-bound gather kernels, and every product is one call of the library's strided batched GEMM --
// filters with batch stride 0 over the images, groups as the second batch axis, the filter gradient as a GEMM
// that reduces over the batch.
#include "ctx_internal.h"

#include <initializer_list>
#include "elem.h"
#include "gemm_internal.h"
#include "conv3x3.h"

#include <cstring>

namespace dfdx_rocm {
namespace {

struct Op {  // dfdx_rocm_conv2d_op narrowed to 32 bits (validated on entry)
    int kernel, stride, padding, dilation, groups, batch, chan_in, chan_out, h_in, h_out, w_in, w_out;
};

// patches[b][c][k1][k2][oh][ow] = img[b][c][oh*stride + dilation*k1 - padding][ow*stride + dilation*k2 - padding],
// zero outside the image.  Unit stride, output width a multiple of the vector: one workgroup per (b, c) plane writes
// the K*K slabs of that plane; a thread owns a vector position (oh, V consecutive ow) and moves one window per tap --
// with a compile-time K the loads of all taps are in flight before the first store.  Each slab is `slab_stride`
// elements long: the rows of the patch matrix may be padded, and the padding is zeros.
template <typename T, int KS>
__global__ __launch_bounds__(256) void unfold_input_plane_kernel(Op op, const T *__restrict__ img, T *__restrict__ patches,
                                                                 int slab_stride) {
    constexpr int V = Elem<T>::VEC;
    const int K = KS ? KS : op.kernel, kk = K * K, n = op.h_out * op.w_out, wg = op.w_out / V;
    const T *plane = img + (int64_t)blockIdx.x * op.h_in * op.w_in;
    T *dst = patches + (int64_t)blockIdx.x * kk * slab_stride;
    if ((int)threadIdx.x < slab_stride - n)
        for (int tap = 0; tap < kk; tap++) Elem<T>::store(dst + (int64_t)tap * slab_stride + n + threadIdx.x, 0.0f);
    for (int g = threadIdx.x; g < n / V; g += 256) {
        const int oh = g / wg, ow = (g - oh * wg) * V;
#pragma unroll
        for (int k1 = 0; k1 < (KS ? KS : 1); k1++)
#pragma unroll
            for (int k2 = 0; k2 < (KS ? KS : 1); k2++) {
                if constexpr (KS != 0) {
                    const int y = oh + op.dilation * k1 - op.padding;
                    *(u32x4 *)(dst + (int64_t)(k1 * K + k2) * slab_stride + g * V) =
                        row_window<T>(plane + (int64_t)y * op.w_in, y >= 0 && y < op.h_in, ow + op.dilation * k2 - op.padding, op.w_in);
                }
            }
        if constexpr (KS == 0) {
            for (int tap = 0; tap < kk; tap++) {
                const int t1 = tap / K, t2 = tap - t1 * K;
                const int y = oh + op.dilation * t1 - op.padding;
                *(u32x4 *)(dst + (int64_t)tap * slab_stride + g * V) =
                    row_window<T>(plane + (int64_t)y * op.w_in, y >= 0 && y < op.h_in, ow + op.dilation * t2 - op.padding, op.w_in);
            }
        }
    }
}

// patches[b][o][k1][k2][y][x] = grad_out[b][o][oh][ow] where oh*stride = y + padding - dilation*k1 (likewise ow),
// zero when no output position reads image pixel (y, x) through filter tap (k1, k2).  Same mapping, unit stride.
template <typename T, int KS>
__global__ __launch_bounds__(256) void unfold_output_plane_kernel(Op op, const T *__restrict__ grad_out, T *__restrict__ patches,
                                                                  int slab_stride) {
    constexpr int V = Elem<T>::VEC;
    const int K = KS ? KS : op.kernel, kk = K * K, n = op.h_in * op.w_in, wg = op.w_in / V;
    const T *plane = grad_out + (int64_t)blockIdx.x * op.h_out * op.w_out;
    T *dst = patches + (int64_t)blockIdx.x * kk * slab_stride;
    if ((int)threadIdx.x < slab_stride - n)
        for (int tap = 0; tap < kk; tap++) Elem<T>::store(dst + (int64_t)tap * slab_stride + n + threadIdx.x, 0.0f);
    for (int g = threadIdx.x; g < n / V; g += 256) {
        const int y = g / wg, x = (g - y * wg) * V;
#pragma unroll
        for (int k1 = 0; k1 < (KS ? KS : 1); k1++)
#pragma unroll
            for (int k2 = 0; k2 < (KS ? KS : 1); k2++) {
                if constexpr (KS != 0) {
                    const int oh = y + op.padding - op.dilation * k1;
                    *(u32x4 *)(dst + (int64_t)(k1 * K + k2) * slab_stride + g * V) =
                        row_window<T>(plane + (int64_t)oh * op.w_out, oh >= 0 && oh < op.h_out, x + op.padding - op.dilation * k2, op.w_out);
                }
            }
        if constexpr (KS == 0) {
            for (int tap = 0; tap < kk; tap++) {
                const int t1 = tap / K, t2 = tap - t1 * K;
                const int oh = y + op.padding - op.dilation * t1;
                *(u32x4 *)(dst + (int64_t)tap * slab_stride + g * V) =
                    row_window<T>(plane + (int64_t)oh * op.w_out, oh >= 0 && oh < op.h_out, x + op.padding - op.dilation * t2, op.w_out);
            }
        }
    }
}

// The same two gathers for every other case (any stride, row widths that are not a multiple of the vector width, small
// images): a thread owns one 16-byte vector of the patch buffer, i.e. V consecutive positions of a flattened (row,
// column) slab -- they may straddle two rows -- whatever the slab size (a 7x7 slab would leave 249 of a workgroup's
// 256 threads idle); positions behind the slab's last element (the row padding) are zeros.
template <typename T>
__global__ __launch_bounds__(256) void unfold_input_flat_kernel(Op op, const T *img, T *patches, int slab_stride, uint32_t vectors, int fold) {
    constexpr int V = Elem<T>::VEC;
    const uint32_t item = blockIdx.x * 256 + threadIdx.x;  // one 16-byte vector of the patch buffer per thread
    if (item >= vectors) return;
    const uint32_t per_slab = (uint32_t)slab_stride / V, slab = item / per_slab;
    const int kk = op.kernel * op.kernel, n = op.h_out * op.w_out;
    const int k2 = (int)(slab % op.kernel), k1 = (int)((slab / op.kernel) % op.kernel);
    const T *plane = img + (int64_t)(slab / kk) * op.h_in * op.w_in;
    // slab = (image, channel, tap).  Folded: the slabs of one (channel, tap) lie next to each other, image after image --
    // the patch matrix of the whole batch, [C K K][batch * slab_stride]
    const uint32_t per_img = (uint32_t)(op.chan_in * kk);
    T *dst = patches + (int64_t)(fold ? (slab % per_img) * (uint32_t)op.batch + slab / per_img : slab) * slab_stride;
    {
        const int pos0 = (int)(item - slab * per_slab) * V;
        int oh = pos0 / op.w_out, ow = pos0 - oh * op.w_out;
        float v[V];
        const int y0 = oh * op.stride + op.dilation * k1 - op.padding, x0 = ow * op.stride + op.dilation * k2 - op.padding;
        if (op.stride == 1 && ow + V <= op.w_out && pos0 + V <= n && y0 >= 0 && y0 < op.h_in && x0 >= 0 && x0 + V <= op.w_in) {
            load_elems_unaligned<T, V>(plane + (int64_t)y0 * op.w_in + x0, v);
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int y = oh * op.stride + op.dilation * k1 - op.padding, x = ow * op.stride + op.dilation * k2 - op.padding;
                const bool ok = pos0 + i < n && y >= 0 && y < op.h_in && x >= 0 && x < op.w_in;
                v[i] = ok ? Elem<T>::load(plane + (int64_t)y * op.w_in + x) : 0.0f;
                if (++ow == op.w_out) { ow = 0; ++oh; }
            }
        }
        store_elems<T, V>(dst + pos0, v);
    }
}
template <typename T, bool UNIT_STRIDE>
__global__ __launch_bounds__(256) void unfold_output_flat_kernel(Op op, const T *grad_out, T *patches, int slab_stride, uint32_t vectors) {
    constexpr int V = Elem<T>::VEC;
    const uint32_t item = blockIdx.x * 256 + threadIdx.x;
    if (item >= vectors) return;
    const uint32_t per_slab = (uint32_t)slab_stride / V, slab = item / per_slab;
    const int kk = op.kernel * op.kernel, n = op.h_in * op.w_in;
    const int k2 = (int)(slab % op.kernel), k1 = (int)((slab / op.kernel) % op.kernel);
    const T *plane = grad_out + (int64_t)(slab / kk) * op.h_out * op.w_out;
    T *dst = patches + (int64_t)slab * slab_stride;
    {
        const int pos0 = (int)(item - slab * per_slab) * V;
        int y = pos0 / op.w_in, x = pos0 - y * op.w_in;
        float v[V];
        const int oh0 = y + op.padding - op.dilation * k1, ow0 = x + op.padding - op.dilation * k2;
        if (op.stride == 1 && x + V <= op.w_in && pos0 + V <= n && oh0 >= 0 && oh0 < op.h_out && ow0 >= 0 && ow0 + V <= op.w_out) {
            load_elems_unaligned<T, V>(plane + (int64_t)oh0 * op.w_out + ow0, v);
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int oh = y + op.padding - op.dilation * k1, ow = x + op.padding - op.dilation * k2;
                if constexpr (UNIT_STRIDE) {  // no divisions
                    const bool ok = pos0 + i < n && oh >= 0 && oh < op.h_out && ow >= 0 && ow < op.w_out;
                    v[i] = ok ? Elem<T>::load(plane + (int64_t)oh * op.w_out + ow) : 0.0f;
                } else {
                    const bool ok = pos0 + i < n && oh >= 0 && oh % op.stride == 0 && oh / op.stride < op.h_out && ow >= 0 &&
                                    ow % op.stride == 0 && ow / op.stride < op.w_out;
                    v[i] = ok ? Elem<T>::load(plane + (int64_t)(oh / op.stride) * op.w_out + ow / op.stride) : 0.0f;
                }
                if (++x == op.w_in) { x = 0; ++y; }
            }
        }
        store_elems<T, V>(dst + pos0, v);
    }
}

// Divisions of small numbers by launch-time constants go through a multiplication with ceil(2^32 / d): exact while
// n * d < 2^32.
struct SmallDivs {  // ceil(2^32 / d) for the divisors of unfold_small_kernel (0 where d = 1)
    uint32_t per_slab, kernel, kk, chan, width, stride, plane, bg;
};
__device__ __forceinline__ uint32_t small_div(uint32_t n, uint32_t d, uint32_t magic) { return d == 1 ? n : __umulhi(n, magic); }
inline uint32_t magic_of(int64_t d) { return d <= 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d); }

// Position-major gather of the image's patch matrix for strided windows (no window load applies there and the flat kernel
// pays its index arithmetic -- five integer divisions, the coordinates of V positions -- once per vector and tap: 236 MB of
// patches of a 7 x 7 / stride-2 layer took 184 us).  blockIdx.x = plane (image, channel), blockIdx.y = block of 256 vectors
// of output positions; a thread computes the source coordinates of its V positions once and walks the K x K taps, a tap only
// shifting them.  Patch layout as everywhere: [plane][tap][slab_stride], zeros outside the image and behind a slab's end.
template <typename T>
__global__ __launch_bounds__(256) void unfold_input_taps_kernel(Op op, const T *img, T *patches, int slab_stride, uint32_t magic_w) {
    constexpr int V = Elem<T>::VEC;
    struct __attribute__((aligned(16))) Vec { T e[V]; };
    const int per_slab = slab_stride / V, vec = blockIdx.y * 256 + threadIdx.x;
    if (vec >= per_slab) return;
    const int n = op.h_out * op.w_out, pos0 = vec * V;
    const T *plane = img + (int64_t)blockIdx.x * op.h_in * op.w_in;
    int row = (int)small_div(pos0, op.w_out, magic_w), col = pos0 - row * op.w_out;
    int by[V], bx[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        by[i] = pos0 + i < n ? row * op.stride - op.padding : -(1 << 20);
        bx[i] = col * op.stride - op.padding;
        if (++col == op.w_out) { col = 0; ++row; }
    }
    T *dst = patches + (int64_t)blockIdx.x * op.kernel * op.kernel * slab_stride + pos0;
    for (int k1 = 0; k1 < op.kernel; k1++)
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int dy = op.dilation * k1, dx = op.dilation * k2;
            Vec out;
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int y = by[i] + dy, x = bx[i] + dx;
                const bool ok = (unsigned)y < (unsigned)op.h_in && (unsigned)x < (unsigned)op.w_in;
                const T val = plane[ok ? y * op.w_in + x : 0];
                out.e[i] = ok ? val : (T)0.0f;
            }
            *(Vec *)dst = out;
            dst += slab_stride;
        }
}

// The same with the image rows a workgroup draws on staged in LDS.  blockIdx.y = band of `band_rows` output rows (whole
// vectors: band_rows * w_out is a multiple of V and at most 256 vectors); the band's windows reach image rows
// y_first = band_row0 * stride - padding ... y_first + in_rows - 1, which are copied into LDS with one coalesced read (rows
// outside the image as zeros), and the K*K*V gathers of a thread then hit LDS instead of the memory system: two-byte
// element loads, every one a request of its own to the texture path, were what the kernel above spends its time on
// (3 -> 64 channels, 7 x 7, stride 2 at 224 x 224: 166 us for 236 MB of patches).
template <typename T>
__global__ __launch_bounds__(256) void unfold_input_taps_lds_kernel(Op op, const T *img, T *patches, int slab_stride, int band_rows, int in_rows) {
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_rows_raw[];
    T *const staged = (T *)staged_rows_raw;
    constexpr int V = Elem<T>::VEC;
    struct __attribute__((aligned(16))) Vec { T e[V]; };
    const int row0 = blockIdx.y * band_rows, y_first = row0 * op.stride - op.padding;
    const T *plane = img + (int64_t)blockIdx.x * op.h_in * op.w_in;
    for (int i = threadIdx.x; i < in_rows * op.w_in; i += 256) {
        const int r = i / op.w_in, y = y_first + r;  // (a division per staged element: a few per thread)
        staged[i] = (unsigned)y < (unsigned)op.h_in ? plane[(int64_t)y * op.w_in + (i - r * op.w_in)] : (T)0.0f;
    }
    __syncthreads();
    const int n = op.h_out * op.w_out, pos0 = row0 * op.w_out + threadIdx.x * V;
    if (threadIdx.x * V >= band_rows * op.w_out || pos0 >= slab_stride) return;
    int row = threadIdx.x * V / op.w_out, col = threadIdx.x * V - row * op.w_out;  // inside the band
    int by[V], bx[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        by[i] = pos0 + i < n ? row * op.stride : (1 << 20);  // relative to y_first; positions behind the slab's last: zeros
        bx[i] = col * op.stride - op.padding;
        if (++col == op.w_out) { col = 0; ++row; }
    }
    T *dst = patches + (int64_t)blockIdx.x * op.kernel * op.kernel * slab_stride + pos0;
    for (int k1 = 0; k1 < op.kernel; k1++)
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int dy = op.dilation * k1, dx = op.dilation * k2;
            Vec out;
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int y = by[i] + dy, x = bx[i] + dx;
                const bool ok = y < in_rows && (unsigned)x < (unsigned)op.w_in;
                const T val = staged[ok ? y * op.w_in + x : 0];
                out.e[i] = ok ? val : (T)0.0f;
            }
            *(Vec *)dst = out;
            dst += slab_stride;
        }
}
// Band height of the staged form for this op (0: use another kernel): as many output rows as give the 256 threads a vector
// each, in whole vectors, with the image rows under them within 48 KB of LDS.
template <typename T> int staged_band_rows(const Op &op, int64_t slab_stride, int *in_rows) {
    constexpr int V = Elem<T>::VEC;
    int unit = 1;
    while ((unit * op.w_out) % V) unit++;  // rows per whole number of vectors
    int rows = (256 * V / op.w_out) / unit * unit;
    for (; rows >= unit; rows -= unit) {
        const int64_t need = ((int64_t)(rows - 1) * op.stride + (int64_t)op.dilation * (op.kernel - 1) + 1) * op.w_in * (int64_t)sizeof(T);
        if (need <= 48 * 1024) {
            *in_rows = (int)((rows - 1) * op.stride + op.dilation * (op.kernel - 1) + 1);
            return rows;
        }
    }
    return 0;
}

// The patch matrix of `op`'s images through the position-major kernels: rows staged in LDS where a band of them fits.
template <typename T> void launch_unfold_taps(const Op &op, const T *img, T *patches, int64_t slab_stride, hipStream_t stream) {
    constexpr int V = Elem<T>::VEC;
    int in_rows = 0;
    // (staging pays from 5 x 5 taps on: at 3 x 3 the two forms measure level, at 1 x 1 the copy into LDS is pure overhead)
    const int band = op.kernel >= 5 ? staged_band_rows<T>(op, slab_stride, &in_rows) : 0;
    const unsigned planes = (unsigned)(op.batch * op.chan_in);
    // bands over the whole slab: the positions behind the last output row (the slab's padding) are written too, as zeros
    const int64_t bands = band > 0 ? (slab_stride + (int64_t)band * op.w_out - 1) / ((int64_t)band * op.w_out) : 0;
    if (band > 0 && bands <= 65535) {
        const size_t lds = (size_t)in_rows * op.w_in * sizeof(T);
        unfold_input_taps_lds_kernel<T><<<dim3(planes, (unsigned)bands), 256, lds, stream>>>(op, img, patches, (int)slab_stride, band, in_rows);
    } else {
        unfold_input_taps_kernel<T><<<dim3(planes, (unsigned)((slab_stride / V + 255) / 256)), 256, 0, stream>>>(op, img, patches, (int)slab_stride, magic_of(op.w_out));
    }
}

// Position-major gather for small planes into the FOLDED patch matrix [chan K K][batch * slab_stride]: a thread owns one
// vector of positions of one plane and walks the K x K taps itself, so the index arithmetic of its V positions is done once
// for all taps (a tap only shifts the source coordinates) and a vector costs ~70 instructions instead of ~250.  A workgroup
// stages the planes of `cg` channels x `bg` consecutive images in LDS (one read of each) -- the same channels of consecutive
// images, because their pieces of a patch row lie next to each other: bg * slab_stride contiguous elements per row instead
// of one image's 112 bytes between the pieces of other workgroups.
// Input side: source = image, positions = output pixels, coordinate = pos * stride - padding + dilation * k.
// Output side (unit stride only): source = grad_out, positions = image pixels, coordinate = pos + padding - dilation * k.
template <typename T, bool OUTPUT_SIDE>
__global__ __launch_bounds__(256) void unfold_small_kernel(Op op, SmallDivs mg, const T *src, T *patches, int slab_stride, int cg, int bg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_raw[];
    T *const staged = (T *)staged_raw;
    constexpr int V = Elem<T>::VEC;
    struct __attribute__((aligned(16))) Vec { T e[V]; };
    const int src_h = OUTPUT_SIDE ? op.h_out : op.h_in, src_w = OUTPUT_SIDE ? op.w_out : op.w_in;
    const int pos_w = OUTPUT_SIDE ? op.w_in : op.w_out, n = OUTPUT_SIDE ? op.h_in * op.w_in : op.h_out * op.w_out;
    const int chan = OUTPUT_SIDE ? op.chan_out : op.chan_in;
    const int scale = OUTPUT_SIDE ? 1 : op.stride, origin = OUTPUT_SIDE ? op.padding : -op.padding;
    const int tap_step = OUTPUT_SIDE ? -op.dilation : op.dilation;
    const uint32_t per_slab = (uint32_t)slab_stride / V;
    const int kk = op.kernel * op.kernel, plane_elems = src_h * src_w;
    const int c0 = blockIdx.x * cg, b0 = blockIdx.y * bg;
    const int channels = min(cg, chan - c0), images = min(bg, op.batch - b0);
    // plane `w` of the workgroup = channel c0 + w / bg of image b0 + w % bg
    for (uint32_t i = threadIdx.x; i < (uint32_t)(channels * bg * plane_elems); i += 256) {
        const uint32_t w = small_div(i, plane_elems, mg.plane), e = i - w * plane_elems;
        const uint32_t cl = small_div(w, bg, mg.bg), bl = w - cl * bg;
        if ((int)bl < images) staged[i] = src[((int64_t)(b0 + bl) * chan + c0 + cl) * plane_elems + e];
    }
    __syncthreads();
    for (uint32_t item = threadIdx.x; item < (uint32_t)(channels * bg) * per_slab; item += 256) {
        const uint32_t w = small_div(item, per_slab, mg.per_slab);
        const uint32_t cl = small_div(w, bg, mg.bg), bl = w - cl * bg;
        if ((int)bl >= images) continue;
        const int pos0 = (int)(item - w * per_slab) * V;
        const T *plane = staged + w * plane_elems;
        int row = (int)small_div(pos0, pos_w, mg.width), col = pos0 - row * pos_w;
        int by[V], bx[V];
#pragma unroll
        for (int i = 0; i < V; i++) {
            by[i] = pos0 + i < n ? row * scale + origin : -(1 << 20);  // positions behind the slab's last: zeros
            bx[i] = col * scale + origin;
            if (++col == pos_w) { col = 0; ++row; }
        }
        // the slab of (channel, tap 0, image); a channel's taps are `batch` slabs apart
        T *dst = patches + ((int64_t)(c0 + cl) * kk * op.batch + b0 + bl) * slab_stride + pos0;
        for (int k1 = 0; k1 < op.kernel; k1++)
            for (int k2 = 0; k2 < op.kernel; k2++) {
                const int dy = tap_step * k1, dx = tap_step * k2;
                Vec out;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    const int y = by[i] + dy, x = bx[i] + dx;
                    const bool ok = (unsigned)y < (unsigned)src_h && (unsigned)x < (unsigned)src_w;
                    const T val = plane[ok ? y * src_w + x : 0];
                    out.e[i] = ok ? val : (T)0.0f;
                }
                *(Vec *)dst = out;
                dst += (int64_t)op.batch * slab_stride;
            }
    }
}
// Launch shape of unfold_small_kernel: bg = 8 images (fewer in a smaller batch), as many channels as give the 256 threads a
// vector each and fit 32 KB of LDS; false when a single plane does not fit.
template <typename T> bool small_unfold_shape(int64_t slab_stride, int64_t plane_elems, int batch, int *cg, int *bg, size_t *lds) {
    *bg = std::min(8, batch);
    const int64_t per_slab = slab_stride / Elem<T>::VEC;
    const int64_t by_work = std::max<int64_t>(1, 256 / (per_slab * *bg));
    const int64_t by_lds = (32 * 1024) / (plane_elems * (int64_t)sizeof(T) * *bg);
    if (by_lds < 1) return false;
    *cg = (int)std::min(by_work, by_lds);
    *lds = (size_t)(*cg * *bg * plane_elems) * sizeof(T);
    return true;
}

// filters (G*O/G, C/G, K, K) <-> transposed (G, C/G, O/G, K*K).  ADD_BACK: filters[..] += transposed[..].
template <typename T, bool ADD_BACK>
__global__ __launch_bounds__(256) void filter_transpose_kernel(Op op, T *filters, T *transposed, uint32_t magic_kk) {
    // blockIdx.x = output channel (all groups); a thread takes element j = (c, tap) of that channel's filter, which is
    // contiguous in `filters`: nothing is divided per element but j by K*K, through a multiplication
    const int kk = op.kernel * op.kernel, og = op.chan_out / op.groups, cg = op.chan_in / op.groups;
    const uint32_t j = blockIdx.y * 256 + threadIdx.x;
    if (j >= (uint32_t)(cg * kk)) return;
    const int row = blockIdx.x, g = row / og, o = row - g * og;
    const uint32_t c = kk == 1 ? j : __umulhi(j, magic_kk), tap = j - c * kk;
    T *f = filters + (int64_t)row * cg * kk + j;
    T *t = transposed + ((int64_t)(g * cg + c) * og + o) * kk + tap;
    if constexpr (ADD_BACK) Elem<T>::store(f, Elem<T>::load(f) + Elem<T>::load(t));
    else *t = *f;
}
// The same through LDS in tiles of 16 output x 16 input channels (whole tiles only): both sides are then read and written
// in runs of 16 K*K contiguous elements, where the kernel above leaves K*K-element pieces a whole filter row apart on the
// transposed side (512 -> 512 channels, 3 x 3: 8.8 us for 4.7 MB).  blockIdx = (tile of input channels, tile of output
// channels, group); dynamic LDS: 256 K*K elements.
template <typename T, bool ADD_BACK>
__global__ __launch_bounds__(256) void filter_transpose_tiled_kernel(Op op, T *filters, T *transposed, uint32_t magic_kk, uint32_t magic_16kk) {
    extern __shared__ __attribute__((aligned(16))) uint8_t tile_raw[];
    T *const tile = (T *)tile_raw;  // [16 output channels][16 input channels][K*K]
    const int kk = op.kernel * op.kernel, og = op.chan_out / op.groups, cg = op.chan_in / op.groups;
    const int run = 16 * kk, c0 = blockIdx.x * 16, o0 = blockIdx.y * 16, g = blockIdx.z;
    T *const f0 = filters + ((int64_t)(g * og + o0) * cg + c0) * kk;      // + ol * cg * kk + (cl * kk + tap)
    T *const t0 = transposed + ((int64_t)(g * cg + c0) * og + o0) * kk;   // + cl * og * kk + (ol * kk + tap)
    if constexpr (!ADD_BACK) {
        for (uint32_t i = threadIdx.x; i < (uint32_t)(16 * run); i += 256) {
            const uint32_t ol = __umulhi(i, magic_16kk), r = i - ol * run;
            tile[i] = f0[(int64_t)ol * cg * kk + r];
        }
    } else {
        for (uint32_t i = threadIdx.x; i < (uint32_t)(16 * run); i += 256) {
            const uint32_t cl = __umulhi(i, magic_16kk), r = i - cl * run;  // r = ol * kk + tap
            const uint32_t ol = kk == 1 ? r : __umulhi(r, magic_kk), tap = r - ol * kk;
            tile[ol * run + cl * kk + tap] = t0[(int64_t)cl * og * kk + r];
        }
    }
    __syncthreads();
    if constexpr (!ADD_BACK) {
        for (uint32_t i = threadIdx.x; i < (uint32_t)(16 * run); i += 256) {
            const uint32_t cl = __umulhi(i, magic_16kk), r = i - cl * run;
            const uint32_t ol = kk == 1 ? r : __umulhi(r, magic_kk), tap = r - ol * kk;
            t0[(int64_t)cl * og * kk + r] = tile[ol * run + cl * kk + tap];
        }
    } else {
        for (uint32_t i = threadIdx.x; i < (uint32_t)(16 * run); i += 256) {
            const uint32_t ol = __umulhi(i, magic_16kk), r = i - ol * run;
            T *f = f0 + (int64_t)ol * cg * kk + r;
            Elem<T>::store(f, Elem<T>::load(f) + Elem<T>::load(tile + i));
        }
    }
}

// Rows of `len` elements <-> rows padded to `padded` elements (zeros behind the data).  When the spatial size of a
// product (OH*OW forward, H*W backward) is not a multiple of the GEMM's vector width, the matrices on that side get
// padded rows in the patch buffer, so that the matrix-core kernels apply instead of the scalar fallback.
template <typename T> __global__ __launch_bounds__(256) void pad_rows_kernel(const T *src, T *dst, int len, int padded, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index into dst
    if (i >= total) return;
    const int64_t row = i / padded;
    const int col = (int)(i - row * padded);
    if (col < len) dst[i] = src[row * len + col];
    else Elem<T>::store(dst + i, 0.0f);
}
// The same in whole 16-byte vectors (len and padded multiples of the vector, aligned buffers): a thread per vector of dst.
template <typename T> __global__ __launch_bounds__(256) void pad_rows_vec_kernel(const T *src, T *dst, int len_v, int padded_v, int64_t total_v) {
    constexpr int V = Elem<T>::VEC;
    struct __attribute__((aligned(16))) Vec { T e[V]; };
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // vector index into dst
    if (i >= total_v) return;
    const int64_t row = i / padded_v;
    const int col = (int)(i - row * padded_v);
    Vec v;
    if (col < len_v) v = ((const Vec *)src)[row * len_v + col];
    else
#pragma unroll
        for (int e = 0; e < V; e++) v.e[e] = (T)0.0f;
    ((Vec *)dst)[i] = v;
}
template <typename T> void launch_pad_rows(const T *src, T *dst, int64_t len, int64_t padded, int64_t total, hipStream_t stream) {
    constexpr int V = Elem<T>::VEC;
    if (len % V == 0 && padded % V == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15u) == 0)
        pad_rows_vec_kernel<T><<<(unsigned)((total / V + 255) / 256), 256, 0, stream>>>(src, dst, (int)(len / V), (int)(padded / V), total / V);
    else pad_rows_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(src, dst, (int)len, (int)padded, total);
}
template <typename T> __global__ __launch_bounds__(256) void unpad_rows_kernel(const T *src, T *dst, int len, int padded, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index into dst
    if (i >= total) return;
    const int64_t row = i / len;
    dst[i] = src[row * padded + (i - row * len)];
}

// The two kernels that move an image-side tensor [batch][rows][len] into and out of the folded layout
// [rows][batch][padded] (padded < 256; zeros behind every row).  A thread handles one element of the tensor the kernel
// writes; the only per-lane divisions are of small numbers (an index inside the workgroup's run of 256 elements; the run's
// origin is divided once, on the scalar unit) and go through a multiplication.
struct FoldDivs { uint32_t len, padded, rows, batch; };  // ceil(2^32 / d), 0 for d = 1
template <typename T> __global__ __launch_bounds__(256) void unfold_rows_kernel(const T *src, T *dst, int len, int padded, int rows, int batch, FoldDivs mg, uint32_t total) {
    const uint32_t first = blockIdx.x * 256, i = first + threadIdx.x;  // index into dst [batch][rows][len]
    if (i >= total) return;
    const uint32_t line0 = first / (uint32_t)len, image0 = line0 / (uint32_t)rows;
    const uint32_t in_run = first - line0 * len + threadIdx.x;           // < 256 + len
    const uint32_t dl = small_div(in_run, len, mg.len), col = in_run - dl * len;
    const uint32_t row_in_image0 = line0 - image0 * rows + dl;           // < rows + 256
    const uint32_t db = small_div(row_in_image0, rows, mg.rows), r = row_in_image0 - db * rows, b = image0 + db;
    dst[i] = src[((int64_t)r * batch + b) * padded + col];
}
template <typename T> __global__ __launch_bounds__(256) void fold_rows_kernel(const T *src, T *dst, int len, int padded, int rows, int batch, FoldDivs mg, uint32_t total) {
    const uint32_t first = blockIdx.x * 256, i = first + threadIdx.x;  // index into dst [rows][batch][padded]
    if (i >= total) return;
    const uint32_t line0 = first / (uint32_t)padded, row0 = line0 / (uint32_t)batch;
    const uint32_t in_run = first - line0 * padded + threadIdx.x;        // < 256 + padded
    const uint32_t dl = small_div(in_run, padded, mg.padded), col = in_run - dl * padded;
    const uint32_t image_in_row0 = line0 - row0 * batch + dl;            // < batch + 256
    const uint32_t dr = small_div(image_in_row0, batch, mg.batch), b = image_in_row0 - dr * batch, r = row0 + dr;
    if (col < (uint32_t)len) dst[i] = src[((int64_t)b * rows + r) * len + col];
    else Elem<T>::store(dst + i, 0.0f);
}

constexpr size_t kPatchBudget = size_t(1) << 30;  // bytes of patches per batch chunk
inline size_t round256(size_t b) { return (b + 255) & ~size_t(255); }

template <typename T> unsigned grid_for(dfdx_rocm_ctx *ctx, uint64_t threads) {
    return (unsigned)std::min<uint64_t>((threads + 255) / 256, (uint64_t)ctx->compute_units * 32);
}

inline int narrow(const dfdx_rocm_conv2d_op *o, Op *op) {
    const size_t f[12] = {o->kernel, o->stride, o->padding, o->dilation, o->groups, o->batch,
                          o->chan_in, o->chan_out, o->h_in, o->h_out, o->w_in, o->w_out};
    for (size_t v : f)
        if (v >= (size_t(1) << 30)) return DFDX_ROCM_ERR_INVALID_ARG;
    *op = {(int)f[0], (int)f[1], (int)f[2], (int)f[3], (int)f[4], (int)f[5], (int)f[6], (int)f[7], (int)f[8], (int)f[9], (int)f[10], (int)f[11]};
    if (op->kernel < 1 || op->stride < 1 || op->dilation < 1 || op->groups < 1) return DFDX_ROCM_ERR_INVALID_ARG;
    if (op->chan_in % op->groups || op->chan_out % op->groups) return DFDX_ROCM_ERR_INVALID_ARG;
    // the output size must be the one the reference derives (conv2d/mod.rs:143-160)
    const int64_t span = (int64_t)op->dilation * (op->kernel - 1) + 1;
    if (op->h_in + 2ll * op->padding < span || op->w_in + 2ll * op->padding < span) return DFDX_ROCM_ERR_INVALID_ARG;
    if (op->h_out != (op->h_in + 2ll * op->padding - span) / op->stride + 1) return DFDX_ROCM_ERR_INVALID_ARG;
    if (op->w_out != (op->w_in + 2ll * op->padding - span) / op->stride + 1) return DFDX_ROCM_ERR_INVALID_ARG;
    return DFDX_ROCM_OK;
}

dfdx_rocm_gemm_desc blank_desc(int dtype, int64_t m, int64_t k, int64_t n) {
    dfdx_rocm_gemm_desc d;
    std::memset(&d, 0, sizeof(d));
    d.dtype = dtype;
    d.m = m; d.k = k; d.n = n;
    d.batch1 = 1; d.batch2 = 1;
    return d;
}

// Unit-stride forward convolutions of the 16-bit types without a patch matrix in memory: the GEMM kernel forms its B
// tiles from the image planes themselves (one window load per 8 pixels, zeros where the window leaves the image), so
// the K*K-fold copy of the image is neither written nor read back.  Returns false when the shape does not fit (the
// caller then unfolds as for every other case).  The backward pass keeps the patch matrix: the filter gradient needs
// it anyway, and reading it back for the image gradient costs less than forming the windows a second time (57 vs
// 81 us at 64 channels, 56x56).
template <typename T>
bool implicit_forward(dfdx_rocm_ctx *ctx, int dtype, const Op &op, const void *filters, const void *img, void *out, int *rc) {
    if (sizeof(T) != 2 || op.stride != 1) return false;
    // narrow rows that are not a multiple of 8 pixels wide make half of the window loads straddle two rows and leave
    // much of a tile past the last pixel: 14x14 runs 118 us this way against 74 us through the patch matrix
    if (op.w_out % 8 != 0 && op.w_out < 24) return false;
    const int64_t kk = (int64_t)op.kernel * op.kernel, hw = (int64_t)op.h_in * op.w_in, ohw = (int64_t)op.h_out * op.w_out;
    const int64_t cg = op.chan_in / op.groups, og = op.chan_out / op.groups;
    GemmProblem g{};  // out (B, G, O/G, OH*OW) = filters (G, O/G, C/G*K*K) . patches of img
    g.dtype = dtype == DFDX_ROCM_F16 ? DT_F16 : DT_BF16;
    g.m = og; g.k = cg * kk; g.n = ohw;
    g.nb1 = op.batch; g.nb2 = op.groups;
    g.a = filters; g.a_rs = g.k; g.a_cs = 1; g.a_b1 = 0; g.a_b2 = g.m * g.k;
    g.b = img; g.b_b1 = op.chan_in * hw; g.b_b2 = cg * hw;
    g.c = out; g.c_rs = ohw; g.c_cs = 1; g.c_b1 = op.chan_out * ohw; g.c_b2 = og * ohw;
    g.compute_units = ctx->compute_units;
    ConvPatches cv{};
    cv.taps = (int)kk; cv.ksize = op.kernel;
    cv.w_dst = op.w_out; cv.h_src = op.h_in; cv.w_src = op.w_in; cv.plane = hw;
    cv.off_y = cv.off_x = -op.padding; cv.step_y = cv.step_x = op.dilation;
    const hipError_t e = launch_mfma16_conv(g, cv, ctx->compute_units, ctx->stream);
    if (e == hipErrorNotSupported) return false;
    *rc = (int)e;
    return true;
}

// 3 x 3 filters at unit stride with padding 1, f16 / bf16 / f32, channel counts in whole chunks: the kernel that keeps a band
// of the image in LDS and reads every tap's operand from it (conv3x3.hip).  The filters go through the patch buffer in
// the order that kernel wants.
template <typename T>
bool tiled3x3_forward(dfdx_rocm_ctx *ctx, int dtype, const Op &op, const void *filters, const void *img, void *out, int *rc) {
    if (sizeof(T) > 4 || op.kernel != 3 || op.stride != 1 || op.padding != 1 || op.dilation != 1 || op.groups != 1) return false;
    if (op.h_out != op.h_in || op.w_out != op.w_in) return false;
    Conv3x3Problem c{};
    c.dtype = dtype == DFDX_ROCM_F16 ? DT_F16 : dtype == DFDX_ROCM_BF16 ? DT_BF16 : DT_F32;
    c.batch = op.batch; c.chan_in = op.chan_in; c.chan_out = op.chan_out; c.h = op.h_in; c.w = op.w_in;
    c.img = img; c.filters = filters; c.out = out;
    c.wt = (void *)16;  // any aligned address: the real one needs the lock below
    if (!conv3x3_supported(c)) return false;
    // Small images in a small batch give that kernel fewer workgroups (64 output channels x 256 pixels x image) than the chip
    // has compute units; one product over the folded batch fills it (f32, batch 32, 256 -> 256 at 14 x 14: 158 us here)
    const int64_t hw = (int64_t)op.h_in * op.w_in, blocks = (int64_t)(op.chan_out / 64) * ((hw + 255) / 256) * op.batch;
    if (blocks < ctx->compute_units && hw < 256 && op.batch > 1) return false;
    CtxLock lock(ctx->mu);  // the patch buffer is shared by every conv2d call on this context
    if ((*rc = ensure_patches(ctx, round256(conv3x3_filter_bytes(c))))) return true;
    c.wt = ctx->patches;
    const hipError_t e = launch_conv3x3(c, ctx->stream);
    if (e == hipErrorNotSupported) return false;
    *rc = (int)e;
    return true;
}

// ---- depthwise convolutions (one input channel per group: filters [G * M][1][K][K]) ---------------------------------------
// As products these are G * batch multiplications of an M x K*K matrix with K*K rows of patches -- 8192 launches' worth of
// 1 x 9 x 784 for 128 channels at 28 x 28 (0.43 ms forward, 4.7 ms backward through the batched GEMM).  They are bound by
// the bytes of the image and the output instead, so each is computed directly, one thread per element, f32 sums, one rounding:
//   forward:   out[b][o][oh][ow]  = sum over taps of filters[o][tap] * img[b][o / M][oh s - p + d k1][ow s - p + d k2]
//   grad_img:  grad_img[b][g][y][x] += sum over m, taps whose window position is whole: filters[g M + m][tap] * grad_out[b][g M + m][oh][ow]
//   grad_filters[o][tap] += sum over b, oh, ow of grad_out[b][o][oh][ow] * img[b][o / M][...]   (one workgroup per output
//                           channel, a fixed summation order: deterministic)
// blockIdx.x = plane, blockIdx.y = block of 256 positions.
template <typename T>
__global__ __launch_bounds__(256) void depthwise_forward_kernel(Op op, const T *img, const T *filters, T *out, uint32_t magic_w) {
    const int n = op.h_out * op.w_out, pos = blockIdx.y * 256 + threadIdx.x;
    if (pos >= n) return;
    const int mult = op.chan_out / op.groups, b = blockIdx.x / op.chan_out, o = blockIdx.x - b * op.chan_out;
    const int oh = (int)small_div(pos, op.w_out, magic_w), ow = pos - oh * op.w_out;
    const T *plane = img + ((int64_t)b * op.chan_in + o / mult) * op.h_in * op.w_in;
    const T *f = filters + (int64_t)o * op.kernel * op.kernel;
    float acc = 0.0f;
    for (int k1 = 0; k1 < op.kernel; k1++) {
        const int y = oh * op.stride - op.padding + op.dilation * k1;
        if ((unsigned)y >= (unsigned)op.h_in) continue;
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int x = ow * op.stride - op.padding + op.dilation * k2;
            if ((unsigned)x < (unsigned)op.w_in) acc += Elem<T>::load(f + k1 * op.kernel + k2) * Elem<T>::load(plane + y * op.w_in + x);
        }
    }
    Elem<T>::store(out + (int64_t)blockIdx.x * n + pos, acc);
}
template <typename T>
__global__ __launch_bounds__(256) void depthwise_grad_img_kernel(Op op, const T *filters, const T *grad_out, T *grad_img, uint32_t magic_w, uint32_t magic_s,
                                                                 bool fresh) {
    const int hw = op.h_in * op.w_in, pos = blockIdx.y * 256 + threadIdx.x;
    if (pos >= hw) return;
    const int mult = op.chan_out / op.groups, b = blockIdx.x / op.chan_in, g = blockIdx.x - b * op.chan_in;
    const int y = (int)small_div(pos, op.w_in, magic_w), x = pos - y * op.w_in, kk = op.kernel * op.kernel, n = op.h_out * op.w_out;
    float acc = 0.0f;
    for (int k1 = 0; k1 < op.kernel; k1++) {
        const int ty = y + op.padding - op.dilation * k1;
        if (ty < 0) break;
        const int oh = (int)small_div(ty, op.stride, magic_s);
        if (oh * op.stride != ty || oh >= op.h_out) continue;
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int tx = x + op.padding - op.dilation * k2;
            if (tx < 0) break;
            const int ow = (int)small_div(tx, op.stride, magic_s);
            if (ow * op.stride != tx || ow >= op.w_out) continue;
            for (int m = 0; m < mult; m++) {
                const int o = g * mult + m;
                acc += Elem<T>::load(filters + (int64_t)o * kk + k1 * op.kernel + k2) *
                       Elem<T>::load(grad_out + ((int64_t)b * op.chan_out + o) * n + oh * op.w_out + ow);
            }
        }
    }
    T *dst = grad_img + (int64_t)blockIdx.x * hw + pos;
    Elem<T>::store(dst, (fresh ? 0.0f : Elem<T>::load(dst)) + acc);
}
template <typename T>
__global__ __launch_bounds__(256) void depthwise_grad_filters_kernel(Op op, const T *img, const T *grad_out, T *grad_filters, uint32_t magic_w) {
    __shared__ float part[4];
    const int o = blockIdx.x, mult = op.chan_out / op.groups, n = op.h_out * op.w_out, hw = op.h_in * op.w_in;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    for (int k1 = 0; k1 < op.kernel; k1++)
        for (int k2 = 0; k2 < op.kernel; k2++) {
            float acc = 0.0f;
            for (int b = 0; b < op.batch; b++) {
                const T *go = grad_out + ((int64_t)b * op.chan_out + o) * n;
                const T *plane = img + ((int64_t)b * op.chan_in + o / mult) * hw;
                for (int pos = threadIdx.x; pos < n; pos += 256) {
                    const int oh = (int)small_div(pos, op.w_out, magic_w), ow = pos - oh * op.w_out;
                    const int y = oh * op.stride - op.padding + op.dilation * k1, x = ow * op.stride - op.padding + op.dilation * k2;
                    if ((unsigned)y < (unsigned)op.h_in && (unsigned)x < (unsigned)op.w_in)
                        acc += Elem<T>::load(go + pos) * Elem<T>::load(plane + y * op.w_in + x);
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);  // the same tree whatever the timing
            __syncthreads();  // (the previous tap's partial sums have been read)
            if (lane == 0) part[wave] = acc;
            __syncthreads();
            if (threadIdx.x == 0) {
                T *dst = grad_filters + (int64_t)o * op.kernel * op.kernel + k1 * op.kernel + k2;
                Elem<T>::store(dst, Elem<T>::load(dst) + ((part[0] + part[1]) + (part[2] + part[3])));
            }
        }
}
// The same with a compile-time kernel size: a thread keeps all K*K sums and visits every (image, position) of its share
// once -- one load of grad_out and one division per position instead of one per position and tap -- and `slices` workgroups
// share the images of a channel; their sums meet in `partial` [O][slices][K*K] and the last line below adds them in slice
// order (deterministic).  grid = (O, slices).
template <typename T, int K>
__global__ __launch_bounds__(256) void depthwise_grad_filters_fixed_kernel(Op op, const T *img, const T *grad_out, float *partial, uint32_t magic_w) {
    constexpr int KK = K * K;
    __shared__ float part[4][KK];
    const int o = blockIdx.x, slices = gridDim.y, mult = op.chan_out / op.groups, n = op.h_out * op.w_out, hw = op.h_in * op.w_in;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    float acc[KK];
#pragma unroll
    for (int t = 0; t < KK; t++) acc[t] = 0.0f;
    for (int b = blockIdx.y; b < op.batch; b += slices) {
        const T *go = grad_out + ((int64_t)b * op.chan_out + o) * n;
        const T *plane = img + ((int64_t)b * op.chan_in + o / mult) * hw;
        for (int pos = threadIdx.x; pos < n; pos += 256) {
            const int oh = (int)small_div(pos, op.w_out, magic_w), ow = pos - oh * op.w_out;
            const float g = Elem<T>::load(go + pos);
            const int y0 = oh * op.stride - op.padding, x0 = ow * op.stride - op.padding;
#pragma unroll
            for (int k1 = 0; k1 < K; k1++) {
                const int y = y0 + op.dilation * k1;
#pragma unroll
                for (int k2 = 0; k2 < K; k2++) {
                    const int x = x0 + op.dilation * k2;
                    const bool ok = (unsigned)y < (unsigned)op.h_in && (unsigned)x < (unsigned)op.w_in;
                    acc[k1 * K + k2] += ok ? g * Elem<T>::load(plane + y * op.w_in + x) : 0.0f;
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < KK; t++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc[t] += __shfl_xor(acc[t], off, 64);
        if (lane == 0) part[wave][t] = acc[t];
    }
    __syncthreads();
    if (threadIdx.x < KK) partial[((int64_t)o * slices + blockIdx.y) * KK + threadIdx.x] =
        (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
}
// The 3 x 3 / unit stride / unit dilation case of the kernel above in quads of positions: four grad_out values of a row
// and the 3 x 6 image pixels under them, 18 + 4 loads for 36 multiplications.  Same slices, same reduction, same `partial`.
template <typename T>
__global__ __launch_bounds__(256) void depthwise3x3_grad_filters_kernel(Op op, const T *img, const T *grad_out, float *partial, uint32_t magic_quads) {
    __shared__ float part[4][9];
    const int o = blockIdx.x, slices = gridDim.y, mult = op.chan_out / op.groups, n = op.h_out * op.w_out, hw = op.h_in * op.w_in;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, quads = (op.w_out + 3) / 4;
    float acc[9];
#pragma unroll
    for (int t = 0; t < 9; t++) acc[t] = 0.0f;
    for (int b = blockIdx.y; b < op.batch; b += slices) {
        const T *go = grad_out + ((int64_t)b * op.chan_out + o) * n;
        const T *plane = img + ((int64_t)b * op.chan_in + o / mult) * hw;
        for (int item = threadIdx.x; item < op.h_out * quads; item += 256) {
            const int oh = (int)small_div(item, quads, magic_quads), ow0 = (item - oh * quads) * 4;
            float g[4];
#pragma unroll
            for (int i = 0; i < 4; i++) g[i] = ow0 + i < op.w_out ? Elem<T>::load(go + oh * op.w_out + ow0 + i) : 0.0f;
#pragma unroll
            for (int a = 0; a < 3; a++) {
                const int y = oh - op.padding + a;
                if ((unsigned)y >= (unsigned)op.h_in) continue;
                float v[6];
#pragma unroll
                for (int j = 0; j < 6; j++) {
                    const int x = ow0 - op.padding + j;
                    v[j] = (unsigned)x < (unsigned)op.w_in ? Elem<T>::load(plane + y * op.w_in + x) : 0.0f;
                }
#pragma unroll
                for (int bb = 0; bb < 3; bb++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[a * 3 + bb] += g[i] * v[i + bb];
            }
        }
    }
#pragma unroll
    for (int t = 0; t < 9; t++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc[t] += __shfl_xor(acc[t], off, 64);
        if (lane == 0) part[wave][t] = acc[t];
    }
    __syncthreads();
    if (threadIdx.x < 9) partial[((int64_t)o * slices + blockIdx.y) * 9 + threadIdx.x] =
        (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
}
template <typename T> __global__ __launch_bounds__(256) void depthwise_grad_filters_add_kernel(const float *partial, T *grad_filters, int slices, int kk, int total) {
    const int i = blockIdx.x * 256 + threadIdx.x;  // (o, tap)
    if (i >= total) return;
    const int o = i / kk, t = i - o * kk;
    float sum = 0.0f;
    for (int s = 0; s < slices; s++) sum += partial[((int64_t)o * slices + s) * kk + t];
    Elem<T>::store(grad_filters + i, Elem<T>::load(grad_filters + i) + sum);
}

// 3 x 3 depthwise filters at unit stride and dilation, forward and image gradient in one kernel: both are
//   dst[y][x] (+)= sum over a, b of wf[a][b] * src[y - q + a][x - q + b]
// (forward: dst = out, src = img, wf = the filter, q = padding; gradient: dst = grad_img, src = grad_out, wf = the filter
// turned by 180 degrees, q = 2 - padding, summed over the group's output channels).  A thread computes four neighbouring dst
// pixels of a row from the 3 x 6 src pixels under them -- 18 loads for 36 multiplications instead of 36 -- and no index is
// divided per tap.  blockIdx.x = dst plane, blockIdx.y = block of 256 quads.
template <typename T, bool GRAD>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(Op op, const T *src, const T *filters, T *dst, uint32_t magic_quads, bool fresh) {
    const int dh = GRAD ? op.h_in : op.h_out, dw = GRAD ? op.w_in : op.w_out, sh = GRAD ? op.h_out : op.h_in, sw = GRAD ? op.w_out : op.w_in;
    const int quads = (dw + 3) / 4, item = blockIdx.y * 256 + threadIdx.x;
    if (item >= dh * quads) return;
    const int y = (int)small_div(item, quads, magic_quads), x0 = (item - y * quads) * 4;
    const int mult = op.chan_out / op.groups, q = GRAD ? 2 - op.padding : op.padding;
    const int dchan = GRAD ? op.chan_in : op.chan_out, b = blockIdx.x / dchan, ch = blockIdx.x - b * dchan;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int m = 0; m < (GRAD ? mult : 1); m++) {
        const int o = GRAD ? ch * mult + m : ch;                 // the filter, and (gradient) the src plane
        const int schan = GRAD ? o : ch / mult;
        const T *plane = src + ((int64_t)b * (GRAD ? op.chan_out : op.chan_in) + schan) * sh * sw;
        float w[9];
#pragma unroll
        for (int t = 0; t < 9; t++) w[t] = Elem<T>::load(filters + (int64_t)o * 9 + (GRAD ? 8 - t : t));
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const int sy = y - q + a;
            if ((unsigned)sy >= (unsigned)sh) continue;
            float v[6];
#pragma unroll
            for (int j = 0; j < 6; j++) {
                const int sx = x0 - q + j;
                v[j] = (unsigned)sx < (unsigned)sw ? Elem<T>::load(plane + sy * sw + sx) : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int bb = 0; bb < 3; bb++) acc[i] += w[a * 3 + bb] * v[i + bb];
        }
    }
    T *out = dst + (int64_t)blockIdx.x * dh * dw + y * dw + x0;
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (x0 + i < dw) Elem<T>::store(out + i, ((GRAD && !fresh) ? Elem<T>::load(out + i) : 0.0f) + acc[i]);
}

inline bool depthwise(const Op &op) {
    return op.groups > 1 && op.chan_in == op.groups && op.chan_out % op.groups == 0 && (int64_t)op.h_in * op.w_in <= 65535ll * 256 &&
           (int64_t)op.h_out * op.w_out <= 65535ll * 256 && (int64_t)op.h_in * op.w_in * std::max(op.w_in, op.stride) < (1ll << 32);
}

template <typename T>
int forward_t(dfdx_rocm_ctx *ctx, int dtype, Op op, const void *img, const void *filters, void *out) {
    constexpr int V = Elem<T>::VEC;
    const int64_t kk = (int64_t)op.kernel * op.kernel, n = (int64_t)op.h_out * op.w_out;
    const int64_t np = (n + V - 1) / V * V;  // row length of the patch matrix (and of a padded output)
    const int64_t m = op.chan_out / op.groups, k = (op.chan_in / op.groups) * kk;
    const int64_t per_image = (int64_t)op.chan_in * kk * np;  // patch elements of one image
    if (per_image == 0 || m == 0) return DFDX_ROCM_OK;
    if (depthwise(op) && (int64_t)op.batch * op.chan_out < (1ll << 31)) {
        if (op.kernel == 3 && op.stride == 1 && op.dilation == 1 && op.padding <= 2) {
            const int quads = (op.w_out + 3) / 4;
            depthwise3x3_kernel<T, false><<<dim3((unsigned)(op.batch * op.chan_out), (unsigned)((op.h_out * quads + 255) / 256)), 256, 0, ctx->stream>>>(
                op, (const T *)img, (const T *)filters, (T *)out, magic_of(quads), false);
            return (int)hipGetLastError();
        }
        depthwise_forward_kernel<T><<<dim3((unsigned)(op.batch * op.chan_out), (unsigned)((n + 255) / 256)), 256, 0, ctx->stream>>>(
            op, (const T *)img, (const T *)filters, (T *)out, magic_of(op.w_out));
        return (int)hipGetLastError();
    }
    if (per_image >= (1ll << 31) || (int64_t)op.chan_out * np >= (1ll << 31)) return DFDX_ROCM_ERR_UNSUPPORTED;
    if (op.kernel > 1) {  // (1x1 filters have no patch matrix to avoid: see `pointwise` below)
        int rc = 0;
        if (tiled3x3_forward<T>(ctx, dtype, op, filters, img, out, &rc)) return rc;
        if (implicit_forward<T>(ctx, dtype, op, filters, img, out, &rc)) return rc;
    }
    CtxLock lock(ctx->mu);  // the patch buffer is shared by every conv2d call on this context
    int64_t chunk = std::max<int64_t>(1, (int64_t)(kPatchBudget / sizeof(T)) / per_image);
    chunk = std::min<int64_t>(std::min<int64_t>(chunk, op.batch), ((1ll << 31) - 1) / per_image);
    const bool padded = np != n;  // the product goes to a padded copy of the output, which is then compacted
    // 1x1 filters at unit stride without padding: the patch matrix IS the image -- no gather, one product for the batch
    const bool pointwise = op.kernel == 1 && op.stride == 1 && op.padding == 0 && !padded && ((uintptr_t)img & 15u) == 0;
    if (pointwise) chunk = op.batch;
    // Small images (a 7 x 7 output is n = 49: a quarter of one 256-column tile per image) multiply as ONE product over the
    // batch: the patch matrix is written [C K K][batch * np], the product lands in [O][batch * np] and a small kernel
    // hands every image its rows.  The filters are then read once per tile row instead of once per image.
    const bool fold = !pointwise && op.groups == 1 && np < 256 && op.batch > 1 && op.chan_in <= 32768 && op.chan_out <= 32768 &&
                      chunk <= 32768 && chunk * std::max(op.chan_in, op.chan_out) * np < (1ll << 31);
    const size_t patch_bytes = pointwise ? 0 : round256((size_t)(chunk * per_image) * sizeof(T));
    const size_t out_bytes = (padded || fold) ? round256((size_t)(chunk * op.chan_out * np) * sizeof(T)) : 0;
    if (int rc = ensure_patches(ctx, patch_bytes + out_bytes)) return rc;
    T *patches = (T *)ctx->patches;
    T *out_p = (T *)((char *)ctx->patches + patch_bytes);
    // a workgroup per image plane when its K*K slabs give the 256 threads a few vectors each
    const bool planes = !fold && op.stride == 1 && op.w_out % V == 0 && op.w_in >= V && (n / V) * kk >= 512;
    for (int64_t b0 = 0; b0 < op.batch; b0 += chunk) {
        const int64_t nb = std::min<int64_t>(chunk, op.batch - b0);
        Op sub = op;
        sub.batch = (int)nb;
        const T *src = (const T *)img + b0 * op.chan_in * op.h_in * op.w_in;
        const unsigned slabs = (unsigned)(nb * op.chan_in * kk);
        if (pointwise) patches = const_cast<T *>(src);
        else if (planes && op.kernel == 3) unfold_input_plane_kernel<T, 3><<<slabs / 9, 256, 0, ctx->stream>>>(sub, src, patches, (int)np);
        else if (planes) unfold_input_plane_kernel<T, 0><<<(unsigned)(slabs / kk), 256, 0, ctx->stream>>>(sub, src, patches, (int)np);
        else {
            const uint32_t vectors = (uint32_t)(slabs * (np / V));  // < 2^28: the chunk's patches stay below 2^31 elements
            int cg = 0, bg = 0;
            size_t lds = 0;
            const int64_t plane_elems = (int64_t)op.h_in * op.w_in;
            if (fold && small_unfold_shape<T>(np, plane_elems, (int)nb, &cg, &bg, &lds)) {
                const SmallDivs mg{magic_of(np / V), magic_of(op.kernel), magic_of(kk), magic_of(op.chan_in), magic_of(op.w_out), magic_of(op.stride),
                                   magic_of(plane_elems), magic_of(bg)};
                unfold_small_kernel<T, false><<<dim3((unsigned)((op.chan_in + cg - 1) / cg), (unsigned)((nb + bg - 1) / bg)), 256, lds, ctx->stream>>>(
                    sub, mg, src, patches, (int)np, cg, bg);
            }
            else if (!fold && op.stride > 1 && np / V >= 64 && np / V <= 65535ll * 256 && n * op.w_out < (1ll << 32))
                launch_unfold_taps<T>(sub, src, patches, np, ctx->stream);
            else unfold_input_flat_kernel<T><<<(vectors + 255) / 256, 256, 0, ctx->stream>>>(sub, src, patches, (int)np, vectors, fold ? 1 : 0);
        }
        HIP_TRY(hipGetLastError());
        T *dst = (T *)out + b0 * op.chan_out * n;
        if (fold) {  // filters (O, C*K*K) . patches (C*K*K, B * np) -> (O, B * np)
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, nb * np);
            d.a = filters; d.a_rs = k; d.a_cs = 1;
            d.b = patches; d.b_rs = nb * np; d.b_cs = 1;
            d.c = out_p; d.c_rs = nb * np; d.c_cs = 1;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
            const int64_t total = nb * op.chan_out * n;
            const FoldDivs fd{magic_of(n), magic_of(np), magic_of(op.chan_out), magic_of(nb)};
            unfold_rows_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(out_p, dst, (int)n, (int)np, op.chan_out, (int)nb, fd, (uint32_t)total);
            HIP_TRY(hipGetLastError());
            continue;
        }
        // filters (G, O/G, C/G*K*K) . patches (B, G, C/G*K*K, OH*OW) -> out (B, G, O/G, OH*OW)
        dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, np);
        d.batch1 = nb; d.batch2 = op.groups;
        d.a = filters; d.a_rs = k; d.a_cs = 1; d.a_b1 = 0; d.a_b2 = m * k;
        d.b = patches; d.b_rs = np; d.b_cs = 1; d.b_b1 = op.groups * k * np; d.b_b2 = k * np;
        d.c = padded ? out_p : dst; d.c_rs = np; d.c_cs = 1; d.c_b1 = op.chan_out * np; d.c_b2 = m * np;
        if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        if (padded) {
            const int64_t total = nb * op.chan_out * n;
            unpad_rows_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(out_p, dst, (int)n, (int)np, total);
            HIP_TRY(hipGetLastError());
        }
    }
    return DFDX_ROCM_OK;
}

// grad_img[b][c][y][x] += sum over the taps (k1, k2) whose window position is whole --
//   oh = (y + padding - dilation k1) / stride, ow = (x + padding - dilation k2) / stride, inside the output --
// of grad_patches[b][c K K + k1 K + k2][oh W_out + ow]: the gather form of col2im, one thread per image pixel, f32 sum,
// one rounding.  blockIdx.x = plane (b, c), blockIdx.y = block of 256 pixels.
template <typename T>
__global__ __launch_bounds__(256) void fold_patches_kernel(Op op, const T *grad_patches, T *grad_img, int slab_stride, uint32_t magic_w, uint32_t magic_s,
                                                           bool fresh) {
    const int hw = op.h_in * op.w_in, pos = blockIdx.y * 256 + threadIdx.x;
    if (pos >= hw) return;
    const int kk = op.kernel * op.kernel;
    const int y = (int)small_div(pos, op.w_in, magic_w), x = pos - y * op.w_in;
    const T *slabs = grad_patches + (int64_t)blockIdx.x * kk * slab_stride;
    float sum = 0.0f;
    for (int k1 = 0; k1 < op.kernel; k1++) {
        const int ty = y + op.padding - op.dilation * k1;
        if (ty < 0) break;  // (larger k1: further up)
        const int oh = (int)small_div(ty, op.stride, magic_s);
        if (oh * op.stride != ty || oh >= op.h_out) continue;
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int tx = x + op.padding - op.dilation * k2;
            if (tx < 0) break;
            const int ow = (int)small_div(tx, op.stride, magic_s);
            if (ow * op.stride != tx || ow >= op.w_out) continue;
            sum += Elem<T>::load(slabs + (int64_t)(k1 * op.kernel + k2) * slab_stride + oh * op.w_out + ow);
        }
    }
    T *dst = grad_img + (int64_t)blockIdx.x * hw + pos;
    Elem<T>::store(dst, (fresh ? 0.0f : Elem<T>::load(dst)) + sum);
}

// The same for stride S in cells of S x S image pixels, one thread per cell: every tap lands on exactly ONE pixel of a cell --
// row (dilation k1 - padding) mod S of it, from window row cell_row + (that row + padding - dilation k1) / S -- so no lane
// tests divisibility or divides, the lanes of a wave read consecutive window positions of one tap, and which pixel of the
// cell a tap belongs to is the same for the whole wave (the per-pixel kernel: 160 us for 64 x 64 planes of 56 x 56).
template <typename T, int S>
__global__ __launch_bounds__(256) void fold_patches_cells_kernel(Op op, const T *grad_patches, T *grad_img, int slab_stride, int cells_w, int cells, uint32_t magic_cw,
                                                                 bool fresh) {
    const int cell = blockIdx.y * 256 + threadIdx.x;
    if (cell >= cells) return;
    const int cy = (int)small_div(cell, cells_w, magic_cw), cx = cell - cy * cells_w;
    const T *slabs = grad_patches + (int64_t)blockIdx.x * op.kernel * op.kernel * slab_stride;
    float acc[S][S];
#pragma unroll
    for (int a = 0; a < S; a++)
#pragma unroll
        for (int b = 0; b < S; b++) acc[a][b] = 0.0f;
    for (int k1 = 0; k1 < op.kernel; k1++) {
        const int shift_y = op.dilation * k1 - op.padding;
        const int ry = ((shift_y % S) + S) % S;       // the cell row this tap row lands on
        const int oh = cy + (ry - shift_y) / S;       // exact: ry = shift_y (mod S)
        if (oh < 0 || oh >= op.h_out) continue;
        for (int k2 = 0; k2 < op.kernel; k2++) {
            const int shift_x = op.dilation * k2 - op.padding;
            const int rx = ((shift_x % S) + S) % S;
            const int ow = cx + (rx - shift_x) / S;
            const float v = (ow >= 0 && ow < op.w_out) ? Elem<T>::load(slabs + (int64_t)(k1 * op.kernel + k2) * slab_stride + oh * op.w_out + ow) : 0.0f;
#pragma unroll
            for (int a = 0; a < S; a++)
#pragma unroll
                for (int b = 0; b < S; b++) acc[a][b] += (a == ry && b == rx) ? v : 0.0f;
        }
    }
    T *plane = grad_img + (int64_t)blockIdx.x * op.h_in * op.w_in;
    if (S == 2 && op.w_in % 2 == 0 && (((uintptr_t)grad_img) & (2 * sizeof(T) - 1)) == 0) {
        // the two pixels of a cell row as one access (rows of even length: every pair is aligned)
        struct __attribute__((aligned(2 * sizeof(T)))) Pair { T e[2]; };
#pragma unroll
        for (int a = 0; a < S; a++) {
            const int y = cy * S + a;
            if (y < op.h_in) {
                Pair *q = (Pair *)(plane + y * op.w_in + cx * S);
                Pair v;
                if (fresh) v.e[0] = v.e[1] = (T)0.0f;
                else v = *q;
                Elem<T>::store(&v.e[0], Elem<T>::load(&v.e[0]) + acc[a][0]);
                Elem<T>::store(&v.e[1], Elem<T>::load(&v.e[1]) + acc[a][S - 1]);
                *q = v;
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < S; a++)
#pragma unroll
        for (int b = 0; b < S; b++) {
            const int y = cy * S + a, x = cx * S + b;
            if (y < op.h_in && x < op.w_in) Elem<T>::store(plane + y * op.w_in + x, (fresh ? 0.0f : Elem<T>::load(plane + y * op.w_in + x)) + acc[a][b]);
        }
}

// Backward pass of a strided convolution (and of one whose image has few channels).  The general form below gathers grad_out into a patch matrix over the INPUT
// positions, [O K K][H W]: at stride s only one position in s*s holds a value, so that matrix is s*s times larger than
// the forward one, mostly zeros, and both products multiply the zeros (64 -> 128 channels, 3 x 3, stride 2 at 56 x 56:
// 650 us against 61 forward; the 7 x 7 / stride-2 first layer of a residual network at 224 x 224: 27 ms against 0.34).
// Here both gradients come from the FORWARD patch matrix of the image, [C K K][OH OW], which has no such zeros:
//   grad_filters (O, C K K) += sum over images of grad_out (O, OH OW) . patches^T          -- in the filters' own layout
//   grad_patches (C K K, OH OW) = filters^T (C K K, O) . grad_out (O, OH OW)                -- filters transposed by strides
//   grad_img += the gather form of col2im of grad_patches (fold_patches_kernel)
// The image gradient's partial sums per tap are rounded to the element type before the taps are added (in f32, with the
// old gradient, one rounding): within the tolerance of the product, not bit-identical to the general form.
template <typename T>
int strided_backward(dfdx_rocm_ctx *ctx, int dtype, const Op &op, const void *img, void *grad_img, const void *filters, void *grad_filters,
                     const void *grad_out, bool fresh_img) {
    constexpr int V = Elem<T>::VEC;
    const int64_t kk = (int64_t)op.kernel * op.kernel, hw = (int64_t)op.h_in * op.w_in, ohw = (int64_t)op.h_out * op.w_out;
    const int64_t align = sizeof(T) == 2 ? 64 : V;  // OH*OW is the k of the filter-gradient product (split-k wants whole k tiles)
    const int64_t np = (ohw + align - 1) / align * align;
    const int64_t cg = op.chan_in / op.groups, og = op.chan_out / op.groups;
    const int64_t per_image = (int64_t)op.chan_in * kk * np;
    if (per_image == 0 || og == 0) return DFDX_ROCM_OK;
    if (per_image >= (1ll << 31) || (int64_t)op.chan_out * np >= (1ll << 31) || hw * op.w_in >= (1ll << 32) || hw > 65535ll * 256)
        return DFDX_ROCM_ERR_UNSUPPORTED;
    CtxLock lock(ctx->mu);  // the patch buffer is shared by every conv2d call on this context
    int64_t chunk = std::max<int64_t>(1, (int64_t)(kPatchBudget / sizeof(T)) / per_image);
    chunk = std::min<int64_t>(std::min<int64_t>(chunk, op.batch), ((1ll << 31) - 1) / std::max<int64_t>(per_image, (int64_t)op.chan_out * np));
    const bool padded = np != ohw;
    const size_t patch_bytes = round256((size_t)(chunk * per_image) * sizeof(T));
    const size_t go_bytes = padded ? round256((size_t)(chunk * op.chan_out * np) * sizeof(T)) : 0;
    if (int rc = ensure_patches(ctx, patch_bytes + go_bytes)) return rc;
    T *patches = (T *)ctx->patches;
    T *go_p = (T *)((char *)ctx->patches + patch_bytes);
    const uint32_t magic_w = magic_of(op.w_in), magic_s = magic_of(op.stride);
    for (int64_t b0 = 0; b0 < op.batch; b0 += chunk) {
        const int64_t nb = std::min<int64_t>(chunk, op.batch - b0);
        Op sub = op;
        sub.batch = (int)nb;
        const T *img_b = (const T *)img + b0 * op.chan_in * hw;
        T *grad_img_b = (T *)grad_img + b0 * op.chan_in * hw;
        const T *go = (const T *)grad_out + b0 * op.chan_out * ohw;
        const uint32_t vectors = (uint32_t)(nb * op.chan_in * kk * (np / V));
        if (np / V >= 64 && np / V <= 65535ll * 256 && ohw * op.w_out < (1ll << 32))
            launch_unfold_taps<T>(sub, img_b, patches, np, ctx->stream);
        else unfold_input_flat_kernel<T><<<(vectors + 255) / 256, 256, 0, ctx->stream>>>(sub, img_b, patches, (int)np, vectors, 0);
        HIP_TRY(hipGetLastError());
        if (padded) {
            const int64_t rows_p = nb * op.chan_out * np;
            launch_pad_rows<T>(go, go_p, ohw, np, rows_p, ctx->stream);
            HIP_TRY(hipGetLastError());
            go = go_p;
        }
        for (int g = 0; g < op.groups; g++) {  // grad_filters (O/G, C/G K K) += sum over images of grad_out . patches^T
            const int64_t m = og, k = np, n = cg * kk;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.accumulate = 1;
            d.reduce_batch = 1;
            d.batch1 = nb;
            d.a = go + g * m * k; d.a_rs = k; d.a_cs = 1; d.a_b1 = op.chan_out * k;
            d.b = patches + g * n * k; d.b_rs = 1; d.b_cs = k; d.b_b1 = per_image;
            d.c = (T *)grad_filters + g * m * n; d.c_rs = n; d.c_cs = 1;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
        {   // grad_patches (B, G, C/G K K, np) = filters^T (G, C/G K K, O/G) . grad_out (B, G, O/G, np), over the patches
            const int64_t m = cg * kk, k = og, n = np;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.batch1 = nb; d.batch2 = op.groups;
            d.a = filters; d.a_rs = 1; d.a_cs = m; d.a_b1 = 0; d.a_b2 = m * k;
            d.b = go; d.b_rs = n; d.b_cs = 1; d.b_b1 = op.chan_out * n; d.b_b2 = k * n;
            d.c = patches; d.c_rs = n; d.c_cs = 1; d.c_b1 = per_image; d.c_b2 = m * n;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
        if (op.stride >= 1 && op.stride <= 4) {
            const int S = op.stride, cells_w = (op.w_in + S - 1) / S, cells = cells_w * ((op.h_in + S - 1) / S);
            const dim3 grid((unsigned)(nb * op.chan_in), (unsigned)((cells + 255) / 256));
            const uint32_t magic_cw = magic_of(cells_w);
            if (S == 1) fold_patches_cells_kernel<T, 1><<<grid, 256, 0, ctx->stream>>>(sub, patches, grad_img_b, (int)np, cells_w, cells, magic_cw, fresh_img);
            else if (S == 2) fold_patches_cells_kernel<T, 2><<<grid, 256, 0, ctx->stream>>>(sub, patches, grad_img_b, (int)np, cells_w, cells, magic_cw, fresh_img);
            else if (S == 3) fold_patches_cells_kernel<T, 3><<<grid, 256, 0, ctx->stream>>>(sub, patches, grad_img_b, (int)np, cells_w, cells, magic_cw, fresh_img);
            else fold_patches_cells_kernel<T, 4><<<grid, 256, 0, ctx->stream>>>(sub, patches, grad_img_b, (int)np, cells_w, cells, magic_cw, fresh_img);
        } else {
            fold_patches_kernel<T><<<dim3((unsigned)(nb * op.chan_in), (unsigned)((hw + 255) / 256)), 256, 0, ctx->stream>>>(sub, patches, grad_img_b, (int)np,
                                                                                                                           magic_w, magic_s, fresh_img);
        }
        HIP_TRY(hipGetLastError());
    }
    return DFDX_ROCM_OK;
}

template <typename T>
int backward_t(dfdx_rocm_ctx *ctx, int dtype, Op op, const void *img, void *grad_img, const void *filters, void *grad_filters,
               const void *grad_out, bool fresh_img) {
    // `fresh_img`: grad_img counts as zero and must not be read.  The forms that store the image gradient in one pass take
    // that as "overwrite"; the others clear it first.
    constexpr int V = Elem<T>::VEC;
    const int64_t kk = (int64_t)op.kernel * op.kernel, hw = (int64_t)op.h_in * op.w_in, ohw = (int64_t)op.h_out * op.w_out;
    // Row length of the patch matrix and of the padded image-side matrices.  H*W is the n of the image-gradient
    // product and the k of the filter-gradient product; for the 16-bit types that k is rounded up to the k tile of the
    // split-k capable kernels -- a filter gradient has few output tiles and a long reduction over batch * H*W.
    const int64_t align = sizeof(T) == 2 ? 64 : V;
    const int64_t hp = (hw + align - 1) / align * align;
    const int64_t cg = op.chan_in / op.groups, og = op.chan_out / op.groups;
    const int64_t per_image = (int64_t)op.chan_out * kk * hp;
    const int64_t f_elems = (int64_t)op.groups * cg * og * kk;
    if (per_image == 0 || f_elems == 0 || ohw == 0) {  // nothing to add; a gradient taken over unfilled is cleared after all
        if (fresh_img && hw > 0) HIP_TRY(launch_zero_fill(grad_img, (size_t)op.batch * op.chan_in * hw * sizeof(T), ctx->compute_units, ctx->stream));
        return DFDX_ROCM_OK;
    }
    if (depthwise(op) && (int64_t)op.batch * op.chan_out < (1ll << 31)) {
        if (op.kernel == 3 && op.stride == 1 && op.dilation == 1 && op.padding <= 2) {
            const int quads = (op.w_in + 3) / 4;
            depthwise3x3_kernel<T, true><<<dim3((unsigned)(op.batch * op.chan_in), (unsigned)((op.h_in * quads + 255) / 256)), 256, 0, ctx->stream>>>(
                op, (const T *)grad_out, (const T *)filters, (T *)grad_img, magic_of(quads), fresh_img);
        } else {
            depthwise_grad_img_kernel<T><<<dim3((unsigned)(op.batch * op.chan_in), (unsigned)((hw + 255) / 256)), 256, 0, ctx->stream>>>(
                op, (const T *)filters, (const T *)grad_out, (T *)grad_img, magic_of(op.w_in), magic_of(op.stride), fresh_img);
        }
        HIP_TRY(hipGetLastError());
        if (op.kernel == 3 || op.kernel == 5 || op.kernel == 7) {
            // enough workgroups to fill the chip twice, at most one per image
            const int slices = (int)std::max<int64_t>(1, std::min<int64_t>(op.batch, (2 * (int64_t)ctx->compute_units + op.chan_out - 1) / op.chan_out));
            CtxLock lock(ctx->mu);  // the patch buffer is shared by every conv2d call on this context
            if (int rc = ensure_patches(ctx, round256((size_t)op.chan_out * slices * kk * sizeof(float)))) return rc;
            const dim3 grid((unsigned)op.chan_out, (unsigned)slices);
            const uint32_t mw = magic_of(op.w_out);
            if (op.kernel == 3 && op.stride == 1 && op.dilation == 1)
                depthwise3x3_grad_filters_kernel<T><<<grid, 256, 0, ctx->stream>>>(op, (const T *)img, (const T *)grad_out, (float *)ctx->patches, magic_of((op.w_out + 3) / 4));
            else if (op.kernel == 3) depthwise_grad_filters_fixed_kernel<T, 3><<<grid, 256, 0, ctx->stream>>>(op, (const T *)img, (const T *)grad_out, (float *)ctx->patches, mw);
            else if (op.kernel == 5) depthwise_grad_filters_fixed_kernel<T, 5><<<grid, 256, 0, ctx->stream>>>(op, (const T *)img, (const T *)grad_out, (float *)ctx->patches, mw);
            else depthwise_grad_filters_fixed_kernel<T, 7><<<grid, 256, 0, ctx->stream>>>(op, (const T *)img, (const T *)grad_out, (float *)ctx->patches, mw);
            HIP_TRY(hipGetLastError());
            const int total = (int)(op.chan_out * kk);
            depthwise_grad_filters_add_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>((const float *)ctx->patches, (T *)grad_filters, slices, (int)kk, total);
            return (int)hipGetLastError();
        }
        depthwise_grad_filters_kernel<T><<<(unsigned)op.chan_out, 256, 0, ctx->stream>>>(op, (const T *)img, (const T *)grad_out, (T *)grad_filters,
                                                                                      magic_of(op.w_out));
        return (int)hipGetLastError();
    }
    // (also at unit stride when the image has far fewer channels than the output -- a first layer, 3 -> 64: the forward patch
    // matrix is O / C times smaller than the one over grad_out, and the products with three rows of filters disappear)
    if (op.stride > 1 || (int64_t)op.chan_in * 4 <= op.chan_out)
        return strided_backward<T>(ctx, dtype, op, img, grad_img, filters, grad_filters, grad_out, fresh_img);
    if (per_image >= (1ll << 31) || f_elems >= (1ll << 31) || (int64_t)op.chan_in * hp >= (1ll << 31)) return DFDX_ROCM_ERR_UNSUPPORTED;
    CtxLock lock(ctx->mu);  // the patch buffer is shared by every conv2d call on this context
    int64_t chunk = std::max<int64_t>(1, (int64_t)(kPatchBudget / sizeof(T)) / per_image);
    chunk = std::min<int64_t>(std::min<int64_t>(chunk, op.batch), ((1ll << 31) - 1) / per_image);
    // H*W not a multiple of the vector width: the image and its gradient take part as padded copies
    // (zeros behind every row; the gradient copy starts from grad_img, so beta = 1 rounds exactly as without it).
    const bool padded = hp != hw;
    // patch buffer: [chunk][O*K*K][hp], the transposed filters and their gradient, then the padded copies
    // 1x1 filters at unit stride without padding: the patch matrix IS grad_out
    const bool pointwise = op.kernel == 1 && op.stride == 1 && op.padding == 0 && !padded && ((uintptr_t)grad_out & 15u) == 0;
    if (pointwise) chunk = op.batch;
    const size_t patch_bytes = pointwise ? 0 : round256((size_t)(chunk * per_image) * sizeof(T));
    const size_t f_bytes = round256((size_t)f_elems * sizeof(T));
    // Small images multiply as ONE product over the batch, as in the forward pass: patches [O K K][batch * hp], the image
    // and its gradient as [C][batch * hp]; the image gradient no longer reads the filters once per image and the filter
    // gradient is a plain product with k = batch * hp.
    int fold_cg = 0, fold_bg = 0;
    size_t fold_lds = 0;
    const bool fold = !pointwise && op.groups == 1 && op.stride == 1 && hp < 256 && op.batch > 1 && op.chan_in <= 32768 && op.chan_out <= 32768 &&
                      chunk <= 32768 && chunk * std::max(op.chan_in, op.chan_out) * hp < (1ll << 31) &&
                      small_unfold_shape<T>(hp, ohw, (int)std::min<int64_t>(chunk, op.batch), &fold_cg, &fold_bg, &fold_lds);
    const size_t img_bytes = (padded || fold) ? round256((size_t)(chunk * op.chan_in * hp) * sizeof(T)) : 0;
    // The image gradient of a 3 x 3, unit-stride, padding-1 convolution is such a convolution of grad_out (filters turned
    // by 180 degrees, channels trading places): f16 / bf16 / f32 run it on the kernel that reads its taps from a band of
    // grad_out in LDS (conv3x3.hip) instead of the product with the patch matrix, which only the filter gradient needs then.
    Conv3x3Problem band{};
    bool use_band = false;
    if (sizeof(T) <= 4 && op.kernel == 3 && op.stride == 1 && op.padding == 1 && op.dilation == 1 && op.groups == 1 &&
        op.h_out == op.h_in && op.w_out == op.w_in) {
        band.dtype = dtype == DFDX_ROCM_F16 ? DT_F16 : dtype == DFDX_ROCM_BF16 ? DT_BF16 : DT_F32;
        band.chan_in = op.chan_out; band.chan_out = op.chan_in; band.h = op.h_in; band.w = op.w_in;
        band.batch = (int)chunk;
        band.img = grad_out; band.filters = filters; band.out = grad_img;
        band.accumulate = fresh_img ? 0 : 1; band.transposed_filters = 1;
        band.wt = (void *)16;  // (placed below)
        use_band = conv3x3_supported(band);
    }
    const size_t wt_bytes = use_band ? round256(conv3x3_filter_bytes(band)) : 0;
    // The filter gradient of such a convolution has its own kernels too (conv3x3_wgrad.hip; 16-bit types: both operands
    // pixel-major in LDS, fragments through transposing reads; f32: channel-major bands, one value per lane and MFMA).
    // With both in place the backward pass forms no patch matrix at all.
    Conv3x3Problem wgrad{};
    bool use_wgrad = false;
    if (use_band) {
        wgrad.dtype = band.dtype;
        wgrad.batch = op.batch; wgrad.chan_in = op.chan_in; wgrad.chan_out = op.chan_out; wgrad.h = op.h_in; wgrad.w = op.w_in;
        wgrad.img = img; wgrad.out = const_cast<void *>(grad_out); wgrad.filters = grad_filters;
        use_wgrad = conv3x3_wgrad_supported(wgrad, ctx->compute_units);
    }
    if (use_band && use_wgrad) {
        const size_t ws_bytes = round256(conv3x3_wgrad_workspace_bytes(wgrad, ctx->compute_units));
        if (int rc = ensure_patches(ctx, ws_bytes + wt_bytes)) return rc;
        band.batch = op.batch;
        band.wt = (char *)ctx->patches + ws_bytes;
        HIP_TRY(launch_conv3x3(band, ctx->stream));
        return (int)launch_conv3x3_wgrad(wgrad, ctx->compute_units, ctx->patches, ctx->stream);
    }
    if (pointwise) {
        // Filters [O][C/G] are plain matrices here and both products take them as they lie, transposed through the strides:
        // no transposed copies, no zeroed scratch gradient, no pass that adds it back.
        //   grad_img (B, G, C/G, H*W) += filters^T (G, C/G, O/G) . grad_out (B, G, O/G, H*W)
        {
            const int64_t m = cg, k = og, n = hw;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.accumulate = fresh_img ? 0 : 1;
            d.batch1 = op.batch; d.batch2 = op.groups;
            d.a = filters; d.a_rs = 1; d.a_cs = m; d.a_b1 = 0; d.a_b2 = m * k;
            d.b = grad_out; d.b_rs = n; d.b_cs = 1; d.b_b1 = op.groups * k * n; d.b_b2 = k * n;
            d.c = grad_img; d.c_rs = n; d.c_cs = 1; d.c_b1 = op.chan_in * n; d.c_b2 = m * n;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
        //   grad_filters (O/G, C/G) += sum over images of grad_out (O/G, H*W) . img^T (H*W, C/G)
        for (int g = 0; g < op.groups; g++) {
            const int64_t m = og, k = hw, n = cg;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.accumulate = 1;
            d.reduce_batch = 1;
            d.batch1 = op.batch;
            d.a = (const T *)grad_out + g * m * k; d.a_rs = k; d.a_cs = 1; d.a_b1 = op.chan_out * k;
            d.b = (const T *)img + g * n * k; d.b_rs = 1; d.b_cs = k; d.b_b1 = op.chan_in * k;
            d.c = (T *)grad_filters + g * m * n; d.c_rs = n; d.c_cs = 1;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
        return DFDX_ROCM_OK;
    }
    if (fresh_img && !use_band && !fold) {  // the product below adds into (a padded copy of) grad_img: clear it after all
        HIP_TRY(launch_zero_fill(grad_img, (size_t)op.batch * op.chan_in * hw * sizeof(T), ctx->compute_units, ctx->stream));
        fresh_img = false;
    }
    if (int rc = ensure_patches(ctx, patch_bytes + 2 * f_bytes + 2 * img_bytes + wt_bytes)) return rc;
    T *patches = (T *)ctx->patches;
    T *f_tr = (T *)((char *)ctx->patches + patch_bytes);
    T *grad_f_tr = (T *)((char *)ctx->patches + patch_bytes + f_bytes);
    T *img_p = (T *)((char *)ctx->patches + patch_bytes + 2 * f_bytes);
    T *grad_img_p = (T *)((char *)ctx->patches + patch_bytes + 2 * f_bytes + img_bytes);
    // (the scratch gradient is not cleared: the first chunk's product overwrites it)
    const dim3 fgrid((unsigned)op.chan_out, (unsigned)((cg * kk + 255) / 256));
    const uint32_t magic_kk = magic_of(kk);
    const bool tiled_tr = cg % 16 == 0 && og % 16 == 0 && 256 * kk * sizeof(T) <= 48 * 1024;
    const dim3 tgrid((unsigned)(cg / 16), (unsigned)(og / 16), (unsigned)op.groups);
    const uint32_t magic_16kk = magic_of(16 * kk);
    if (tiled_tr)
        filter_transpose_tiled_kernel<T, false><<<tgrid, 256, 256 * kk * sizeof(T), ctx->stream>>>(op, (T *)const_cast<void *>(filters), f_tr, magic_kk, magic_16kk);
    else filter_transpose_kernel<T, false><<<fgrid, 256, 0, ctx->stream>>>(op, (T *)const_cast<void *>(filters), f_tr, magic_kk);
    HIP_TRY(hipGetLastError());
    const bool planes = op.stride == 1 && op.w_in % V == 0 && op.w_out >= V && (hw / V) * kk >= 512;
    for (int64_t b0 = 0; b0 < op.batch; b0 += chunk) {
        const int64_t nb = std::min<int64_t>(chunk, op.batch - b0);
        Op sub = op;
        sub.batch = (int)nb;
        const T *go = (const T *)grad_out + b0 * op.chan_out * ohw;
        const unsigned slabs = (unsigned)(nb * op.chan_out * kk);
        if (fold && !use_band) {
            const T *img_b = (const T *)img + b0 * op.chan_in * hw;
            T *grad_img_b = (T *)grad_img + b0 * op.chan_in * hw;
            const int64_t nf = nb * hp;  // columns of the folded matrices
            const int bg = std::min<int>(fold_bg, (int)nb);
            const SmallDivs mg{magic_of(hp / V), magic_of(op.kernel), magic_of(kk), magic_of(op.chan_out), magic_of(op.w_in), magic_of(op.stride),
                               magic_of(ohw), magic_of(bg)};
            unfold_small_kernel<T, true><<<dim3((unsigned)((op.chan_out + fold_cg - 1) / fold_cg), (unsigned)((nb + bg - 1) / bg)), 256, fold_lds, ctx->stream>>>(
                sub, mg, go, patches, (int)hp, fold_cg, bg);
            HIP_TRY(hipGetLastError());
            const int64_t folded = op.chan_in * nf;
            const unsigned g = (unsigned)((folded + 255) / 256);
            const FoldDivs fd{magic_of(hw), magic_of(hp), magic_of(op.chan_in), magic_of(nb)};
            fold_rows_kernel<T><<<g, 256, 0, ctx->stream>>>(img_b, img_p, (int)hw, (int)hp, op.chan_in, (int)nb, fd, (uint32_t)folded);
            HIP_TRY(hipGetLastError());
            if (!fresh_img) {
                fold_rows_kernel<T><<<g, 256, 0, ctx->stream>>>(grad_img_b, grad_img_p, (int)hw, (int)hp, op.chan_in, (int)nb, fd, (uint32_t)folded);
                HIP_TRY(hipGetLastError());
            }
            {   // grad_img (C, B * hp) += filters^T (C, O*K*K) . patches (O*K*K, B * hp); the copy started from grad_img: one rounding
                const int64_t m = cg, k = og * kk;
                dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, nf);
                d.accumulate = fresh_img ? 0 : 1;
                d.a = f_tr; d.a_rs = k; d.a_cs = 1;
                d.b = patches; d.b_rs = nf; d.b_cs = 1;
                d.c = grad_img_p; d.c_rs = nf; d.c_cs = 1;
                if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
            }
            const int64_t total = nb * op.chan_in * hw;
            unfold_rows_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(grad_img_p, grad_img_b, (int)hw, (int)hp, op.chan_in, (int)nb, fd, (uint32_t)total);
            HIP_TRY(hipGetLastError());
            {   // grad_filters^T (C, O*K*K) += img (C, B * hp) . patches^T (B * hp, O*K*K)
                const int64_t m = cg, n = og * kk;
                dfdx_rocm_gemm_desc d = blank_desc(dtype, m, nf, n);
                d.accumulate = b0 > 0;
                d.a = img_p; d.a_rs = nf; d.a_cs = 1;
                d.b = patches; d.b_rs = 1; d.b_cs = nf;
                d.c = grad_f_tr; d.c_rs = n; d.c_cs = 1;
                if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
            }
            continue;
        }
        if (planes && op.kernel == 3) unfold_output_plane_kernel<T, 3><<<slabs / 9, 256, 0, ctx->stream>>>(sub, go, patches, (int)hp);
        else if (planes) unfold_output_plane_kernel<T, 0><<<(unsigned)(slabs / kk), 256, 0, ctx->stream>>>(sub, go, patches, (int)hp);
        else {
            const uint32_t vectors = (uint32_t)(slabs * (hp / V));
            if (op.stride == 1) unfold_output_flat_kernel<T, true><<<(vectors + 255) / 256, 256, 0, ctx->stream>>>(sub, go, patches, (int)hp, vectors);
            else unfold_output_flat_kernel<T, false><<<(vectors + 255) / 256, 256, 0, ctx->stream>>>(sub, go, patches, (int)hp, vectors);
        }
        HIP_TRY(hipGetLastError());
        const T *img_b = (const T *)img + b0 * op.chan_in * hw;
        T *grad_img_b = (T *)grad_img + b0 * op.chan_in * hw;
        const int64_t rows_p = nb * op.chan_in * hp;
        if (padded) {
            launch_pad_rows<T>(img_b, img_p, hw, hp, rows_p, ctx->stream);
            HIP_TRY(hipGetLastError());
            if (!use_band) {
                launch_pad_rows<T>(grad_img_b, grad_img_p, hw, hp, rows_p, ctx->stream);
                HIP_TRY(hipGetLastError());
            }
        }
        if (use_band) {
            band.batch = (int)nb;
            band.img = go; band.out = grad_img_b;
            band.wt = (char *)ctx->patches + patch_bytes + 2 * f_bytes + 2 * img_bytes;
            HIP_TRY(launch_conv3x3(band, ctx->stream));
        } else {   // grad_img (B, G, C/G, H*W) += filters^T (G, C/G, O/G*K*K) . patches (B, G, O/G*K*K, H*W)
            const int64_t m = cg, k = og * kk, n = hp;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.accumulate = 1;
            d.batch1 = nb; d.batch2 = op.groups;
            d.a = f_tr; d.a_rs = k; d.a_cs = 1; d.a_b1 = 0; d.a_b2 = m * k;
            d.b = patches; d.b_rs = n; d.b_cs = 1; d.b_b1 = op.groups * k * n; d.b_b2 = k * n;
            d.c = padded ? grad_img_p : grad_img_b; d.c_rs = n; d.c_cs = 1; d.c_b1 = op.chan_in * n; d.c_b2 = m * n;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
        if (padded && !use_band) {
            const int64_t total = nb * op.chan_in * hw;
            unpad_rows_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(grad_img_p, grad_img_b, (int)hw, (int)hp, total);
            HIP_TRY(hipGetLastError());
        }
        for (int g = 0; g < op.groups; g++) {
            // grad_filters^T (C/G, O/G*K*K) += sum over images of img (C/G, H*W) . patches^T (H*W, O/G*K*K)
            const int64_t m = cg, k = hp, n = og * kk;
            dfdx_rocm_gemm_desc d = blank_desc(dtype, m, k, n);
            d.accumulate = b0 > 0;
            d.reduce_batch = 1;
            d.batch1 = nb;
            d.a = (padded ? (const T *)img_p : img_b) + g * cg * k; d.a_rs = k; d.a_cs = 1; d.a_b1 = op.chan_in * k;
            d.b = patches + g * n * k; d.b_rs = 1; d.b_cs = k; d.b_b1 = per_image;
            d.c = grad_f_tr + g * m * n; d.c_rs = n; d.c_cs = 1;
            if (int rc = dfdx_rocm_gemm(ctx, &d)) return rc;
        }
    }
    if (tiled_tr) filter_transpose_tiled_kernel<T, true><<<tgrid, 256, 256 * kk * sizeof(T), ctx->stream>>>(op, (T *)grad_filters, grad_f_tr, magic_kk, magic_16kk);
    else filter_transpose_kernel<T, true><<<fgrid, 256, 0, ctx->stream>>>(op, (T *)grad_filters, grad_f_tr, magic_kk);
    return (int)hipGetLastError();
}

}  // namespace
}  // namespace dfdx_rocm

using namespace dfdx_rocm;

extern "C" {

int dfdx_rocm_conv2d_forward(dfdx_rocm_ctx *ctx, int dtype, const dfdx_rocm_conv2d_op *op, const void *img,
                             const void *filters, void *out) {
    if (int e = bind(ctx)) return e;
    Op o;
    if (!op) return DFDX_ROCM_ERR_INVALID_ARG;
    if (int e = narrow(op, &o)) return e;
    if (o.batch == 0 || o.chan_out == 0 || o.h_out == 0 || o.w_out == 0) return DFDX_ROCM_OK;
    if (!img || !filters || !out) return DFDX_ROCM_ERR_INVALID_ARG;
    for (const void *p : {img, filters, (const void *)out})  // deferred zero fills among the operands run first
        if (int e = settle(ctx, p)) return e;
    switch (dtype) {
    case DFDX_ROCM_F32: return forward_t<float>(ctx, dtype, o, img, filters, out);
    case DFDX_ROCM_F16: return forward_t<_Float16>(ctx, dtype, o, img, filters, out);
    case DFDX_ROCM_BF16: return forward_t<__bf16>(ctx, dtype, o, img, filters, out);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

int dfdx_rocm_conv2d_backward(dfdx_rocm_ctx *ctx, int dtype, const dfdx_rocm_conv2d_op *op, const void *img, void *grad_img,
                              const void *filters, void *grad_filters, const void *grad_out) {
    if (int e = bind(ctx)) return e;
    Op o;
    if (!op) return DFDX_ROCM_ERR_INVALID_ARG;
    if (int e = narrow(op, &o)) return e;
    if (o.batch == 0 || o.chan_out == 0 || o.chan_in == 0) return DFDX_ROCM_OK;
    if (!img || !grad_img || !filters || !grad_filters || !grad_out) return DFDX_ROCM_ERR_INVALID_ARG;
    // deferred zero fills among the operands run first (the gradients are reached through several kernels here)
    for (const void *p : {img, filters, grad_out, (const void *)grad_filters})
        if (int e = settle(ctx, p)) return e;
    // grad_img: a buffer declared zero whose fill has not run and that this call covers is taken over unfilled -- the image
    // gradient is then stored instead of added (0 + value: the same bits, without the fill's write and the read of the zeros)
    bool fresh_img = false;
    const size_t es = dtype == DFDX_ROCM_F32 ? 4 : 2;
    if (dtype == DFDX_ROCM_F32 || dtype == DFDX_ROCM_F16 || dtype == DFDX_ROCM_BF16) {
        if (int e = settle_output(ctx, grad_img, (size_t)o.batch * o.chan_in * o.h_in * o.w_in * es, true, &fresh_img)) return e;
    } else if (int e = settle(ctx, grad_img)) return e;
    int rc;
    switch (dtype) {
    case DFDX_ROCM_F32: rc = backward_t<float>(ctx, dtype, o, img, grad_img, filters, grad_filters, grad_out, fresh_img); break;
    case DFDX_ROCM_F16: rc = backward_t<_Float16>(ctx, dtype, o, img, grad_img, filters, grad_filters, grad_out, fresh_img); break;
    case DFDX_ROCM_BF16: rc = backward_t<__bf16>(ctx, dtype, o, img, grad_img, filters, grad_filters, grad_out, fresh_img); break;
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
    // a call that fails after taking the gradient over unfilled leaves it as it was declared: zeros
    if (rc != DFDX_ROCM_OK && fresh_img)
        (void)launch_zero_fill(grad_img, (size_t)o.batch * o.chan_in * o.h_in * o.w_in * es, ctx->compute_units, ctx->stream);
    return rc;
}

}  // extern "C"
