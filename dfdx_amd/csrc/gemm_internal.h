// Internal interfaces between the C ABI (api.cpp) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>

namespace dfdx_rocm {

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2, DT_F64 = 3 };
enum { BIAS_NONE = 0, BIAS_PER_COL = 1, BIAS_PER_ROW = 2 };
enum { KSUM_NONE = 0, KSUM_OF_A = 1, KSUM_OF_B = 2 };

// One strided, batched GEMM:  C[b][i,j] = (accumulate ? C : 0) + bias + sum_k A[b][i,k] * B[b][k,j].
// Strides are in elements.  With `reduce` set, all nb1*nb2 batches are summed into one C.
struct GemmProblem {
    int dtype;
    int accumulate;
    int reduce;
    int bias_mode;
    int64_t m, n, k;
    int64_t nb1, nb2;
    const void *a;
    int64_t a_rs, a_cs, a_b1, a_b2;
    const void *b;
    int64_t b_rs, b_cs, b_b1, b_b2;
    void *c;
    int64_t c_rs, c_cs, c_b1, c_b2;
    const void *bias;
    // Optional second result, in the element type: the sums of one operand over the contraction (and over the batches
    // of a reduced product), ksum[i] (+)= sum_k A[i,k] (KSUM_OF_A, length m) or ksum[j] (+)= sum_k B[k,j] (KSUM_OF_B,
    // length n).  `Linear`'s bias gradient is the latter for the weight-gradient product x^T . grad_out.  Only some
    // kernels produce it (mfma16dma_ksum_supported, small_ksum_supported); the caller clears `ksum` and runs the reduction
    // itself otherwise.
    void *ksum = nullptr;
    int ksum_of = KSUM_NONE;
    int ksum_accumulate = 0;
    // split-k (filled in by the planner): `splits` workgroups share one C tile; f32 partials go to `workspace`
    int splits;
    float *workspace;
    int compute_units;  // of the device the launch goes to (persistent kernels size their grid with it)
};

// The patch matrix of a unit-stride convolution as the B operand of a GEMM, never materialised: row k = (channel,
// tap (k1, k2)), column = pixel (r, x) of a `w_dst`-wide grid; element = plane[channel][r + off_y + step_y * k1]
// [x + off_x + step_x * k2], zero outside the h_src x w_src plane.
struct ConvPatches {
    int taps, ksize;     // K*K, K
    int w_dst;           // pixels per row of the column index space (>= 8)
    int h_src, w_src;    // the planes the windows come from (w_src >= 8)
    int off_y, off_x, step_y, step_x;
    int64_t plane;       // elements between channels
};

// What a launcher learns once per kernel instance AND device (the dynamic-LDS attribute is set, the occupancy is known):
// one word per device, 0 = not yet.  Two host threads that arrive together both do the set-up and store the same value.
struct PerDevice {
    std::atomic<int> word[64];
    std::atomic<int> &here() {
        int dev = 0;
        (void)hipGetDevice(&dev);
        return word[dev & 63];
    }
};

static inline size_t dtype_size(int dt) { return dt == DT_F32 ? 4 : (dt == DT_F64 ? 8 : 2); }

// Swap the roles of the operands: C^T = B^T A^T.  Used to turn a column-major C into a row-major one.
static inline GemmProblem transposed(const GemmProblem &p) {
    GemmProblem t = p;
    t.m = p.n; t.n = p.m;
    t.a = p.b; t.a_rs = p.b_cs; t.a_cs = p.b_rs; t.a_b1 = p.b_b1; t.a_b2 = p.b_b2;
    t.b = p.a; t.b_rs = p.a_cs; t.b_cs = p.a_rs; t.b_b1 = p.a_b1; t.b_b2 = p.a_b2;
    t.c_rs = p.c_cs; t.c_cs = p.c_rs;
    if (p.bias_mode == BIAS_PER_COL) t.bias_mode = BIAS_PER_ROW;
    else if (p.bias_mode == BIAS_PER_ROW) t.bias_mode = BIAS_PER_COL;
    if (p.ksum_of == KSUM_OF_A) t.ksum_of = KSUM_OF_B;
    else if (p.ksum_of == KSUM_OF_B) t.ksum_of = KSUM_OF_A;
    return t;
}

// ---- generic kernel (gemm_generic.hip): every dtype, every stride pattern ----
hipError_t launch_generic(const GemmProblem &p, hipStream_t stream);

// ---- MFMA kernels for 16-bit inputs (gemm_mfma16.hip) ----
// Variants are numbered from 1.  `supported` checks alignment / layout preconditions.
int mfma16_variant_count();
const char *mfma16_variant_name(int variant);
bool mfma16_supported(const GemmProblem &p, int variant);
int mfma16_pick_variant(const GemmProblem &p, int compute_units);
int mfma16_dma_first_variant();  // variant ids >= this are the LDS-DMA kernels ...
int mfma16_small_variant();      // ... except the last one, the small-product kernel
// split-k of the register-staged variants (ids below mfma16_dma_first_variant)
int mfma16_plan_splits(const GemmProblem &p, int variant, int compute_units, int forced_splits);
size_t mfma16_workspace_bytes(const GemmProblem &p, int variant, int splits);
double mfma16_staged_time(const GemmProblem &p, int variant, int splits, int compute_units);  // estimated seconds
// a few rows or columns against a large matrix: the 64 x 64 register-staged tile with split-k (0 = does not apply)
int mfma16_skinny_plan(const GemmProblem &p, int compute_units, int forced_splits, int *splits, double *seconds);
hipError_t launch_mfma16(const GemmProblem &p, int variant, hipStream_t stream);
// The same product with B given as a patch matrix (`p.b` = channel 0 of the first image, b_b1 / b_b2 = image and group
// strides, b_rs / b_cs unused): register-staged kernels only, tile chosen inside.  Returns hipErrorNotSupported when
// the shape does not fit (the caller then unfolds).
hipError_t launch_mfma16_conv(const GemmProblem &p, const ConvPatches &conv, int compute_units, hipStream_t stream);

// ---- LDS-DMA MFMA kernels for 16-bit inputs, K % 64 == 0 (gemm_mfma16_dma.hip) ----
// Reached through the mfma16_* entry points above: their variant ids follow the register-staged ones.
int mfma16dma_variant_count();
const char *mfma16dma_variant_name(int variant);
bool mfma16dma_supported(const GemmProblem &p, int variant);
int mfma16dma_pick_variant(const GemmProblem &p, int compute_units);
hipError_t launch_mfma16dma(const GemmProblem &p, int variant, hipStream_t stream);
// Split-k planning for the LDS-DMA kernels: picks tile variant and split count together.  `forced_splits`
// > 0 overrides the count (clamped to what the k extent allows).  `seconds` (may be null) receives the estimate.
void mfma16dma_plan_split(const GemmProblem &p, int compute_units, int forced_variant, int forced_splits, int *variant,
                          int *splits, double *seconds = nullptr);
size_t mfma16dma_workspace_bytes(const GemmProblem &p, int variant, int splits);
bool mfma16dma_ksum_supported(const GemmProblem &p, int variant, int splits);  // can this plan also produce p.ksum?

// ---- split-k combine (splitk_reduce.hip): C = (accumulate ? C : 0) + bias + sum_s partial[s], s ascending ----
// `ws_ksum` (may be null): [ksum_slots][ws_ksum_stride] f32 partial sums of p.ksum, added up in slot order into p.ksum.
hipError_t launch_splitk_reduce(const GemmProblem &p, int64_t ws_ld, int64_t ws_split_stride, hipStream_t stream,
                                const float *ws_ksum = nullptr, int64_t ws_ksum_stride = 0, int ksum_slots = 0);

// ---- MFMA kernels for f32 (gemm_mfma32.hip) ----
int mfma32_variant_count();
const char *mfma32_variant_name(int variant);
bool mfma32_supported(const GemmProblem &p, int variant);
int mfma32_pick_variant(const GemmProblem &p, int compute_units, int forced_splits, double *seconds = nullptr);  // + its estimate
int mfma32_plan_splits(const GemmProblem &p, int variant, int compute_units, int forced_splits);
size_t mfma32_workspace_bytes(const GemmProblem &p, int variant, int splits);
hipError_t launch_mfma32(const GemmProblem &p, int variant, hipStream_t stream);
bool mfma32_ksum_supported(const GemmProblem &p, int variant);  // can this variant also produce p.ksum? (the small kernel)

// ---- MFMA kernels for f64 (gemm_mfma64.hip) ----
int mfma64_variant_count();
const char *mfma64_variant_name(int variant);
bool mfma64_supported(const GemmProblem &p, int variant);
int mfma64_pick_variant(const GemmProblem &p, int compute_units);
int mfma64_small_variant();
double mfma64_time(const GemmProblem &p, int variant, int compute_units);  // estimated seconds of a tiled variant
hipError_t launch_mfma64(const GemmProblem &p, int variant, hipStream_t stream);

// ---- small products in every element type (gemm_small.hip): 16 x 16 tiles, the contraction cut over the waves ----
// Any operand strides, one product per launch, row-major C.  Each family lists it as its last variant.
bool small_supported(const GemmProblem &p);
bool small_ksum_supported(const GemmProblem &p);  // p.ksum of A as a second result
double small_time(const GemmProblem &p, int compute_units);  // estimated seconds
hipError_t launch_small(const GemmProblem &p, hipStream_t stream);

// ---- bandwidth-bound vector products (gemv.hip) ----
bool gemv_supported(const GemmProblem &p);
size_t gemv_workspace_bytes(const GemmProblem &p);  // f32 partial sums of the k slices (0 when not sliced)
hipError_t launch_gemv(const GemmProblem &p, hipStream_t stream);

// ---- two to eight vectors against one streamed matrix (gemv_multi.hip): M or N of 2 .. 8, the other operand a megabyte at least ----
bool gemv_multi_supported(const GemmProblem &p);
size_t gemv_multi_workspace_bytes(const GemmProblem &p);
double gemv_multi_time(const GemmProblem &p);  // estimated seconds
hipError_t launch_gemv_multi(const GemmProblem &p, hipStream_t stream);

// ---- thin contractions with large outputs on the matrix cores (gemm_small.hip): k <= 32, f32 / f16 / bf16, row-major C ----
bool thin_mfma_supported(const GemmProblem &p);
hipError_t launch_thin_mfma(const GemmProblem &p, hipStream_t stream);

// ---- rank-1 updates and thin contractions, k = 1 .. 8 (rank1.hip): every dtype, any operand strides, row-major C ----
bool rank1_supported(const GemmProblem &p);
hipError_t launch_rank1(const GemmProblem &p, hipStream_t stream);

// XCD-aware remap of a linear workgroup id: consecutive ids are dispatched round-robin
// over the 8 XCDs, so ids that share an XCD (and its L2) are pid, pid+8, pid+16 ...
// This returns a work index such that each XCD owns one contiguous range of work.
__device__ __forceinline__ int xcd_remap(int pid, int total) {
    constexpr int NXCD = 8;
    if (total < 2 * NXCD) return pid;
    const int per = (total + NXCD - 1) / NXCD;
    const int tall = (total % NXCD == 0) ? NXCD : total % NXCD;  // XCDs that own `per` items; the rest own per-1
    const int xcd = pid % NXCD, local = pid / NXCD;
    return xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
}

}  // namespace dfdx_rocm
