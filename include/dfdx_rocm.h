/*
 * dfdx_rocm.h -- C ABI of the MI355X (gfx950) matrix-multiplication backend
 * for dfdx.
 *
 * These are the entry points a `Rocm` device inside dfdx-core binds over FFI in
 * order to implement the kernel traits its `Cpu` and `Cuda` devices implement
 * for `matmul`.  Each declaration names the reference interface it stands in
 * for (paths relative to the dfdx repository, v0.13.0).
 *
 * Conventions
 *   - Every function returns 0 on success.  Positive values are `hipError_t`
 *     codes, negative values are the DFDX_ROCM_ERR_* codes below;
 *     dfdx_rocm_strerror() renders either.  Nothing throws or aborts across
 *     this boundary (the Rust side maps the code into `tensor::Error`,
 *     dfdx-core/src/tensor/error.rs:5-28).
 *   - Pointers named a/b/c/lhs/rhs/out/grad_* are DEVICE pointers owned by the
 *     caller; the library never frees or retains them.
 *   - Strides and batch strides are in ELEMENTS (not bytes), exactly the
 *     `strides: [usize; N]` a dfdx `Tensor` carries
 *     (dfdx-core/src/tensor/tensor_impls.rs:32-39).  Any stride pattern a dfdx
 *     view can produce is accepted for inputs: transposed, permuted
 *     (head-interleaved), broadcast (stride 0).
 *   - Work is asynchronous on the context's stream; dfdx_rocm_synchronize()
 *     blocks until it is done.
 *   - f16 and bf16 products accumulate in f32 and round to nearest even once
 *     on store; f32 accumulates in f32; f64 in f64.
 *   - Every entry point takes all four element types, conv2d excepted (f16,
 *     bf16, f32): the ops around the products evaluate their formula in f32
 *     for the 16- and 32-bit types and round once, and in f64 for f64.
 */
#ifndef DFDX_ROCM_H
#define DFDX_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dfdx_rocm_ctx dfdx_rocm_ctx;

/* Element types (dfdx-core/src/dtypes/mod.rs:87-116).  `f16` and `AMP<f16>`
 * are both DFDX_ROCM_F16 (same storage, f32 math: dtypes/amp.rs:8-10). */
enum {
    DFDX_ROCM_F32 = 0,
    DFDX_ROCM_F16 = 1,
    DFDX_ROCM_BF16 = 2,
    DFDX_ROCM_F64 = 3
};

enum {
    DFDX_ROCM_OK = 0,
    DFDX_ROCM_ERR_INVALID_ARG = -1,   /* null pointer, negative size, unknown dtype ...          */
    DFDX_ROCM_ERR_UNSUPPORTED = -2,   /* valid request this build has no kernel for              */
    DFDX_ROCM_ERR_NO_DEVICE = -3,     /* no usable gfx950 device                                 */
    DFDX_ROCM_ERR_ALIASED_OUTPUT = -4, /* output view maps several logical elements to one address */
    DFDX_ROCM_ERR_SCRATCH_TOO_SMALL = -5 /* dfdx_rocm_gemm_noalloc: the plan needs more scratch than the fixed array holds */
};

/* Kernel families, for dfdx_rocm_gemm_desc.kernel (0 lets the library choose). */
enum {
    DFDX_ROCM_KERNEL_AUTO = 0,
    DFDX_ROCM_KERNEL_GENERIC = 1, /* any strides, any dtype (scalar loads, LDS tiled)   */
    DFDX_ROCM_KERNEL_MFMA = 2,    /* matrix-core kernels; variant chosen by `variant`   */
    DFDX_ROCM_KERNEL_GEMV = 3     /* bandwidth-bound: M or N of 1..8, K of 1..32        */
};

/* ---- device context -----------------------------------------------------
 * Stands in for `Cuda::try_build(ordinal, seed)` and the handles it owns
 * (dfdx-core/src/tensor/cuda/device.rs:22-33,72-90).  `stream` is a
 * `hipStream_t` to run on, or NULL for the device's default stream. */
int dfdx_rocm_create(int ordinal, void *stream, dfdx_rocm_ctx **out);
int dfdx_rocm_destroy(dfdx_rocm_ctx *ctx);
const char *dfdx_rocm_strerror(int code);
/* Device name ("gfx950..."), compute-unit count and clock, for roofline reports. */
int dfdx_rocm_device_info(dfdx_rocm_ctx *ctx, char *name, size_t name_len, int *compute_units, int *clock_mhz);

/* ---- storage --------------------------------------------------------------
 * What `Storage::try_alloc_len` (zero-filled; cuda/device.rs:259-266),
 * `alloc_empty` (cuda/device.rs:97-106), `CopySlice` / `tensor_to_vec`
 * (tensor/storage_traits.rs:93-96) and `Synchronize` (storage_traits.rs:31-39)
 * need from the device.  The zero fill (`zeroed` != 0, `dfdx_rocm_memset_zero`) is a
 * kernel launch on the context's stream, not a memset node: stream-ordered like every
 * other call, any alignment and length, and safe to record into a captured graph. */
int dfdx_rocm_alloc(dfdx_rocm_ctx *ctx, size_t bytes, int zeroed, void **out);
int dfdx_rocm_free(dfdx_rocm_ctx *ctx, void *ptr);
int dfdx_rocm_memset_zero(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes);
int dfdx_rocm_copy_h2d(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes);
int dfdx_rocm_copy_d2h(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes);
int dfdx_rocm_copy_d2d(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes);
int dfdx_rocm_synchronize(dfdx_rocm_ctx *ctx);

/* Deferred zero fill, for gradient storage.  `Gradients::get_or_alloc_mut`
 * (dfdx-core/src/tensor/gradients.rs:53-58) allocates every gradient
 * zero-filled and the backward ops then accumulate into it: in a training
 * step the fill and the first read of those zeros are pure HBM traffic.
 * A buffer allocated with `zeroed` = DFDX_ROCM_ZERO_DEFERRED (or declared
 * with dfdx_rocm_zero_deferred, for storage the caller owns) is zero as far as
 * any call of this library can tell, but its fill has not run:
 *   - the first call that accumulates into every byte of it (a backward
 *     entry or an accumulating GEMM whose output view is a permutation of
 *     the contiguous layout, starting at the buffer's first byte) stores
 *     0 + value without reading it, and the fill never runs;
 *   - any other first use through this library (an input operand, a partial
 *     or strided write, a copy out of it) runs the fill first;
 *   - dfdx_rocm_synchronize, dfdx_rocm_settle_zeros and dfdx_rocm_destroy run
 *     every fill still pending; dfdx_rocm_free drops the buffer's.
 * Results are bit-identical to the eager fill.  A deferred buffer is looked
 * up by the pointer a call is given: hand views of it to the library by a
 * pointer inside the buffer.  Code outside this library that reads the memory
 * (another stream, a host copy not made by dfdx_rocm_copy_d2h) must call
 * dfdx_rocm_settle_zeros or dfdx_rocm_synchronize first.
 * A declaration on storage the caller owns (dfdx_rocm_zero_deferred) lives
 * until a call consumes it; the library cannot see that storage being
 * released.  Before the caller frees, reuses or hands back such memory it must
 * either settle it (dfdx_rocm_settle_zeros, dfdx_rocm_synchronize) or
 * withdraw the declaration with dfdx_rocm_forget_zeros(ptr, bytes): every
 * declaration that lies wholly inside [ptr, ptr + bytes) is dropped without a
 * fill, one that reaches beyond either end is filled now (the memory is still
 * the caller's at that point).  Otherwise a later settle would write zeros
 * into memory that belongs to somebody else by then (the reference releases
 * gradient storage in mid-step: `Gradients::drop_non_leafs`,
 * tensor/gradients.rs:73-78).  Forgetting a range without declarations is not
 * an error. */
#define DFDX_ROCM_ZERO_DEFERRED 2
int dfdx_rocm_zero_deferred(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes);
int dfdx_rocm_settle_zeros(dfdx_rocm_ctx *ctx);
int dfdx_rocm_forget_zeros(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes);

/* The allocation cache of the device (`Cache::try_enable_cache`,
 * `try_disable_cache`, `try_empty_cache`: dfdx-core/src/tensor/
 * storage_traits.rs:41-77; `TensorCache`, tensor/cache.rs:36-149, which the
 * Cuda device consults in `try_alloc_len` and feeds from `Drop`).  Off at
 * first, as in the reference.  While it is on, dfdx_rocm_free keeps the
 * buffer (no synchronisation, no hipFree) and the next dfdx_rocm_alloc of
 * exactly that many bytes gets it back (zero-filled again when asked): a
 * training step's gradient buffers then cost no hipMalloc / hipFree after
 * the first step.  The reference keys on (bytes, element size, alignment)
 * for the sake of the Rust allocator; device buffers are 256 B-aligned raw
 * bytes, so the key is the byte count.  disable also empties; empty frees
 * what is held (after draining the stream); an allocation that fails for
 * lack of memory empties the cache and tries once more.
 * dfdx_rocm_cache_stats reports what is held right now (tests, tooling). */
int dfdx_rocm_enable_cache(dfdx_rocm_ctx *ctx);
int dfdx_rocm_disable_cache(dfdx_rocm_ctx *ctx);
int dfdx_rocm_empty_cache(dfdx_rocm_ctx *ctx);
int dfdx_rocm_cache_stats(dfdx_rocm_ctx *ctx, size_t *buffers, size_t *bytes);

/* ---- the strided (batched) GEMM -------------------------------------------
 * Stands in for `MatMulImpl::matmul` on Cpu
 * (dfdx-core/src/tensor_ops/matmul/cpu_kernel.rs:38-50) and for `Cuda::gemm` /
 * `Cuda::gemm_batch` (matmul/cuda_kernel.rs:153-181,184-237), which the conv
 * ops also call directly (conv2d/cuda_kernel.rs:115-139).
 *
 *   for b1 < batch1, b2 < batch2:
 *     C[b1,b2][i,j] = (accumulate ? C[b1,b2][i,j] : 0) + bias[j]
 *                     + sum_k A[b1,b2][i,k] * B[b1,b2][k,j]
 *   X[b1,b2][r,c] lives at x + b1*x_b1 + b2*x_b2 + r*x_rs + c*x_cs.
 *
 * `reduce_batch` != 0 sums all batches into ONE C (c_b1, c_b2 ignored): the
 * shared `grad_rhs` accumulator of the broadcast-rhs backward
 * (cpu_kernel.rs:339-348), which cuBLAS cannot express
 * (cuda_kernel.rs:358-371).  `bias` (length n, may be NULL) is the fused
 * `Bias1D` add of `Linear` (dfdx/src/nn/layers/linear.rs:82-89). */
typedef struct dfdx_rocm_gemm_desc {
    int32_t dtype;
    int32_t accumulate; /* 0: overwrite (forward); 1: add into C (every backward) */
    int64_t m, n, k;
    int64_t batch1, batch2; /* >= 1 */
    const void *a;
    int64_t a_rs, a_cs, a_b1, a_b2;
    const void *b;
    int64_t b_rs, b_cs, b_b1, b_b2;
    void *c;
    int64_t c_rs, c_cs, c_b1, c_b2;
    const void *bias;
    int32_t reduce_batch;
    int32_t kernel;  /* DFDX_ROCM_KERNEL_* ; 0 = automatic */
    int32_t variant; /* tile variant inside the family; 0 = automatic */
    int32_t flags;   /* DFDX_ROCM_GEMM_* bits below; 0 = defaults */
} dfdx_rocm_gemm_desc;

/* flags.  Long contractions with few output tiles (weight gradients) are split along k over several
 * workgroups whose f32 partial sums are combined in a fixed order (deterministic).  NO_SPLIT_K keeps the
 * contraction order of the tiled kernels: no split, no k-sliced small-product kernel, and none of the vector-product
 * kernels for few rows or columns (they cut k into slices too).  The broadcast-rhs forward / grad_lhs use it so that
 * they stay bit-identical to the batched kernels whatever the number of rows (dfdx tests assert that equality,
 * matmul/mod.rs:460-473).  SPLIT_K(n) forces n splits (testing / tuning). */
#define DFDX_ROCM_GEMM_NO_SPLIT_K 1
#define DFDX_ROCM_GEMM_SPLIT_K(n) (((n) & 0xff) << 8)

int dfdx_rocm_gemm(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc);

/* The same product for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference (its devices allocate freely).
 * dfdx_rocm_gemm grows a context-owned buffer on demand for the f32 partial
 * sums of a split reduction (split-k weight gradients, k-sliced vector
 * products); this entry point plans exactly as dfdx_rocm_gemm does -- same
 * kernels, same bits -- but keeps those partial sums in a fixed array of
 * DFDX_ROCM_NOALLOC_SCRATCH_BYTES that lives in the library's device image
 * (one copy per GPU, held until the process ends) and calls no hipMalloc /
 * hipFree or any other allocating routine.  A plan whose partial sums do not
 * fit is refused with DFDX_ROCM_ERR_SCRATCH_TOO_SMALL before anything is
 * launched and before any pending zero declaration of an operand is touched
 * (the caller may then lower or forbid the split through `flags`, or call
 * dfdx_rocm_gemm with the same descriptor).
 * Nothing in the array has to start at zero: every partial sum that is read
 * has been written by the same call.  All calls on one GPU share the array,
 * so calls that overlap on one GPU (two contexts, two streams, two threads)
 * race; calls on one context are ordered by its stream. */
#define DFDX_ROCM_NOALLOC_SCRATCH_BYTES (32u << 20)
int dfdx_rocm_gemm_noalloc(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc);

/* Which kernel dfdx_rocm_gemm would run for `desc`: writes the family, the
 * variant and a short name ("mfma16_256x256x64_kc_kc" ...).  No launch. */
int dfdx_rocm_gemm_plan(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, int *kernel, int *variant,
                        char *name, size_t name_len);
/* Number of MFMA tile variants available for `dtype` (variants are 1..count).  The last one
 * in every type is the small-product kernel (16 x 16 tiles of C, the contraction cut over
 * the waves of a workgroup; any operand strides, unbatched), which the planner picks by itself
 * for products of a few microseconds. */
int dfdx_rocm_mfma_variant_count(int dtype);

/* Times `iters` back-to-back launches of `desc` with HIP events recorded on
 * the context's stream (after `warmup` untimed launches) and returns the
 * average milliseconds per launch.  Benchmark aid; no reference counterpart
 * (dfdx's benches time with `Instant` around `synchronize`,
 * dfdx/benches/conv2d.rs:25-45). */
int dfdx_rocm_gemm_time(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, int warmup, int iters, float *avg_ms);
/* The same over `count` descriptors taken in turn (launch i runs descs[i % count]):
 * with each descriptor on its own buffers and more bytes in flight than the
 * 256 MB last-level cache holds, every launch reads HBM, not the previous
 * launch's lines.  Benchmark aid; no reference counterpart. */
int dfdx_rocm_gemm_time_rotating(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *descs, int count, int warmup, int iters,
                                 float *avg_ms);

/* ---- the four kernel traits -------------------------------------------------
 * One function per trait method.  `out` and `grad_out` are contiguous
 * row-major of the output shape; `grad_lhs` / `grad_rhs` are buffers laid out
 * like the operand's physical storage and are ACCUMULATED into through the
 * operand's own strides (cpu_kernel.rs:266-285).  `*_strides` have one entry
 * per tensor axis. */

/* MatMatKernel (matmul/mod.rs:116-131): (M,K) x (K,N). */
int dfdx_rocm_matmat_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t m, int64_t k, int64_t n,
                             const void *lhs, const int64_t lhs_strides[2],
                             const void *rhs, const int64_t rhs_strides[2], void *out);
int dfdx_rocm_matmat_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t m, int64_t k, int64_t n,
                              const void *lhs, const int64_t lhs_strides[2], void *grad_lhs,
                              const void *rhs, const int64_t rhs_strides[2], void *grad_rhs,
                              const void *grad_out);

/* MatMatBrKernel (matmul/mod.rs:197-212): (B,M,K) x (K,N), rhs broadcast over the batch. */
int dfdx_rocm_matmat_br_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                const void *lhs, const int64_t lhs_strides[3],
                                const void *rhs, const int64_t rhs_strides[2], void *out);
int dfdx_rocm_matmat_br_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                 const void *lhs, const int64_t lhs_strides[3], void *grad_lhs,
                                 const void *rhs, const int64_t rhs_strides[2], void *grad_rhs,
                                 const void *grad_out);

/* MatMatBatch3Kernel (matmul/mod.rs:234-249): (B,M,K) x (B,K,N). */
int dfdx_rocm_matmat_batch3_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                    const void *lhs, const int64_t lhs_strides[3],
                                    const void *rhs, const int64_t rhs_strides[3], void *out);
int dfdx_rocm_matmat_batch3_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                     const void *lhs, const int64_t lhs_strides[3], void *grad_lhs,
                                     const void *rhs, const int64_t rhs_strides[3], void *grad_rhs,
                                     const void *grad_out);

/* MatMatBatch4Kernel (matmul/mod.rs:273-288): (B,S,M,K) x (B,S,K,N). */
int dfdx_rocm_matmat_batch4_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t seq, int64_t m, int64_t k,
                                    int64_t n, const void *lhs, const int64_t lhs_strides[4],
                                    const void *rhs, const int64_t rhs_strides[4], void *out);
int dfdx_rocm_matmat_batch4_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t seq, int64_t m, int64_t k,
                                     int64_t n, const void *lhs, const int64_t lhs_strides[4], void *grad_lhs,
                                     const void *rhs, const int64_t rhs_strides[4], void *grad_rhs,
                                     const void *grad_out);

/* ---- Linear with the bias add fused into the GEMM store ---------------------
 * `Linear::try_forward` (dfdx/src/nn/layers/linear.rs:82-89): x (rows, I)
 * with strides x_strides, weight stored (O, I) row-major and consumed through
 * its zero-copy (I, O) view, bias (O,) or NULL; out (rows, O) contiguous.
 * A (B, S, I) input is passed with rows = B*S when contiguous. */
int dfdx_rocm_linear_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t in_dim, int64_t out_dim,
                             const void *x, const int64_t x_strides[2], const void *weight, const void *bias,
                             void *out);

/* Backward of the same Linear: grad_x (through x_strides) += grad_out . W,
 * grad_weight (O, I) += grad_out^T . x, grad_bias (O,) += column sums of
 * grad_out; grad_out is (rows, O) contiguous.  The two products are the
 * MatMat backward on the weight's permuted view (linear.rs:85-86 with
 * matmul/mod.rs:116-131); the bias term is the backward of the broadcast
 * add (bias1d.rs:62-78).  grad_bias may be NULL. */
int dfdx_rocm_linear_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t in_dim, int64_t out_dim,
                              const void *x, const int64_t x_strides[2], void *grad_x, const void *weight,
                              void *grad_weight, void *grad_bias, const void *grad_out);

/* ---- Bias1D ------------------------------------------------------------------
 * `Bias1D::try_forward` (dfdx/src/nn/layers/bias1d.rs:62-78): the (cols,)
 * bias is broadcast over every leading axis of a contiguous input and added;
 * a (B, S, cols) input is passed with rows = B*S.  out may be x. */
int dfdx_rocm_bias_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *bias,
                           void *out);
/* Backward of that add for the broadcast operand (binary-op backward through
 * a broadcast view, dfdx-core/src/tensor_ops/utilities/cpu_kernels.rs:164-203):
 * grad_bias[c] += sum over rows of grad_out[r][c].  The reference adds row
 * after row in the storage type; here the column is summed in f32 and rounded
 * once.  (grad_x of the add is grad_out itself and needs no kernel.) */
int dfdx_rocm_bias_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *grad_out,
                            void *grad_bias);

/* ---- The ops between attention's GEMMs ---------------------------------------
 * MultiHeadAttention::try_forward (dfdx/src/nn/layers/multi_head_attention.rs:
 * 105-146) runs, between its matmuls, a multiplication by a scalar, a softmax
 * over the last axis and one reshape of a permuted tensor.  These entry points
 * keep those on the device. */

/* `t * scalar` (ScalarMulKernelOp, dfdx-core/src/tensor_ops/mul/cpu_kernel.rs:
 * 5-17, run by the unary kernel over the tensor's physical storage,
 * utilities/cpu_kernels.rs:46-109): out[i] = x[i] * s for i < len, with s
 * rounded to the element type first; out may be x.  Backward:
 * grad_inp[i] += s * grad_out[i]. */
int dfdx_rocm_scalar_mul_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, double scalar, void *out);
int dfdx_rocm_scalar_mul_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, double scalar, void *grad_inp,
                                  const void *grad_out);

/* Softmax over the last axis of a contiguous (rows, cols) matrix
 * (`try_softmax::<Axis<3>>`, dfdx-core/src/tensor_ops/softmax.rs:70-83:
 * exp(t - max) / sum exp(t - max)), applied to scale * x so that attention's
 * scalar multiplication can be folded in (scale = 1 for a plain softmax).
 * The reference composes it from max / sub / exp / sum / div kernels, each
 * rounding to the element type; here a row is processed in f32 (f64 rows in
 * f64) and rounded once.  `scale` is a float: an f64 caller whose scalar has
 * no exact float value applies dfdx_rocm_scalar_mul_forward first and passes
 * 1.  out may be x.  Backward of the composition, from the saved output:
 * grad_x[r][c] += scale * out[r][c] * (grad_out[r][c] - sum_j grad_out[r][j] * out[r][j]). */
int dfdx_rocm_softmax_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, float scale,
                              void *out);
int dfdx_rocm_softmax_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *out, float scale,
                               void *grad_x, const void *grad_out);

/* ReshapeKernel (dfdx-core/src/tensor_ops/reshape_to/mod.rs:90-115,
 * cpu_kernel.rs:7-35) for a view that is not contiguous: forward copies the
 * view's elements, in logical row-major order, into the contiguous `out`;
 * backward adds grad_out (contiguous) into grad_inp through the view's
 * strides.  rank <= 6, strides in elements.  A zero stride on an axis longer
 * than 1 (a broadcast view) is read repeatedly by forward; backward sums the
 * grad_out elements that the view maps onto one grad_inp element
 * (cpu_kernel.rs:28-32 adds them one after the other; here in f32, rounded
 * once). */
int dfdx_rocm_reshape_forward(dfdx_rocm_ctx *ctx, int dtype, int rank, const int64_t *shape, const int64_t *inp_strides,
                              const void *inp, void *out);
int dfdx_rocm_reshape_backward(dfdx_rocm_ctx *ctx, int dtype, int rank, const int64_t *shape, const int64_t *inp_strides,
                               void *grad_inp, const void *grad_out);

/* ---- The ops between a transformer encoder block's GEMMs ----------------------
 * TransformerEncoderBlock (dfdx/src/nn/layers/transformer.rs:24-48) is
 * ResidualAdd<MultiHeadAttention>, LayerNorm1D, ResidualAdd<(Linear, ReLU,
 * Linear)>, LayerNorm1D.  These entry points keep the three ops that are not
 * matmuls on the device. */

/* LayerNorm1D over the last axis of a contiguous (rows, cols) matrix
 * (dfdx/src/nn/layers/layer_norm1d.rs:87-91: normalize, multiply by gamma, add
 * beta; normalize = (t - mean) / sqrt(mean((t - mean)^2) + epsilon),
 * dfdx-core/src/tensor_ops/normalize.rs:35-49).  The reference composes it from
 * mean / sub / square / mean / add / sqrt / div / mul / add tensor ops, each
 * rounding to the element type; here a row is processed in f32 and rounded
 * once.  gamma and beta have `cols` elements.  Backward of the composition,
 * from the saved input, with xhat the normalized row and gh = grad_out * gamma:
 *   grad_x     += (gh - mean(gh) - xhat * mean(gh * xhat)) / sqrt(var + epsilon)
 *   grad_gamma += sum over rows of grad_out * xhat
 *   grad_beta  += sum over rows of grad_out. */
int dfdx_rocm_layer_norm_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *gamma,
                                 const void *beta, double epsilon, void *out);
int dfdx_rocm_layer_norm_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t cols, const void *x, const void *gamma,
                                  double epsilon, void *grad_x, void *grad_gamma, void *grad_beta, const void *grad_out);

/* ReLU (ReLUKernelOp, dfdx-core/src/tensor_ops/relu/cpu_kernel.rs:3-18, run by
 * the unary kernel over the tensor's physical storage): out[i] = max(x[i], 0);
 * out may be x.  Backward, from the saved input:
 * grad_x[i] += (x[i] > 0 ? 1 : 0) * grad_out[i]. */
int dfdx_rocm_relu_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, void *out);
int dfdx_rocm_relu_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *x, void *grad_x, const void *grad_out);

/* The binary add of two tensors with the same layout (BinaryAddKernelOp,
 * dfdx-core/src/tensor_ops/add/cpu_kernel.rs:4-26; ResidualAdd::try_forward,
 * dfdx/src/nn/layers/residual_add.rs:38-45): out[i] = lhs[i] + rhs[i]; out may
 * be either operand.  Backward: grad_lhs[i] += grad_out[i] and
 * grad_rhs[i] += grad_out[i] (grad_lhs == grad_rhs, the gradient of t + t,
 * receives grad_out twice). */
int dfdx_rocm_add_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, const void *lhs, const void *rhs, void *out);
int dfdx_rocm_add_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t len, void *grad_lhs, void *grad_rhs, const void *grad_out);

/* ---- conv2d: unfold + batched GEMM, and the forms that avoid its patch matrix -
 * Conv2DKernel (dfdx-core/src/tensor_ops/conv2d/mod.rs:31-55; Cpu impl
 * cpu_kernel.rs:40-278, Cuda impl cuda_kernel.rs:62-281).  The op struct has
 * the fields and order of the reference's #[repr(C)] Conv2DOp (mod.rs:14-29),
 * so the Rust side passes its own value by pointer.  img is (batch, chan_in,
 * h_in, w_in), filters (chan_out, chan_in/groups, kernel, kernel), out
 * (batch, chan_out, h_out, w_out), all contiguous as the reference requires
 * (mod.rs:290-292); an unbatched image is batch = 1.  Forward overwrites out;
 * backward accumulates into grad_img and grad_filters (a grad_img declared zero
 * whose fill is still deferred is stored into instead: same result, no fill).
 * The general form is
 * the reference's: gather the patch matrix, multiply (cpu_kernel.rs:52-170).
 * Which form runs depends on the shape; every form computes the same sums with
 * f32 accumulation and results within the tolerance of the general form, not
 * bit-identical to it:
 *   - 3 x 3 filters at unit stride with padding 1 and whole blocks of channels
 *     run on kernels that keep a band of the image in LDS and form no patch
 *     matrix, forward and both gradients;
 *   - images of fewer than 256 output positions multiply as one product over
 *     the batch (patch matrix [C K K][batch * positions]);
 *   - strided layers, and layers whose image has a quarter of the output's
 *     channels or fewer, take both gradients from the forward patch matrix
 *     (the image gradient's per-tap partial sums are rounded to the element
 *     type before the taps are added in f32);
 *   - depthwise layers (one input channel per group) are computed directly;
 *   - 1 x 1 filters at unit stride use the image itself as the patch matrix. */
typedef struct dfdx_rocm_conv2d_op {
    size_t kernel, stride, padding, dilation, groups, batch, chan_in, chan_out, h_in, h_out, w_in, w_out;
} dfdx_rocm_conv2d_op;

int dfdx_rocm_conv2d_forward(dfdx_rocm_ctx *ctx, int dtype, const dfdx_rocm_conv2d_op *op, const void *img,
                             const void *filters, void *out);
int dfdx_rocm_conv2d_backward(dfdx_rocm_ctx *ctx, int dtype, const dfdx_rocm_conv2d_op *op, const void *img,
                              void *grad_img, const void *filters, void *grad_filters, const void *grad_out);

#ifdef __cplusplus
}
#endif
#endif /* DFDX_ROCM_H */
