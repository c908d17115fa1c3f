// C ABI of the dfdx ROCm matmul backend: context, storage helpers, GEMM dispatch.
#include "ctx_internal.h"
#include "gemm_internal.h"

#include <algorithm>
#include <cstdio>
#include <cstring>

using namespace dfdx_rocm;

namespace dfdx_rocm {

int bind(dfdx_rocm_ctx *ctx) {
    if (!ctx) return DFDX_ROCM_ERR_INVALID_ARG;
    HIP_TRY(hipSetDevice(ctx->device));
    return DFDX_ROCM_OK;
}

// Frees the buffers that `grow` replaced.  The caller has drained the stream.
static hipError_t free_retired(dfdx_rocm_ctx *ctx) {
    hipError_t first = hipSuccess;
    for (void *p : ctx->retired) {
        const hipError_t e = hipFree(p);
        if (first == hipSuccess) first = e;
    }
    ctx->retired.clear();
    return first;
}

// The stream is not drained here: work already queued keeps the old buffer, which is retired, and the call in hand
// gets a new one (only a failed allocation drains, frees what is retired and tries once more).
static int grow(dfdx_rocm_ctx *ctx, void **buf, size_t *have, size_t bytes) {
    CtxLock lock(ctx->mu);
    if (bytes <= *have) return DFDX_ROCM_OK;
    if (*buf) {
        ctx->retired.push_back(*buf);
        *buf = nullptr;
        *have = 0;
    }
    bytes = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    hipError_t e = hipMalloc(buf, bytes);
    if (e == hipErrorOutOfMemory && !ctx->retired.empty()) {
        (void)hipGetLastError();
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        (void)free_retired(ctx);
        e = hipMalloc(buf, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();  // the failed allocation must not surface again in the next launch check
        *buf = nullptr;
        return (int)e;
    }
    *have = bytes;
    return DFDX_ROCM_OK;
}

static std::map<uintptr_t, size_t>::iterator pending_holding(dfdx_rocm_ctx *ctx, uintptr_t p) {
    auto it = ctx->pending_zero.upper_bound(p);
    if (it == ctx->pending_zero.begin()) return ctx->pending_zero.end();
    --it;
    return p < it->first + it->second ? it : ctx->pending_zero.end();
}

static int fill_and_drop(dfdx_rocm_ctx *ctx, std::map<uintptr_t, size_t>::iterator it) {
    const hipError_t e = launch_zero_fill((void *)it->first, it->second, ctx->compute_units, ctx->stream);
    if (e != hipSuccess) return (int)e;
    ctx->pending_zero.erase(it);
    ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
    return DFDX_ROCM_OK;
}

int settle(dfdx_rocm_ctx *ctx, const void *ptr) {
    if (!ptr || ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    CtxLock lock(ctx->mu);
    auto it = pending_holding(ctx, (uintptr_t)ptr);
    return it == ctx->pending_zero.end() ? DFDX_ROCM_OK : fill_and_drop(ctx, it);
}

int settle_output(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes, bool accumulates, bool *fresh) {
    if (fresh) *fresh = false;
    if (!ptr || ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    CtxLock lock(ctx->mu);
    auto it = pending_holding(ctx, (uintptr_t)ptr);
    if (it == ctx->pending_zero.end()) return DFDX_ROCM_OK;
    const bool covered = bytes && it->first == (uintptr_t)ptr && it->second == bytes;
    if (covered && (!accumulates || fresh)) {  // every byte is stored without being read first: no fill needed
        ctx->pending_zero.erase(it);
        ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
        if (fresh) *fresh = accumulates;
        return DFDX_ROCM_OK;
    }
    return fill_and_drop(ctx, it);
}

// Runs every deferred fill that overlaps [ptr, ptr + bytes) (a read of that range follows).
static int settle_range(dfdx_rocm_ctx *ctx, const void *ptr, size_t bytes) {
    if (!ptr || ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    CtxLock lock(ctx->mu);
    const uintptr_t lo = (uintptr_t)ptr, hi = lo + bytes;
    auto first = pending_holding(ctx, lo);
    if (first != ctx->pending_zero.end())
        if (int e = fill_and_drop(ctx, first)) return e;
    for (auto it = ctx->pending_zero.lower_bound(lo); it != ctx->pending_zero.end() && it->first < hi;
         it = ctx->pending_zero.lower_bound(lo))
        if (int e = fill_and_drop(ctx, it)) return e;
    return DFDX_ROCM_OK;
}

// Forgets (without filling) every deferred fill that lies wholly inside [ptr, ptr + bytes); one that straddles an end is run.
static int drop_pending_inside(dfdx_rocm_ctx *ctx, const void *ptr, size_t bytes) {
    if (!ptr || ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    CtxLock lock(ctx->mu);
    const uintptr_t lo = (uintptr_t)ptr, hi = lo + bytes;
    auto first = pending_holding(ctx, lo);
    if (first != ctx->pending_zero.end() && first->first < lo)
        if (int e = fill_and_drop(ctx, first)) return e;
    for (auto it = ctx->pending_zero.lower_bound(lo); it != ctx->pending_zero.end() && it->first < hi;) {
        if (it->first + it->second > hi) {
            if (int e = fill_and_drop(ctx, it)) return e;
            break;
        }
        it = ctx->pending_zero.erase(it);
    }
    ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
    return DFDX_ROCM_OK;
}

int settle_all(dfdx_rocm_ctx *ctx) {
    if (ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    CtxLock lock(ctx->mu);
    while (!ctx->pending_zero.empty())
        if (int e = fill_and_drop(ctx, ctx->pending_zero.begin())) return e;
    return DFDX_ROCM_OK;
}

size_t dense_bytes(int rank, const int64_t *extents, const int64_t *strides, size_t elem_bytes) {
    int64_t ext[8], str[8];
    int n = 0;
    if (rank > 8) return 0;
    for (int i = 0; i < rank; i++) {
        if (extents[i] == 0) return 0;
        if (extents[i] == 1) continue;
        if (strides[i] <= 0) return 0;
        int j = n++;
        for (; j > 0 && str[j - 1] > strides[i]; j--) {  // insertion sort by stride
            ext[j] = ext[j - 1];
            str[j] = str[j - 1];
        }
        ext[j] = extents[i];
        str[j] = strides[i];
    }
    int64_t run = 1;
    for (int i = 0; i < n; i++) {
        if (str[i] != run) return 0;
        run *= ext[i];
    }
    return (size_t)run * elem_bytes;
}

int ensure_workspace(dfdx_rocm_ctx *ctx, size_t bytes) { return grow(ctx, &ctx->workspace, &ctx->workspace_bytes, bytes); }
int ensure_patches(dfdx_rocm_ctx *ctx, size_t bytes) { return grow(ctx, &ctx->patches, &ctx->patches_bytes, bytes); }

}  // namespace dfdx_rocm

namespace {

// Scratch of dfdx_rocm_gemm_noalloc: partial sums of split reductions for callers that may not allocate.  Every device
// the library runs on holds its own copy of this array, at its own address, until the process ends.  In host code the
// array's NAME is only a handle for hipGetSymbolAddress: the address a kernel may use is looked up once per device in
// dfdx_rocm_create (with that device current) and kept in `scratch_of_device` / the context.
__device__ __align__(256) __attribute__((used)) static unsigned char scratch[DFDX_ROCM_NOALLOC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::mutex scratch_mu;
void *scratch_of_device[kMaxDevices];  // guarded by scratch_mu

// The calling thread's current device must be `ordinal`.
int scratch_address(int ordinal, void **out) {
    if (ordinal < 0 || ordinal >= kMaxDevices) return DFDX_ROCM_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(scratch_mu);
    if (!scratch_of_device[ordinal]) {
        void *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return (int)hipErrorInvalidSymbol;
        scratch_of_device[ordinal] = ptr;
    }
    *out = scratch_of_device[ordinal];
    return DFDX_ROCM_OK;
}

// Validates `d` and produces the canonical problem (row-major C whenever the view allows it).
// `colsum_b` (may be null): where the caller would like the sums of B over the contraction; it stays in the problem only
// when the problem is the plain one (no aliased output axis).
int make_problem(const dfdx_rocm_gemm_desc *d, GemmProblem *out, void *colsum_b = nullptr) {
    if (!d) return DFDX_ROCM_ERR_INVALID_ARG;
    if (d->dtype < DFDX_ROCM_F32 || d->dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_INVALID_ARG;
    if (d->m < 0 || d->n < 0 || d->k < 0 || d->batch1 < 1 || d->batch2 < 1) return DFDX_ROCM_ERR_INVALID_ARG;
    if (d->m == 0 || d->n == 0) {
        out->m = 0;
        return DFDX_ROCM_OK;
    }
    if (!d->c || (d->k > 0 && (!d->a || !d->b))) return DFDX_ROCM_ERR_INVALID_ARG;
    if (d->c_rs < 0 || d->c_cs < 0 || d->c_b1 < 0 || d->c_b2 < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (!d->reduce_batch && ((d->batch1 > 1 && d->c_b1 == 0) || (d->batch2 > 1 && d->c_b2 == 0)))
        return DFDX_ROCM_ERR_ALIASED_OUTPUT;
    // An output view with a zero stride along a matrix axis maps a whole row (or column) of logical elements to one
    // address: the gradient of an operand that was broadcast along that axis (matmul/mod.rs:318-320 lets such views
    // in).  The elements that share an address are SUMMED, which is the gradient of a broadcast (the reference's Cpu
    // path lets them overwrite each other, its Cuda path reads past the buffer).  The aliased axis becomes a batch axis
    // of a product with one row (or column), reduced over the batch.
    const bool rows_alias = d->m > 1 && d->c_rs == 0, cols_alias = d->n > 1 && d->c_cs == 0;
    if (rows_alias || cols_alias) {
        if (d->batch1 * d->batch2 != 1 || d->reduce_batch || d->bias) return DFDX_ROCM_ERR_ALIASED_OUTPUT;
        dfdx_rocm_gemm_desc r = *d;
        r.reduce_batch = 1;
        r.c_b1 = r.c_b2 = 0;
        if (rows_alias) {  // C[j] += sum_i sum_k A[i,k] B[k,j]: the rows become batch 1
            r.m = 1;
            r.batch1 = d->m;
            r.a_b1 = d->a_rs;
            r.b_b1 = 0;
            r.c_rs = cols_alias ? 1 : d->n * (d->c_cs > 0 ? d->c_cs : 1);
        }
        if (cols_alias) {  // C[i] += sum_j sum_k A[i,k] B[k,j]: the columns become batch 2
            r.n = 1;
            r.batch2 = d->n;
            r.a_b2 = 0;
            r.b_b2 = d->b_cs;
            r.c_cs = 1;
        }
        r.flags |= DFDX_ROCM_GEMM_NO_SPLIT_K;
        return make_problem(&r, out);
    }
    GemmProblem p;
    p.dtype = d->dtype;
    p.accumulate = d->accumulate != 0;
    p.reduce = d->reduce_batch != 0 && d->batch1 * d->batch2 > 1;
    p.bias_mode = d->bias ? BIAS_PER_COL : BIAS_NONE;
    p.m = d->m; p.n = d->n; p.k = d->k;
    p.nb1 = d->batch1; p.nb2 = d->batch2;
    p.a = d->a; p.a_rs = d->a_rs; p.a_cs = d->a_cs; p.a_b1 = d->a_b1; p.a_b2 = d->a_b2;
    p.b = d->b; p.b_rs = d->b_rs; p.b_cs = d->b_cs; p.b_b1 = d->b_b1; p.b_b2 = d->b_b2;
    p.c = d->c; p.c_rs = d->c_rs; p.c_cs = d->c_cs;
    p.c_b1 = p.reduce ? 0 : d->c_b1; p.c_b2 = p.reduce ? 0 : d->c_b2;
    p.bias = d->bias;
    p.ksum = colsum_b;
    p.ksum_of = colsum_b ? KSUM_OF_B : KSUM_NONE;
    p.ksum_accumulate = 1;
    p.splits = 1;
    p.workspace = nullptr;
    p.compute_units = 0;
    // column-major C (a permuted operand's gradient): compute C^T = B^T A^T instead
    if (p.c_cs != 1 && p.c_rs == 1 && p.n > 1) p = transposed(p);
    *out = p;
    return DFDX_ROCM_OK;
}

// Frees every buffer the cache holds.  Work that may still use them is drained first.
int drop_cache(dfdx_rocm_ctx *ctx) {
    CtxLock lock(ctx->mu);
    if (ctx->cache.empty()) return DFDX_ROCM_OK;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    hipError_t first = free_retired(ctx);
    for (auto &kv : ctx->cache)
        for (void *p : kv.second) {
            const hipError_t e = hipFree(p);
            if (first == hipSuccess) first = e;
        }
    ctx->cache.clear();
    ctx->cache_bytes = 0;
    return (int)first;
}

struct Plan {
    int kernel, variant, splits;
};

// Rank-1 updates and k = 2 stream their rows on the vector ALUs; from k = 3 on the matrix-core form of the thin
// contraction is the faster one wherever it applies (f32 4096 x 8 x 4096: 42.5 against 16.7 us; at k = 2 the vector ALUs
// are level or up to 10 % ahead).
inline bool use_rank1(const GemmProblem &p) {
    return rank1_supported(p) && !(p.k >= 3 && thin_mfma_supported(p));
}

// The bandwidth-bound kernels (`Plan::variant` of a DFDX_ROCM_KERNEL_GEMV plan).
enum { BW_NONE = 0, BW_RANK1 = 1, BW_GEMV_MULTI = 2, BW_GEMV = 3, BW_THIN_MFMA = 4 };

// Which of them takes `p`, if any.  `plain_order`: the caller asked for the contraction order of the tiled kernels
// (DFDX_ROCM_GEMM_NO_SPLIT_K: the broadcast-rhs forward and grad_lhs, whose results must equal those of the batched
// product of the same slices bit for bit, matmul/mod.rs:460-473).  The vector-product kernels cut k into grid slices
// and sum inside a slice in an order of their own, and the vector-ALU form of the thin contraction sums by fused
// multiply-adds, so none of them qualifies; a rank-1 update has nothing to order, and the matrix-core form of the thin
// contraction walks k exactly as the tiles do.
int bandwidth_kernel(const GemmProblem &p, bool plain_order) {
    if (plain_order) {
        if (p.k == 1 && rank1_supported(p)) return BW_RANK1;
        return thin_mfma_supported(p) ? BW_THIN_MFMA : BW_NONE;
    }
    if (use_rank1(p)) return BW_RANK1;
    if (gemv_multi_supported(p)) return BW_GEMV_MULTI;
    if (gemv_supported(p)) return BW_GEMV;
    return thin_mfma_supported(p) ? BW_THIN_MFMA : BW_NONE;
}

const char *bandwidth_kernel_name(const GemmProblem &p, int which) {
    switch (which) {
    case BW_RANK1: return p.k == 1 ? "rank1" : "thin_k";
    case BW_GEMV_MULTI: return "gemv_multi";
    case BW_GEMV: return "gemv";
    case BW_THIN_MFMA: return "thin_k_mfma";
    default: return "none";
    }
}

int make_plan(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *d, const GemmProblem &p, Plan *plan) {
    const bool is16 = p.dtype == DT_F16 || p.dtype == DT_BF16;
    const bool is32 = p.dtype == DT_F32, is64 = p.dtype == DT_F64;
    // split-k: 1 = never (NO_SPLIT_K), n = forced by the caller, 0 = let the planner decide
    const int forced_splits = (d->flags & DFDX_ROCM_GEMM_NO_SPLIT_K) ? 1 : ((d->flags >> 8) & 0xff);
    switch (d->kernel) {
    case DFDX_ROCM_KERNEL_GENERIC:
        *plan = {DFDX_ROCM_KERNEL_GENERIC, 0, 1};
        return DFDX_ROCM_OK;
    case DFDX_ROCM_KERNEL_GEMV: {  // the bandwidth-bound kernels, forced: the caller's choice outranks the order flag
        const int bw = bandwidth_kernel(p, false);
        if (!bw) return DFDX_ROCM_ERR_UNSUPPORTED;
        *plan = {DFDX_ROCM_KERNEL_GEMV, bw, 1};
        return DFDX_ROCM_OK;
    }
    case DFDX_ROCM_KERNEL_MFMA: {
        int v = d->variant;
        if (is16 && (v == 0 || (v >= mfma16_dma_first_variant() && v != mfma16_small_variant()))) {  // LDS-DMA family: tile and split count together
            int dv = 0, splits = 1;
            mfma16dma_plan_split(p, ctx->compute_units, v ? v - mfma16_dma_first_variant() + 1 : 0, forced_splits, &dv, &splits);
            if (dv) {
                *plan = {DFDX_ROCM_KERNEL_MFMA, dv + mfma16_dma_first_variant() - 1, splits};
                return DFDX_ROCM_OK;
            }
            if (v) return DFDX_ROCM_ERR_UNSUPPORTED;
        }
        if (v == 0)
            v = is16 ? mfma16_pick_variant(p, ctx->compute_units)
                     : is32 ? mfma32_pick_variant(p, ctx->compute_units, forced_splits) : is64 ? mfma64_pick_variant(p, ctx->compute_units) : 0;
        const bool ok = is16 ? mfma16_supported(p, v) : is32 ? mfma32_supported(p, v) : is64 ? mfma64_supported(p, v) : false;
        if (!ok) return DFDX_ROCM_ERR_UNSUPPORTED;
        *plan = {DFDX_ROCM_KERNEL_MFMA, v,
                 is32 ? mfma32_plan_splits(p, v, ctx->compute_units, forced_splits)
                      : is16 ? mfma16_plan_splits(p, v, ctx->compute_units, forced_splits) : 1};
        return DFDX_ROCM_OK;
    }
    case DFDX_ROCM_KERNEL_AUTO:
        break;
    default:
        return DFDX_ROCM_ERR_INVALID_ARG;
    }
    // The bandwidth-bound kernels first.  The multi-vector form is weighed against the matrix-core plans by estimated
    // time (the k-sliced small kernel streams a [n][k] matrix faster for most sizes, the tiles a large [k][n] one); the
    // others have no rival.
    const int bw = bandwidth_kernel(p, (d->flags & DFDX_ROCM_GEMM_NO_SPLIT_K) != 0);
    double t_bw = 1e300;
    if (bw == BW_GEMV_MULTI) {
        t_bw = gemv_multi_time(p);
    } else if (bw) {
        *plan = {DFDX_ROCM_KERNEL_GEMV, bw, 1};
        return DFDX_ROCM_OK;
    }
    const Plan bw_plan = {DFDX_ROCM_KERNEL_GEMV, BW_GEMV_MULTI, 1};
    // The small-product kernel where its estimate beats the family's (the f32 family weighs it among its own variants);
    // not where the caller fixed the order of the contraction.
    const bool may_small = forced_splits == 0 && (is16 || is64) && small_supported(p);
    const double t_small = may_small ? small_time(p, ctx->compute_units) : 1e300;
    const Plan small_plan = {DFDX_ROCM_KERNEL_MFMA, is16 ? mfma16_small_variant() : mfma64_small_variant(), 1};
    if (is16) {
        int dv = 0, splits = 1;
        double t_dma = 1e300;
        mfma16dma_plan_split(p, ctx->compute_units, 0, forced_splits, &dv, &splits, &t_dma);
        if (dv) {
            // that family's estimate ranks its own tiles and split counts; on products of a few microseconds it runs
            // 1 - 2 us above the clock, and 8 us above it for a split plan
            t_dma -= splits > 1 ? 6.5e-6 : 1.0e-6;
            *plan = t_small < t_dma ? small_plan : Plan{DFDX_ROCM_KERNEL_MFMA, dv + mfma16_dma_first_variant() - 1, splits};
            double t_best = std::min(t_small, t_dma);
            int skinny_splits = 1;
            double t_skinny = 1e300;
            if (const int sv = mfma16_skinny_plan(p, ctx->compute_units, forced_splits, &skinny_splits, &t_skinny)) {
                if (t_skinny < t_best) {
                    *plan = {DFDX_ROCM_KERNEL_MFMA, sv, skinny_splits};
                    t_best = t_skinny;
                }
            }
            if (t_bw < t_best) *plan = bw_plan;
            return DFDX_ROCM_OK;
        }
    }
    double t_family = 1e300;
    int v = is16 ? mfma16_pick_variant(p, ctx->compute_units)
                 : is32 ? mfma32_pick_variant(p, ctx->compute_units, forced_splits, &t_family) : is64 ? mfma64_pick_variant(p, ctx->compute_units) : 0;
    if (v > 0) {
        *plan = {DFDX_ROCM_KERNEL_MFMA, v,
                 is32 ? mfma32_plan_splits(p, v, ctx->compute_units, forced_splits)
                      : is16 ? mfma16_plan_splits(p, v, ctx->compute_units, forced_splits) : 1};
        if (!is32) t_family = is16 ? mfma16_staged_time(p, v, plan->splits, ctx->compute_units) : mfma64_time(p, v, ctx->compute_units);
        if (may_small && t_small < t_family) *plan = small_plan;
        if (t_bw < std::min(t_small, t_family)) *plan = bw_plan;
        return DFDX_ROCM_OK;
    }
    if (bw) {  // no tiled kernel takes these strides, the multi-vector kernel does
        *plan = t_small < t_bw ? small_plan : bw_plan;
        return DFDX_ROCM_OK;
    }
    // no tiled kernel takes these strides: the small-product kernel takes any, up to the size where 16 x 16 tiles pay
    if (may_small && (double)p.m * (double)p.n * (double)p.k <= 134217728.0) {
        *plan = small_plan;
        return DFDX_ROCM_OK;
    }
    *plan = {DFDX_ROCM_KERNEL_GENERIC, 0, 1};
    return DFDX_ROCM_OK;
}

// Where the partial sums of a split plan go: the context's own buffer (grown on demand), or -- `static_scratch` --
// the device's fixed scratch array, in which case nothing is allocated and a plan that needs more is refused.
int partials_buffer(dfdx_rocm_ctx *ctx, size_t need, bool static_scratch, float **out) {
    if (static_scratch) {
        if (need > (size_t)DFDX_ROCM_NOALLOC_SCRATCH_BYTES) return DFDX_ROCM_ERR_SCRATCH_TOO_SMALL;
        if (!ctx->static_scratch) return DFDX_ROCM_ERR_INVALID_ARG;
        *out = (float *)ctx->static_scratch;
        return DFDX_ROCM_OK;
    }
    if (int rc = ensure_workspace(ctx, need)) return rc;
    *out = (float *)ctx->workspace;
    return DFDX_ROCM_OK;
}

// The f32 partial sums `plan` needs for `p`, in bytes (0: none).
size_t partials_bytes(const GemmProblem &p, const Plan &plan) {
    if (plan.kernel == DFDX_ROCM_KERNEL_MFMA && plan.splits > 1)
        return p.dtype == DT_F32 ? mfma32_workspace_bytes(p, plan.variant, plan.splits)
               : plan.variant < mfma16_dma_first_variant()
                   ? mfma16_workspace_bytes(p, plan.variant, plan.splits)
                   : mfma16dma_workspace_bytes(p, plan.variant - mfma16_dma_first_variant() + 1, plan.splits);
    if (plan.kernel == DFDX_ROCM_KERNEL_GEMV && plan.variant == BW_GEMV_MULTI) return gemv_multi_workspace_bytes(p);
    if (plan.kernel == DFDX_ROCM_KERNEL_GEMV && plan.variant == BW_GEMV) return gemv_workspace_bytes(p);
    return 0;
}

// Makes sure the partial sums of `plan` have a place, BEFORE the caller resolves pending zero fills among the operands:
// a call that is refused here (scratch too small, out of memory) must leave every declaration as it found it.
int reserve_partials(dfdx_rocm_ctx *ctx, const GemmProblem &problem, const Plan &plan, bool static_scratch) {
    GemmProblem p = problem;
    p.compute_units = ctx->compute_units;
    float *unused = nullptr;
    const size_t need = partials_bytes(p, plan);
    return need ? partials_buffer(ctx, need, static_scratch, &unused) : DFDX_ROCM_OK;
}

int run_plan(dfdx_rocm_ctx *ctx, const GemmProblem &problem, const Plan &plan, bool static_scratch = false) {
    CtxLock lock(ctx->mu);  // a split plan is two launches around the shared workspace
    GemmProblem p = problem;
    p.splits = 1;
    p.workspace = nullptr;
    p.compute_units = ctx->compute_units;
    if (const size_t need = partials_bytes(p, plan)) {
        if (int rc = partials_buffer(ctx, need, static_scratch, &p.workspace)) return rc;
    }
    if (plan.kernel == DFDX_ROCM_KERNEL_MFMA && plan.splits > 1) p.splits = plan.splits;
    hipError_t e;
    switch (plan.kernel) {
    case DFDX_ROCM_KERNEL_GENERIC: e = launch_generic(p, ctx->stream); break;
    case DFDX_ROCM_KERNEL_GEMV:
        e = plan.variant == BW_RANK1 ? launch_rank1(p, ctx->stream)
            : plan.variant == BW_GEMV_MULTI ? launch_gemv_multi(p, ctx->stream)
            : plan.variant == BW_GEMV ? launch_gemv(p, ctx->stream)
            : plan.variant == BW_THIN_MFMA ? launch_thin_mfma(p, ctx->stream) : hipErrorInvalidValue;
        break;
    case DFDX_ROCM_KERNEL_MFMA:
        e = (p.dtype == DT_F32) ? launch_mfma32(p, plan.variant, ctx->stream)
                                : (p.dtype == DT_F64) ? launch_mfma64(p, plan.variant, ctx->stream) : launch_mfma16(p, plan.variant, ctx->stream);
        break;
    default: return DFDX_ROCM_ERR_INVALID_ARG;
    }
    return (int)e;
}

// Deferred zero fills among the operands: inputs are filled now; an accumulation that covers the whole of a pending C
// becomes a plain store (`may_overwrite`), which leaves the same bits as 0 + value.
int settle_operands(dfdx_rocm_ctx *ctx, GemmProblem *p, bool may_overwrite) {
    if (ctx->pending_count.load(std::memory_order_acquire) == 0) return DFDX_ROCM_OK;
    if (p->k > 0) {
        if (int e = settle(ctx, p->a)) return e;
        if (int e = settle(ctx, p->b)) return e;
    }
    if (int e = settle(ctx, p->bias)) return e;
    const int64_t ext[4] = {p->reduce ? 1 : p->nb1, p->reduce ? 1 : p->nb2, p->m, p->n};
    const int64_t str[4] = {p->c_b1, p->c_b2, p->c_rs, p->c_cs};
    const size_t es = p->dtype == DT_F64 ? 8 : p->dtype == DT_F32 ? 4 : 2;
    bool fresh = false;
    if (int e = settle_output(ctx, p->c, dense_bytes(4, ext, str, es), p->accumulate, may_overwrite ? &fresh : nullptr)) return e;
    if (fresh) p->accumulate = false;
    return DFDX_ROCM_OK;
}

}  // namespace

namespace dfdx_rocm {

int gemm_with_colsum(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, void *colsum_b, bool *fused) {
    *fused = false;
    if (int e = bind(ctx)) return e;
    GemmProblem p;
    if (int e = make_problem(desc, &p, colsum_b)) return e;
    if (p.m == 0) return DFDX_ROCM_OK;
    Plan plan;  // from the product as the caller states it: a pending zero fill of C must not change which kernel runs
    if (int e = make_plan(ctx, desc, p, &plan)) return e;
    if (int e = reserve_partials(ctx, p, plan, false)) return e;
    if (int e = settle_operands(ctx, &p, /*may_overwrite=*/true)) return e;
    bool can = p.ksum && plan.kernel == DFDX_ROCM_KERNEL_MFMA;
    if (can && (p.dtype == DT_F16 || p.dtype == DT_BF16))
        can = plan.variant == mfma16_small_variant()
                  ? small_ksum_supported(p)
                  : plan.variant >= mfma16_dma_first_variant() &&
                        mfma16dma_ksum_supported(p, plan.variant - mfma16_dma_first_variant() + 1, plan.splits);
    else if (can && p.dtype == DT_F32)
        can = plan.splits <= 1 && mfma32_ksum_supported(p, plan.variant);
    else if (can && p.dtype == DT_F64)
        can = plan.variant == mfma64_small_variant() && small_ksum_supported(p);
    else
        can = false;
    if (can) {
        bool fresh = false;
        const int64_t len = p.ksum_of == KSUM_OF_A ? p.m : p.n;
        if (int e = settle_output(ctx, p.ksum, (size_t)len * dtype_size(p.dtype), true, &fresh)) return e;
        p.ksum_accumulate = !fresh;
        *fused = true;
    } else {
        p.ksum = nullptr;
        p.ksum_of = KSUM_NONE;
    }
    return run_plan(ctx, p, plan);
}

}  // namespace dfdx_rocm

extern "C" {

int dfdx_rocm_create(int ordinal, void *stream, dfdx_rocm_ctx **out) {
    if (!out || ordinal < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || ordinal >= count) return DFDX_ROCM_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, ordinal));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) return DFDX_ROCM_ERR_NO_DEVICE;  // code objects are gfx950 only
    HIP_TRY(hipSetDevice(ordinal));
    void *static_scratch = nullptr;
    if (int e = scratch_address(ordinal, &static_scratch)) return e;
    dfdx_rocm_ctx *ctx = new (std::nothrow) dfdx_rocm_ctx();
    if (!ctx) return (int)hipErrorOutOfMemory;
    ctx->static_scratch = static_scratch;
    ctx->device = ordinal;
    ctx->stream = (hipStream_t)stream;
    ctx->compute_units = prop.multiProcessorCount;
    ctx->clock_mhz = prop.clockRate / 1000;
    std::snprintf(ctx->name, sizeof(ctx->name), "%s (%s)", prop.name, prop.gcnArchName);
    *out = ctx;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_destroy(dfdx_rocm_ctx *ctx) {
    if (!ctx) return DFDX_ROCM_OK;
    if (ctx->workspace || ctx->patches || !ctx->retired.empty() || !ctx->cache.empty() || ctx->pending_count.load()) {
        (void)hipSetDevice(ctx->device);
        (void)settle_all(ctx);  // the caller's buffers outlive the context: they must hold the zeros they were promised
        (void)hipStreamSynchronize(ctx->stream);
        (void)free_retired(ctx);
        if (ctx->workspace) (void)hipFree(ctx->workspace);
        if (ctx->patches) (void)hipFree(ctx->patches);
        (void)drop_cache(ctx);
    }
    delete ctx;
    return DFDX_ROCM_OK;
}

const char *dfdx_rocm_strerror(int code) {
    switch (code) {
    case DFDX_ROCM_OK: return "ok";
    case DFDX_ROCM_ERR_INVALID_ARG: return "dfdx_rocm: invalid argument";
    case DFDX_ROCM_ERR_UNSUPPORTED: return "dfdx_rocm: no kernel for this request";
    case DFDX_ROCM_ERR_NO_DEVICE: return "dfdx_rocm: no usable gfx950 device";
    case DFDX_ROCM_ERR_ALIASED_OUTPUT: return "dfdx_rocm: output view aliases itself (zero stride)";
    case DFDX_ROCM_ERR_SCRATCH_TOO_SMALL:
        return "dfdx_rocm: the split reduction of this product needs more than the fixed scratch of the no-allocation entry";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "dfdx_rocm: unknown error";
}

int dfdx_rocm_device_info(dfdx_rocm_ctx *ctx, char *name, size_t name_len, int *compute_units, int *clock_mhz) {
    if (!ctx) return DFDX_ROCM_ERR_INVALID_ARG;
    if (name && name_len) std::snprintf(name, name_len, "%s", ctx->name);
    if (compute_units) *compute_units = ctx->compute_units;
    if (clock_mhz) *clock_mhz = ctx->clock_mhz;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_alloc(dfdx_rocm_ctx *ctx, size_t bytes, int zeroed, void **out) {
    if (!out) return DFDX_ROCM_ERR_INVALID_ARG;
    *out = nullptr;
    if (int e = bind(ctx)) return e;
    if (bytes == 0) bytes = 16;
    void *p = nullptr;
    bool recycled = false;
    {   // a cached buffer of exactly this size, if the cache is on and has one (cache.rs:105-149)
        CtxLock lock(ctx->mu);
        if (ctx->cache_enabled) {
            auto it = ctx->cache.find(bytes);
            if (it != ctx->cache.end()) {
                p = it->second.back();
                it->second.pop_back();
                if (it->second.empty()) ctx->cache.erase(it);
                ctx->cache_bytes -= bytes;
                recycled = true;
            }
        }
    }
    if (!recycled) {
        const hipError_t e = hipMalloc(&p, bytes);
        if (e == hipErrorOutOfMemory) {
            // once more with everything the context can give back: the cached buffers and the outgrown workspaces
            (void)hipGetLastError();
            (void)dfdx_rocm_empty_cache(ctx);
            {
                CtxLock lock(ctx->mu);
                if (!ctx->retired.empty()) {
                    HIP_TRY(hipStreamSynchronize(ctx->stream));
                    (void)free_retired(ctx);
                }
            }
            const hipError_t again = hipMalloc(&p, bytes);
            if (again != hipSuccess) {
                (void)hipGetLastError();
                return (int)again;
            }
        } else if (e != hipSuccess) {
            (void)hipGetLastError();
            return (int)e;
        }
        CtxLock lock(ctx->mu);
        ctx->sizes[p] = bytes;
    }
    if (zeroed == DFDX_ROCM_ZERO_DEFERRED) {
        CtxLock lock(ctx->mu);
        ctx->pending_zero[(uintptr_t)p] = bytes;
        ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
    } else if (zeroed) {
        hipError_t e = launch_zero_fill(p, bytes, ctx->compute_units, ctx->stream);
        if (e != hipSuccess) {
            (void)dfdx_rocm_free(ctx, p);
            return (int)e;
        }
    }
    *out = p;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_free(dfdx_rocm_ctx *ctx, void *ptr) {
    if (int e = bind(ctx)) return e;
    if (!ptr) return DFDX_ROCM_OK;
    {
        CtxLock lock(ctx->mu);
        auto it = ctx->sizes.find(ptr);
        if (ctx->pending_count.load(std::memory_order_acquire)) {  // a fill nobody waited for is not run
            if (it != ctx->sizes.end()) {
                if (int e = drop_pending_inside(ctx, ptr, it->second)) return e;
            } else if (ctx->pending_zero.erase((uintptr_t)ptr)) {
                ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
            }
        }
        if (it != ctx->sizes.end() && ctx->cache_enabled) {
            // Kept for the next allocation of this size.  No synchronisation: whoever gets the buffer next uses it
            // through this context's stream, behind the work that still reads it.
            ctx->cache[it->second].push_back(ptr);
            ctx->cache_bytes += it->second;
            return DFDX_ROCM_OK;
        }
        if (it != ctx->sizes.end()) ctx->sizes.erase(it);
    }
    HIP_TRY(hipStreamSynchronize(ctx->stream));  // pending kernels may still use the buffer
    HIP_TRY(hipFree(ptr));
    CtxLock lock(ctx->mu);
    HIP_TRY(free_retired(ctx));  // the stream is drained: nothing uses the outgrown workspaces either
    return DFDX_ROCM_OK;
}

int dfdx_rocm_enable_cache(dfdx_rocm_ctx *ctx) {
    if (!ctx) return DFDX_ROCM_ERR_INVALID_ARG;
    CtxLock lock(ctx->mu);
    ctx->cache_enabled = true;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_disable_cache(dfdx_rocm_ctx *ctx) {
    if (int e = bind(ctx)) return e;
    {
        CtxLock lock(ctx->mu);
        ctx->cache_enabled = false;
    }
    return dfdx_rocm_empty_cache(ctx);
}

int dfdx_rocm_empty_cache(dfdx_rocm_ctx *ctx) {
    if (int e = bind(ctx)) return e;
    CtxLock lock(ctx->mu);
    for (auto &kv : ctx->cache)
        for (void *p : kv.second) ctx->sizes.erase(p);
    return drop_cache(ctx);
}

int dfdx_rocm_cache_stats(dfdx_rocm_ctx *ctx, size_t *buffers, size_t *bytes) {
    if (!ctx) return DFDX_ROCM_ERR_INVALID_ARG;
    CtxLock lock(ctx->mu);
    size_t n = 0;
    for (auto &kv : ctx->cache) n += kv.second.size();
    if (buffers) *buffers = n;
    if (bytes) *bytes = ctx->cache_bytes;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_memset_zero(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if (!ptr && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    if (bytes) {
        if (int e = drop_pending_inside(ctx, ptr, bytes)) return e;
        HIP_TRY(launch_zero_fill(ptr, bytes, ctx->compute_units, ctx->stream));
    }
    return DFDX_ROCM_OK;
}

int dfdx_rocm_zero_deferred(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if (!ptr && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    if (!bytes) return DFDX_ROCM_OK;
    if (int e = drop_pending_inside(ctx, ptr, bytes)) return e;  // earlier declarations inside the range are replaced
    CtxLock lock(ctx->mu);
    if (pending_holding(ctx, (uintptr_t)ptr) != ctx->pending_zero.end())  // still inside a larger pending buffer
        return DFDX_ROCM_OK;                                             // which already stands for these zeros
    ctx->pending_zero[(uintptr_t)ptr] = bytes;
    ctx->pending_count.store((int)ctx->pending_zero.size(), std::memory_order_release);
    return DFDX_ROCM_OK;
}

int dfdx_rocm_settle_zeros(dfdx_rocm_ctx *ctx) {
    if (int e = bind(ctx)) return e;
    return settle_all(ctx);
}

int dfdx_rocm_forget_zeros(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if (!ptr && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    return bytes ? drop_pending_inside(ctx, ptr, bytes) : DFDX_ROCM_OK;
}

int dfdx_rocm_copy_h2d(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if ((!dst || !src) && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    if (bytes) {
        if (int e = drop_pending_inside(ctx, dst, bytes)) return e;
        HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));  // the host buffer may be reused on return
        CtxLock lock(ctx->mu);
        HIP_TRY(free_retired(ctx));
    }
    return DFDX_ROCM_OK;
}

int dfdx_rocm_copy_d2h(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if ((!dst || !src) && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    if (bytes) {
        if (int e = settle_range(ctx, src, bytes)) return e;
        HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        CtxLock lock(ctx->mu);
        HIP_TRY(free_retired(ctx));
    }
    return DFDX_ROCM_OK;
}

int dfdx_rocm_copy_d2d(dfdx_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    if (int e = bind(ctx)) return e;
    if ((!dst || !src) && bytes) return DFDX_ROCM_ERR_INVALID_ARG;
    if (bytes) {
        if (int e = settle_range(ctx, src, bytes)) return e;
        if (int e = drop_pending_inside(ctx, dst, bytes)) return e;
        HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    }
    return DFDX_ROCM_OK;
}

int dfdx_rocm_synchronize(dfdx_rocm_ctx *ctx) {
    if (int e = bind(ctx)) return e;
    if (int e = settle_all(ctx)) return e;  // whoever reads the memory after this call must find the zeros
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    CtxLock lock(ctx->mu);
    HIP_TRY(free_retired(ctx));  // workspaces outgrown since the last call: nothing on the stream uses them any more
    return DFDX_ROCM_OK;
}

int dfdx_rocm_gemm(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc) {
    if (int e = bind(ctx)) return e;
    GemmProblem p;
    if (int e = make_problem(desc, &p)) return e;
    if (p.m == 0) return DFDX_ROCM_OK;
    Plan plan;  // from the product as the caller states it: a pending zero fill of C must not change which kernel runs
    if (int e = make_plan(ctx, desc, p, &plan)) return e;
    if (int e = reserve_partials(ctx, p, plan, false)) return e;
    if (int e = settle_operands(ctx, &p, /*may_overwrite=*/true)) return e;
    return run_plan(ctx, p, plan);
}

int dfdx_rocm_gemm_noalloc(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc) {
    if (int e = bind(ctx)) return e;
    GemmProblem p;
    if (int e = make_problem(desc, &p)) return e;
    if (p.m == 0) return DFDX_ROCM_OK;
    Plan plan;  // from the product as the caller states it: a pending zero fill of C must not change which kernel runs
    if (int e = make_plan(ctx, desc, p, &plan)) return e;
    if (int e = reserve_partials(ctx, p, plan, /*static_scratch=*/true)) return e;
    if (int e = settle_operands(ctx, &p, /*may_overwrite=*/true)) return e;
    return run_plan(ctx, p, plan, /*static_scratch=*/true);
}

int dfdx_rocm_gemm_plan(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, int *kernel, int *variant, char *name,
                        size_t name_len) {
    if (!ctx) return DFDX_ROCM_ERR_INVALID_ARG;
    GemmProblem p;
    if (int e = make_problem(desc, &p)) return e;
    Plan plan = {DFDX_ROCM_KERNEL_GENERIC, 0, 1};
    if (p.m != 0)
        if (int e = make_plan(ctx, desc, p, &plan)) return e;
    if (kernel) *kernel = plan.kernel;
    if (variant) *variant = plan.kernel == DFDX_ROCM_KERNEL_GEMV ? 0 : plan.variant;  // (a tile variant; the bandwidth kernels have none)
    if (name && name_len) {
        if (plan.kernel == DFDX_ROCM_KERNEL_MFMA && plan.splits > 1)
            std::snprintf(name, name_len, "%s_%s_splitk%d", p.dtype == DT_F32 ? "mfma32" : "mfma16",
                          p.dtype == DT_F32 ? mfma32_variant_name(plan.variant) : mfma16_variant_name(plan.variant), plan.splits);
        else if (plan.kernel == DFDX_ROCM_KERNEL_MFMA && p.dtype == DT_F64)
            std::snprintf(name, name_len, "mfma64_%s", mfma64_variant_name(plan.variant));
        else if (plan.kernel == DFDX_ROCM_KERNEL_MFMA)
            std::snprintf(name, name_len, "%s_%s", p.dtype == DT_F32 ? "mfma32" : "mfma16",
                          p.dtype == DT_F32 ? mfma32_variant_name(plan.variant) : mfma16_variant_name(plan.variant));
        else
            std::snprintf(name, name_len, "%s", plan.kernel != DFDX_ROCM_KERNEL_GEMV ? "generic" : bandwidth_kernel_name(p, plan.variant));
    }
    return DFDX_ROCM_OK;
}

int dfdx_rocm_mfma_variant_count(int dtype) {
    if (dtype == DFDX_ROCM_F16 || dtype == DFDX_ROCM_BF16) return mfma16_variant_count();
    if (dtype == DFDX_ROCM_F32) return mfma32_variant_count();
    if (dtype == DFDX_ROCM_F64) return mfma64_variant_count();
    return 0;
}

int dfdx_rocm_gemm_time_rotating(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *descs, int count, int warmup, int iters,
                                 float *avg_ms) {
    if (!avg_ms || !descs || count < 1 || iters < 1 || warmup < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (int e = bind(ctx)) return e;
    std::vector<GemmProblem> problems((size_t)count);
    std::vector<Plan> plans((size_t)count);
    for (int i = 0; i < count; i++) {
        if (int e = make_problem(&descs[i], &problems[(size_t)i])) return e;
        if (problems[(size_t)i].m == 0) {   // an empty product launches nothing: there is no time to report
            *avg_ms = 0.0f;
            return DFDX_ROCM_OK;
        }
        if (int e = make_plan(ctx, &descs[i], problems[(size_t)i], &plans[(size_t)i])) return e;
        if (int e = settle_operands(ctx, &problems[(size_t)i], /*may_overwrite=*/false)) return e;
    }
    for (int i = 0; i < warmup; i++)
        if (int e = run_plan(ctx, problems[(size_t)(i % count)], plans[(size_t)(i % count)])) return e;
    hipEvent_t t0, t1;
    HIP_TRY(hipEventCreate(&t0));
    HIP_TRY(hipEventCreate(&t1));
    int rc = DFDX_ROCM_OK;
    hipError_t he = hipEventRecord(t0, ctx->stream);
    for (int i = 0; i < iters && rc == DFDX_ROCM_OK && he == hipSuccess; i++)
        rc = run_plan(ctx, problems[(size_t)(i % count)], plans[(size_t)(i % count)]);
    if (he == hipSuccess) he = hipEventRecord(t1, ctx->stream);
    if (he == hipSuccess) he = hipEventSynchronize(t1);
    float ms = 0.0f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, t0, t1);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    if (rc != DFDX_ROCM_OK) return rc;
    if (he != hipSuccess) return (int)he;
    *avg_ms = ms / (float)iters;
    return DFDX_ROCM_OK;
}

int dfdx_rocm_gemm_time(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, int warmup, int iters, float *avg_ms) {
    return dfdx_rocm_gemm_time_rotating(ctx, desc, desc ? 1 : 0, warmup, iters, avg_ms);
}

}  // extern "C"
