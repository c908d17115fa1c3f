// The library context as the host-side sources see it (the C ABI only exposes an opaque pointer).
#pragma once
#include "../../include/dfdx_rocm.h"

#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdint>
#include <map>
#include <mutex>
#include <vector>

struct dfdx_rocm_ctx {
    int device;
    hipStream_t stream;
    int compute_units;
    int clock_mhz;
    char name[128];
    // Serialises every call sequence that uses `workspace` or `patches` (several launches that must not
    // interleave with another host thread's on the same stream); recursive because conv2d holds it across its GEMMs.
    std::recursive_mutex mu;
    void *workspace = nullptr;  // partial sums of split reductions; grown on demand, owned by the context
    size_t workspace_bytes = 0;
    // Outgrown workspace / patch buffers.  Launches already on the stream may still use them, so they are not freed where
    // they are replaced (that would mean draining the stream in the middle of a GEMM call) but at the next
    // dfdx_rocm_synchronize, at destroy, or when an allocation fails for lack of memory.
    std::vector<void *> retired;
    void *static_scratch = nullptr;  // this device's copy of the fixed scratch array of dfdx_rocm_gemm_noalloc (never freed)
    // The allocation cache (tensor/cache.rs:36-149): freed buffers kept by size for the next dfdx_rocm_alloc of that size.
    // Off until dfdx_rocm_enable_cache.  The reference keys on (bytes, element size, alignment) because the Rust
    // allocator wants a buffer back with the layout it was made with; device allocations are all 256 B-aligned raw
    // bytes, so the key here is the byte count.
    bool cache_enabled = false;
    std::map<size_t, std::vector<void *>> cache;
    size_t cache_bytes = 0;
    std::map<void *, size_t> sizes;  // every live buffer of dfdx_rocm_alloc (free learns the size from here)
    // Buffers declared zero whose fill has not run (start address -> bytes): dfdx_rocm_alloc with
    // DFDX_ROCM_ZERO_DEFERRED and dfdx_rocm_zero_deferred put them here.  The first call that reads such a buffer, or
    // writes part of it, runs the fill; a call that accumulates into ALL of it takes it out and stores 0 + value.
    std::map<uintptr_t, size_t> pending_zero;
    std::atomic<int> pending_count{0};  // pending_zero.size(), readable without the lock
    void *patches = nullptr;  // unfolded images of conv2d (alive across the GEMMs that may regrow `workspace`)
    size_t patches_bytes = 0;
};

namespace dfdx_rocm {

#define HIP_TRY(expr)                           \
    do {                                        \
        hipError_t e__ = (expr);                \
        if (e__ != hipSuccess) return (int)e__; \
    } while (0)

typedef std::lock_guard<std::recursive_mutex> CtxLock;

// Makes the context's device current for the calling thread.
int bind(dfdx_rocm_ctx *ctx);
// Grows the context's workspace to at least `bytes`; work that may still use the old one is drained first.
int ensure_workspace(dfdx_rocm_ctx *ctx, size_t bytes);
// Same for the conv2d patch buffer.
int ensure_patches(dfdx_rocm_ctx *ctx, size_t bytes);
// `ptr` is about to be read, or written in part: if it points into a buffer whose zero fill is deferred, the fill runs
// now (on the context's stream, ahead of the caller's launch).
int settle(dfdx_rocm_ctx *ctx, const void *ptr);
// `ptr` is about to be written: `bytes` = the extent the call writes when it writes every byte of [ptr, ptr + bytes),
// 0 when the written bytes have gaps.  If ptr points into a buffer with a deferred fill: a full cover takes the buffer
// out of the pending set without filling it and reports *fresh = accumulates (the caller then stores 0 + value and
// does not read the old contents); anything else runs the fill.  *fresh is false otherwise.
int settle_output(dfdx_rocm_ctx *ctx, void *ptr, size_t bytes, bool accumulates, bool *fresh);
// Runs every deferred fill of the context.
int settle_all(dfdx_rocm_ctx *ctx);
// Bytes a dense view covers: extents/strides (elements) of up to `rank` axes; 0 if the view has gaps, overlaps or does
// not start at its lowest address.  Any permutation of a contiguous layout is dense.
size_t dense_bytes(int rank, const int64_t *extents, const int64_t *strides, size_t elem_bytes);
// dfdx_rocm_gemm(ctx, desc) which, where the kernel it picks can, also adds the sums of B over the contraction (and over
// the batches of a reduced product) to colsum_b[0 .. n) in the element type: colsum_b[j] += sum_k B[k][j].  *fused tells
// whether it did; when not, colsum_b has not been touched and the caller runs that reduction itself.
int gemm_with_colsum(dfdx_rocm_ctx *ctx, const dfdx_rocm_gemm_desc *desc, void *colsum_b, bool *fused);
// Clears `bytes` bytes at `ptr` (any alignment) with a fill kernel on `stream`.
hipError_t launch_zero_fill(void *ptr, size_t bytes, int compute_units, hipStream_t stream);

}  // namespace dfdx_rocm
