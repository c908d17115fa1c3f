// Host side of the `Rocm` device for the matmul path: the four kernel traits'
// forward / backward, expressed as calls of the strided batched GEMM entry.
// Mirrors the structure of the reference's Cpu impls
// (dfdx-core/src/tensor_ops/matmul/cpu_kernel.rs:231-486): same operands, same
// stride swaps, gradients always accumulated -- but every per-batch loop of the
// reference becomes ONE launch (batch in the grid, or folded into the k loop when
// all batches share one gradient accumulator).
#include "../../include/dfdx_rocm.h"
#include "ctx_internal.h"

#include <cstring>

namespace {

dfdx_rocm_gemm_desc blank(int dtype, int64_t m, int64_t k, int64_t n) {
    dfdx_rocm_gemm_desc d;
    std::memset(&d, 0, sizeof(d));
    d.dtype = dtype;
    d.m = m; d.k = k; d.n = n;
    d.batch1 = 1; d.batch2 = 1;
    return d;
}

bool bad(const void *a, const void *b, const void *c) { return !a || !b || !c; }

// Can `batch` matrices of `rows` rows, batch stride bs and row stride rs, be seen as one matrix of batch*rows rows?
bool rows_fold(int64_t batch, int64_t rows, int64_t bs, int64_t rs) { return batch == 1 || bs == rows * rs; }

}  // namespace

extern "C" {

// MatMatKernel::forward (cpu_kernel.rs:235-254): out = lhs . rhs, out fresh and contiguous.
int dfdx_rocm_matmat_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t m, int64_t k, int64_t n, const void *lhs,
                             const int64_t ls[2], const void *rhs, const int64_t rs[2], void *out) {
    if (!ls || !rs || (m > 0 && n > 0 && bad(lhs, rhs, out))) return DFDX_ROCM_ERR_INVALID_ARG;
    dfdx_rocm_gemm_desc d = blank(dtype, m, k, n);
    d.a = lhs; d.a_rs = ls[0]; d.a_cs = ls[1];
    d.b = rhs; d.b_rs = rs[0]; d.b_cs = rs[1];
    d.c = out; d.c_rs = n; d.c_cs = 1;
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatKernel::backward (cpu_kernel.rs:255-287).
int dfdx_rocm_matmat_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t m, int64_t k, int64_t n, const void *lhs,
                              const int64_t ls[2], void *grad_lhs, const void *rhs, const int64_t rs[2],
                              void *grad_rhs, const void *grad_out) {
    if (!ls || !rs) return DFDX_ROCM_ERR_INVALID_ARG;
    if (m > 0 && k > 0 && n > 0 && (bad(lhs, rhs, grad_out) || !grad_lhs || !grad_rhs)) return DFDX_ROCM_ERR_INVALID_ARG;
    // grad_lhs (m,k) += grad_out (m,n) . rhs^T (n,k)
    dfdx_rocm_gemm_desc d = blank(dtype, m, n, k);
    d.accumulate = 1;
    d.a = grad_out; d.a_rs = n; d.a_cs = 1;
    d.b = rhs; d.b_rs = rs[1]; d.b_cs = rs[0];
    d.c = grad_lhs; d.c_rs = ls[0]; d.c_cs = ls[1];
    if (int e = dfdx_rocm_gemm(ctx, &d)) return e;
    // grad_rhs (k,n) += lhs^T (k,m) . grad_out (m,n)
    d = blank(dtype, k, m, n);
    d.accumulate = 1;
    d.a = lhs; d.a_rs = ls[1]; d.a_cs = ls[0];
    d.b = grad_out; d.b_rs = n; d.b_cs = 1;
    d.c = grad_rhs; d.c_rs = rs[0]; d.c_cs = rs[1];
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBrKernel::forward (cpu_kernel.rs:294-316): (B,M,K) x (K,N).
int dfdx_rocm_matmat_br_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                const void *lhs, const int64_t ls[3], const void *rhs, const int64_t rs[2],
                                void *out) {
    if (!ls || !rs || batch < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0) return DFDX_ROCM_OK;
    dfdx_rocm_gemm_desc d;
    if (rows_fold(batch, m, ls[0], ls[1])) {  // a Linear over (batch*m) rows: one plain GEMM
        d = blank(dtype, batch * m, k, n);
        d.a = lhs; d.a_rs = ls[1]; d.a_cs = ls[2];
    } else {
        d = blank(dtype, m, k, n);
        d.batch1 = batch;
        d.a = lhs; d.a_rs = ls[1]; d.a_cs = ls[2]; d.a_b1 = ls[0];
        d.c_b1 = m * n;
    }
    d.b = rhs; d.b_rs = rs[0]; d.b_cs = rs[1];  // batch stride 0: shared by every batch
    d.c = out; d.c_rs = n; d.c_cs = 1;
    d.flags = DFDX_ROCM_GEMM_NO_SPLIT_K;  // same k order as the batched kernels: Br == Batch3 bit for bit (mod.rs:467-472)
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBrKernel::backward (cpu_kernel.rs:317-351).
int dfdx_rocm_matmat_br_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                 const void *lhs, const int64_t ls[3], void *grad_lhs, const void *rhs,
                                 const int64_t rs[2], void *grad_rhs, const void *grad_out) {
    if (!ls || !rs || batch < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0) return DFDX_ROCM_OK;
    const bool fold = rows_fold(batch, m, ls[0], ls[1]);
    // grad_lhs[i] (m,k) += grad_out[i] (m,n) . rhs^T (n,k)
    dfdx_rocm_gemm_desc d = blank(dtype, fold ? batch * m : m, n, k);
    d.accumulate = 1;
    d.flags = DFDX_ROCM_GEMM_NO_SPLIT_K;  // grad_lhs must equal the Batch3 result bit for bit (mod.rs:471)
    d.a = grad_out; d.a_rs = n; d.a_cs = 1;
    d.b = rhs; d.b_rs = rs[1]; d.b_cs = rs[0];
    d.c = grad_lhs; d.c_rs = ls[1]; d.c_cs = ls[2];
    if (!fold) {
        d.batch1 = batch;
        d.a_b1 = m * n;
        d.c_b1 = ls[0];
    }
    if (int e = dfdx_rocm_gemm(ctx, &d)) return e;
    // grad_rhs (k,n) += sum_i lhs[i]^T (k,m) . grad_out[i] (m,n): the batch extends the contraction
    if (fold) {
        d = blank(dtype, k, batch * m, n);
    } else {
        d = blank(dtype, k, m, n);
        d.batch1 = batch;
        d.reduce_batch = 1;
        d.a_b1 = ls[0];
        d.b_b1 = m * n;
    }
    d.accumulate = 1;
    d.a = lhs; d.a_rs = ls[2]; d.a_cs = ls[1];
    d.b = grad_out; d.b_rs = n; d.b_cs = 1;
    d.c = grad_rhs; d.c_rs = rs[0]; d.c_cs = rs[1];
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBatch3Kernel::forward (cpu_kernel.rs:358-382): (B,M,K) x (B,K,N).
int dfdx_rocm_matmat_batch3_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                    const void *lhs, const int64_t ls[3], const void *rhs, const int64_t rs[3],
                                    void *out) {
    if (!ls || !rs || batch < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0) return DFDX_ROCM_OK;
    dfdx_rocm_gemm_desc d = blank(dtype, m, k, n);
    d.batch1 = batch;
    d.a = lhs; d.a_b1 = ls[0]; d.a_rs = ls[1]; d.a_cs = ls[2];
    d.b = rhs; d.b_b1 = rs[0]; d.b_rs = rs[1]; d.b_cs = rs[2];
    d.c = out; d.c_b1 = m * n; d.c_rs = n; d.c_cs = 1;
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBatch3Kernel::backward (cpu_kernel.rs:383-417).
int dfdx_rocm_matmat_batch3_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t m, int64_t k, int64_t n,
                                     const void *lhs, const int64_t ls[3], void *grad_lhs, const void *rhs,
                                     const int64_t rs[3], void *grad_rhs, const void *grad_out) {
    if (!ls || !rs || batch < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0) return DFDX_ROCM_OK;
    dfdx_rocm_gemm_desc d = blank(dtype, m, n, k);
    d.accumulate = 1;
    d.batch1 = batch;
    d.a = grad_out; d.a_b1 = m * n; d.a_rs = n; d.a_cs = 1;
    d.b = rhs; d.b_b1 = rs[0]; d.b_rs = rs[2]; d.b_cs = rs[1];
    d.c = grad_lhs; d.c_b1 = ls[0]; d.c_rs = ls[1]; d.c_cs = ls[2];
    if (int e = dfdx_rocm_gemm(ctx, &d)) return e;
    d = blank(dtype, k, m, n);
    d.accumulate = 1;
    d.batch1 = batch;
    d.a = lhs; d.a_b1 = ls[0]; d.a_rs = ls[2]; d.a_cs = ls[1];
    d.b = grad_out; d.b_b1 = m * n; d.b_rs = n; d.b_cs = 1;
    d.c = grad_rhs; d.c_b1 = rs[0]; d.c_rs = rs[1]; d.c_cs = rs[2];
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBatch4Kernel::forward (cpu_kernel.rs:424-448): (B,S,M,K) x (B,S,K,N).
int dfdx_rocm_matmat_batch4_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t seq, int64_t m, int64_t k,
                                    int64_t n, const void *lhs, const int64_t ls[4], const void *rhs,
                                    const int64_t rs[4], void *out) {
    if (!ls || !rs || batch < 0 || seq < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0 || seq == 0) return DFDX_ROCM_OK;
    dfdx_rocm_gemm_desc d = blank(dtype, m, k, n);
    d.batch1 = batch; d.batch2 = seq;
    d.a = lhs; d.a_b1 = ls[0]; d.a_b2 = ls[1]; d.a_rs = ls[2]; d.a_cs = ls[3];
    d.b = rhs; d.b_b1 = rs[0]; d.b_b2 = rs[1]; d.b_rs = rs[2]; d.b_cs = rs[3];
    d.c = out; d.c_b1 = seq * m * n; d.c_b2 = m * n; d.c_rs = n; d.c_cs = 1;
    return dfdx_rocm_gemm(ctx, &d);
}

// MatMatBatch4Kernel::backward (cpu_kernel.rs:449-485).
int dfdx_rocm_matmat_batch4_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t batch, int64_t seq, int64_t m, int64_t k,
                                     int64_t n, const void *lhs, const int64_t ls[4], void *grad_lhs,
                                     const void *rhs, const int64_t rs[4], void *grad_rhs, const void *grad_out) {
    if (!ls || !rs || batch < 0 || seq < 0) return DFDX_ROCM_ERR_INVALID_ARG;
    if (batch == 0 || seq == 0) return DFDX_ROCM_OK;
    dfdx_rocm_gemm_desc d = blank(dtype, m, n, k);
    d.accumulate = 1;
    d.batch1 = batch; d.batch2 = seq;
    d.a = grad_out; d.a_b1 = seq * m * n; d.a_b2 = m * n; d.a_rs = n; d.a_cs = 1;
    d.b = rhs; d.b_b1 = rs[0]; d.b_b2 = rs[1]; d.b_rs = rs[3]; d.b_cs = rs[2];
    d.c = grad_lhs; d.c_b1 = ls[0]; d.c_b2 = ls[1]; d.c_rs = ls[2]; d.c_cs = ls[3];
    if (int e = dfdx_rocm_gemm(ctx, &d)) return e;
    d = blank(dtype, k, m, n);
    d.accumulate = 1;
    d.batch1 = batch; d.batch2 = seq;
    d.a = lhs; d.a_b1 = ls[0]; d.a_b2 = ls[1]; d.a_rs = ls[3]; d.a_cs = ls[2];
    d.b = grad_out; d.b_b1 = seq * m * n; d.b_b2 = m * n; d.b_rs = n; d.b_cs = 1;
    d.c = grad_rhs; d.c_b1 = rs[0]; d.c_b2 = rs[1]; d.c_rs = rs[2]; d.c_cs = rs[3];
    return dfdx_rocm_gemm(ctx, &d);
}

// Linear::try_forward (dfdx/src/nn/layers/linear.rs:82-89) with Bias1D (bias1d.rs:62-78) fused into the store.
int dfdx_rocm_linear_forward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t in_dim, int64_t out_dim,
                             const void *x, const int64_t xs[2], const void *weight, const void *bias, void *out) {
    if (!xs) return DFDX_ROCM_ERR_INVALID_ARG;
    dfdx_rocm_gemm_desc d = blank(dtype, rows, in_dim, out_dim);
    d.a = x; d.a_rs = xs[0]; d.a_cs = xs[1];
    d.b = weight; d.b_rs = 1; d.b_cs = in_dim;  // the (I,O) view of the (O,I) storage
    d.c = out; d.c_rs = out_dim; d.c_cs = 1;
    d.bias = bias;
    return dfdx_rocm_gemm(ctx, &d);
}

int dfdx_rocm_linear_backward(dfdx_rocm_ctx *ctx, int dtype, int64_t rows, int64_t in_dim, int64_t out_dim,
                              const void *x, const int64_t xs[2], void *grad_x, const void *weight, void *grad_weight,
                              void *grad_bias, const void *grad_out) {
    if (!xs) return DFDX_ROCM_ERR_INVALID_ARG;
    // every step below supports all four element types; an unknown one is refused before any gradient is touched
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_INVALID_ARG;
    const int64_t ws[2] = {1, in_dim};  // the (I,O) view of the (O,I) storage; its gradient lands in (O,I) row-major
    if (!grad_bias || rows == 0 || in_dim == 0 || out_dim == 0) {
        if (int e = dfdx_rocm_matmat_backward(ctx, dtype, rows, in_dim, out_dim, x, xs, grad_x, weight, ws, grad_weight, grad_out))
            return e;
        return grad_bias ? dfdx_rocm_bias_backward(ctx, dtype, rows, out_dim, grad_out, grad_bias) : DFDX_ROCM_OK;
    }
    // The two products of MatMatKernel::backward (cpu_kernel.rs:265-286), the second one asked to produce the bias
    // gradient as well: grad_out is its B operand, and the column sums of B over the contraction (the rows) are
    // exactly what Bias1D's backward adds to grad_bias.  Kernels that cannot do that leave it to the reduction kernel.
    if (bad(x, weight, grad_out) || !grad_x || !grad_weight) return DFDX_ROCM_ERR_INVALID_ARG;
    dfdx_rocm_gemm_desc d = blank(dtype, rows, out_dim, in_dim);
    d.accumulate = 1;
    d.a = grad_out; d.a_rs = out_dim; d.a_cs = 1;
    d.b = weight; d.b_rs = ws[1]; d.b_cs = ws[0];
    d.c = grad_x; d.c_rs = xs[0]; d.c_cs = xs[1];
    if (int e = dfdx_rocm_gemm(ctx, &d)) return e;
    d = blank(dtype, in_dim, rows, out_dim);
    d.accumulate = 1;
    d.a = x; d.a_rs = xs[1]; d.a_cs = xs[0];
    d.b = grad_out; d.b_rs = out_dim; d.b_cs = 1;
    d.c = grad_weight; d.c_rs = ws[0]; d.c_cs = ws[1];
    bool fused = false;
    if (int e = dfdx_rocm::gemm_with_colsum(ctx, &d, grad_bias, &fused)) return e;
    return fused ? DFDX_ROCM_OK : dfdx_rocm_bias_backward(ctx, dtype, rows, out_dim, grad_out, grad_bias);
}

}  // extern "C"
