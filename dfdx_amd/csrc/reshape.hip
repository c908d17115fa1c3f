// Reshape of a non-contiguous view: the copy `ReshapeKernel::forward` makes (out, contiguous, takes the view's
// elements in logical row-major order) and its backward (grad_inp, through the view's strides, += grad_out).
// HBM-bound gather / scatter; the view's innermost run of contiguous elements is moved 16 bytes at a time when it
// allows (a head permute of attention keeps rows of head_dim elements contiguous).
#include "ctx_internal.h"
#include "elem.h"

namespace dfdx_rocm {
namespace {

constexpr int MAX_RANK = 6;

struct ViewDims {
    int rank;
    uint32_t shape[MAX_RANK];   // innermost axis counted in groups of N elements
    int64_t stride[MAX_RANK];   // elements
};

// offset (elements) of the g-th N-element group of the view in logical order
template <typename Index> __device__ __forceinline__ int64_t view_offset(const ViewDims &d, Index g) {
    int64_t off = 0;
#pragma unroll
    for (int a = MAX_RANK - 1; a >= 0; a--) {
        if (a < d.rank) {
            const Index q = g / d.shape[a];
            off += (int64_t)(g - q * d.shape[a]) * d.stride[a];
            g = q;
        }
    }
    return off;
}

template <typename T, int N, typename Index>
__global__ __launch_bounds__(256) void reshape_forward_kernel(const T *inp, T *out, ViewDims d, Index groups) {
    for (Index g = (Index)blockIdx.x * 256 + threadIdx.x; g < groups; g += (Index)gridDim.x * 256) {
        if constexpr (sizeof(T) == 8) {  // f64: one element per thread (N == 1)
            out[(int64_t)g] = inp[view_offset<Index>(d, g)];
        } else {
            float v[N];
            load_elems<T, N>(inp + view_offset<Index>(d, g), v);
            store_elems<T, N>(out + (int64_t)g * N, v);
        }
    }
}

template <typename T, int N, typename Index>
__global__ __launch_bounds__(256) void reshape_backward_kernel(T *grad_inp, const T *grad_out, ViewDims d, Index groups, bool fresh) {
    for (Index g = (Index)blockIdx.x * 256 + threadIdx.x; g < groups; g += (Index)gridDim.x * 256) {
        if constexpr (sizeof(T) == 8) {  // f64: one element per thread (N == 1)
            T *dst64 = grad_inp + view_offset<Index>(d, g);
            *dst64 = (fresh ? T(0) : *dst64) + grad_out[(int64_t)g];
            continue;
        }
        float v[N], old[N];
        load_elems<T, N>(grad_out + (int64_t)g * N, v);
        T *dst = grad_inp + view_offset<Index>(d, g);
        if (fresh) {  // grad_inp counts as zero and is not read
#pragma unroll
            for (int i = 0; i < N; i++) old[i] = 0.0f;
        } else {
            load_elems<T, N>(dst, old);
        }
#pragma unroll
        for (int i = 0; i < N; i++) old[i] += v[i];
        store_elems<T, N>(dst, old);
    }
}

// Backward through a view with broadcast axes (stride 0, extent > 1): every grad_inp element receives the SUM of the
// grad_out elements that the view maps onto it (reshape_to/cpu_kernel.rs:28-32 adds them one after the other).  A thread
// owns one grad_inp element -- an index over the kept axes -- and walks the broadcast axes itself: no atomics, a fixed
// order, f32 accumulation with one rounding.
struct ReduceDims {
    int nkeep, nbro;
    uint32_t keep_shape[MAX_RANK], bro_shape[MAX_RANK];
    int64_t keep_dst[MAX_RANK];                       // stride in grad_inp (elements)
    int64_t keep_src[MAX_RANK], bro_src[MAX_RANK];    // stride in the contiguous grad_out (elements)
};

template <typename T>
__global__ __launch_bounds__(256) void reshape_backward_reduce_kernel(T *grad_inp, const T *grad_out, ReduceDims d, int64_t kept,
                                                                      int64_t folded) {
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < kept; e += (int64_t)gridDim.x * 256) {
        int64_t dst = 0, src0 = 0, q = e;
        for (int a = d.nkeep - 1; a >= 0; a--) {
            const int64_t i = q % d.keep_shape[a];
            q /= d.keep_shape[a];
            dst += i * d.keep_dst[a];
            src0 += i * d.keep_src[a];
        }
        typename Acc<T>::type sum = 0;
        for (int64_t r = 0; r < folded; r++) {
            int64_t src = src0, t = r;
            for (int a = d.nbro - 1; a >= 0; a--) {
                src += (t % d.bro_shape[a]) * d.bro_src[a];
                t /= d.bro_shape[a];
            }
            sum += Elem<T>::load(grad_out + src);
        }
        Elem<T>::store(grad_inp + dst, Elem<T>::load(grad_inp + dst) + sum);
    }
}

template <typename T>
int launch_reduce(dfdx_rocm_ctx *ctx, int rank, const int64_t *shape, const int64_t *strides, const void *grad_out, void *grad_inp) {
    ReduceDims d = {};
    int64_t kept = 1, folded = 1, logical = 1;
    int64_t ls[MAX_RANK];  // row-major stride of each axis in grad_out
    for (int a = rank - 1; a >= 0; a--) {
        ls[a] = logical;
        logical *= shape[a];
        if (shape[a] > 1 && strides[a] == 0) folded *= shape[a];
        else if (shape[a] > 1) kept *= shape[a];
    }
    for (int a = 0; a < rank; a++) {
        if (shape[a] <= 1) continue;
        if (strides[a] == 0) {
            d.bro_shape[d.nbro] = (uint32_t)shape[a];
            d.bro_src[d.nbro++] = ls[a];
        } else {
            d.keep_shape[d.nkeep] = (uint32_t)shape[a];
            d.keep_dst[d.nkeep] = strides[a];
            d.keep_src[d.nkeep++] = ls[a];
        }
    }
    const unsigned grid = (unsigned)std::min<int64_t>((kept + 255) / 256, (int64_t)ctx->compute_units * 16);
    reshape_backward_reduce_kernel<T><<<grid, 256, 0, ctx->stream>>>((T *)grad_inp, (const T *)grad_out, d, kept, folded);
    return (int)hipGetLastError();
}

// ---- a permutation that moves the innermost axis: tiled transpose through LDS ---------------------------------------------
// When the view's innermost logical axis is not the one that is contiguous in its storage (a transposed matrix, heads x
// (dim, seq)), the kernels above read or write single elements a whole row apart: 0.5 - 1.8 TB/s.  Here a workgroup moves a
// 64 x 64 tile over (the storage-contiguous axis J, the innermost logical axis L): both sides are touched in runs of 64
// contiguous elements, the tile turns in LDS.  The other axes are a batch (blockIdx.z).  `strided` is the view's storage,
// `dense` the contiguous tensor; forward copies strided -> dense, backward adds dense into strided.
struct TransposeDims {
    int rank;                      // batch axes (canonical axes other than J and L)
    uint32_t shape[MAX_RANK];      // their extents
    int64_t sstride[MAX_RANK];     // their strides in the view's storage
    int64_t dstride[MAX_RANK];     // ... in the dense tensor
    uint32_t nj, nl;               // extents of J and L
    int64_t l_sstride, j_dstride;  // stride of L in the storage (J's is 1), of J in the dense tensor (L's is 1)
};
template <typename T, bool FWD>
__global__ __launch_bounds__(256) void reshape_transpose_kernel(const T *src, T *dst, TransposeDims d, bool fresh) {
    __shared__ T tile[64][65];
    int64_t soff = 0, doff = 0;
    uint32_t b = blockIdx.z;
#pragma unroll
    for (int a = MAX_RANK - 1; a >= 0; a--) {
        if (a < d.rank) {
            const uint32_t q = b / d.shape[a], r = b - q * d.shape[a];
            soff += (int64_t)r * d.sstride[a];
            doff += (int64_t)r * d.dstride[a];
            b = q;
        }
    }
    const uint32_t j0 = blockIdx.x * 64, l0 = blockIdx.y * 64, tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    // `strided` side: element (j, l) at soff + j + l * l_sstride; `dense` side: at doff + j * j_dstride + l
    const T *strided_in = FWD ? src : nullptr;
    T *strided_out = FWD ? nullptr : dst;
    const T *dense_in = FWD ? nullptr : src;
    T *dense_out = FWD ? dst : nullptr;
    if constexpr (FWD) {
        for (uint32_t l = ty; l < 64; l += 4)
            if (j0 + tx < d.nj && l0 + l < d.nl) tile[l][tx] = strided_in[soff + (int64_t)(j0 + tx) + (int64_t)(l0 + l) * d.l_sstride];
        __syncthreads();
        for (uint32_t j = ty; j < 64; j += 4)
            if (j0 + j < d.nj && l0 + tx < d.nl) dense_out[doff + (int64_t)(j0 + j) * d.j_dstride + (int64_t)(l0 + tx)] = tile[tx][j];
    } else {
        for (uint32_t j = ty; j < 64; j += 4)
            if (j0 + j < d.nj && l0 + tx < d.nl) tile[tx][j] = dense_in[doff + (int64_t)(j0 + j) * d.j_dstride + (int64_t)(l0 + tx)];
        __syncthreads();
        for (uint32_t l = ty; l < 64; l += 4)
            if (j0 + tx < d.nj && l0 + l < d.nl) {
                T *p = strided_out + soff + (int64_t)(j0 + tx) + (int64_t)(l0 + l) * d.l_sstride;
                if (fresh) *p = tile[l][tx];
                else Elem<T>::store(p, Elem<T>::load(p) + Elem<T>::load(&tile[l][tx]));
            }
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// Drops size-1 axes and merges neighbours that are contiguous with respect to each other.
int canonical(int rank, const int64_t *shape, const int64_t *strides, int64_t *cs, int64_t *cst) {
    int n = 0;
    for (int a = 0; a < rank; a++) {
        if (shape[a] == 1) continue;
        if (n > 0 && cst[n - 1] == strides[a] * shape[a]) {
            cs[n - 1] *= shape[a];
            cst[n - 1] = strides[a];
        } else {
            cs[n] = shape[a];
            cst[n] = strides[a];
            n++;
        }
    }
    if (n == 0) {
        cs[0] = 1;
        cst[0] = 1;
        n = 1;
    }
    return n;
}

template <typename T, bool FWD>
int launch_t(dfdx_rocm_ctx *ctx, int rank, const int64_t *shape, const int64_t *strides, const void *src, void *dst, bool fresh) {
    // forward: src = inp (strided), dst = out (contiguous);  backward: src = grad_out (contiguous), dst = grad_inp (strided)
    int64_t cs[MAX_RANK], cst[MAX_RANK];
    const int n = canonical(rank, shape, strides, cs, cst);
    int64_t total = 1;
    for (int a = 0; a < n; a++) total *= cs[a];
    constexpr int V = Elem<T>::VEC;
    const void *strided = FWD ? src : dst;
    if constexpr (sizeof(T) != 8) {
        // the innermost logical axis is strided and exactly one other axis is contiguous in the storage: a (batched) transpose
        int jax = -1, ones = 0;
        for (int a = 0; a + 1 < n; a++)
            if (cst[a] == 1) { jax = a; ones++; }
        bool distinct = true;  // (a permutation: no broadcast axis)
        for (int a = 0; a < n; a++) distinct = distinct && cst[a] > 0;
        if (n >= 2 && cst[n - 1] != 1 && ones == 1 && distinct && cs[jax] >= 16 && cs[n - 1] >= 16) {
            TransposeDims t{};
            int64_t dense_stride[MAX_RANK];
            int64_t run = 1, batch = 1;
            for (int a = n - 1; a >= 0; a--) { dense_stride[a] = run; run *= cs[a]; }
            for (int a = 0; a < n; a++) {
                if (a == jax || a == n - 1) continue;
                t.shape[t.rank] = (uint32_t)cs[a]; t.sstride[t.rank] = cst[a]; t.dstride[t.rank] = dense_stride[a];
                t.rank++;
                batch *= cs[a];
            }
            t.nj = (uint32_t)cs[jax]; t.nl = (uint32_t)cs[n - 1];
            t.l_sstride = cst[n - 1]; t.j_dstride = dense_stride[jax];
            const int64_t gx = (cs[jax] + 63) / 64, gy = (cs[n - 1] + 63) / 64;
            if (batch <= 65535 && gy <= 65535 && gx < (1ll << 31)) {
                reshape_transpose_kernel<T, FWD><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)batch), 256, 0, ctx->stream>>>((const T *)src, (T *)dst, t, fresh);
                return (int)hipGetLastError();
            }
        }
    }
    bool vec = sizeof(T) != 8 && cst[n - 1] == 1 && cs[n - 1] % V == 0 && aligned16(src) && aligned16(dst);
    for (int a = 0; a + 1 < n && vec; a++) vec = cst[a] % V == 0;
    (void)strided;
    const int g = vec ? V : 1;
    ViewDims d;
    d.rank = n;
    for (int a = 0; a < MAX_RANK; a++) {
        d.shape[a] = a < n ? (uint32_t)(a == n - 1 ? cs[a] / g : cs[a]) : 1u;
        d.stride[a] = a < n ? (a == n - 1 ? cst[a] * g : cst[a]) : 0;
    }
    const int64_t groups = total / g;
    const unsigned grid = (unsigned)std::min<int64_t>((groups + 255) / 256, (int64_t)ctx->compute_units * 16);
    const bool small = groups < (1ll << 31);
    hipStream_t s = ctx->stream;
#define DFDX_RESHAPE(N, IDX)                                                                                       \
    do {                                                                                                           \
        if constexpr (FWD) reshape_forward_kernel<T, N, IDX><<<grid, 256, 0, s>>>((const T *)src, (T *)dst, d, (IDX)groups); \
        else reshape_backward_kernel<T, N, IDX><<<grid, 256, 0, s>>>((T *)dst, (const T *)src, d, (IDX)groups, fresh); \
    } while (0)
    if constexpr (sizeof(T) != 8) {
        if (vec && small) {
            DFDX_RESHAPE(V, uint32_t);
            return (int)hipGetLastError();
        }
        if (vec) {
            DFDX_RESHAPE(V, uint64_t);
            return (int)hipGetLastError();
        }
    }
    if (small) DFDX_RESHAPE(1, uint32_t);
    else DFDX_RESHAPE(1, uint64_t);
#undef DFDX_RESHAPE
    return (int)hipGetLastError();
}

template <bool FWD>
int dispatch(dfdx_rocm_ctx *ctx, int dtype, int rank, const int64_t *shape, const int64_t *strides, const void *src, void *dst) {
    if (int e = bind(ctx)) return e;
    if (rank < 0 || rank > MAX_RANK || (rank > 0 && (!shape || !strides))) return DFDX_ROCM_ERR_INVALID_ARG;
    int64_t total = 1;
    bool broadcast = false;
    for (int a = 0; a < rank; a++) {
        if (shape[a] < 0 || strides[a] < 0 || shape[a] >= (1ll << 32)) return DFDX_ROCM_ERR_INVALID_ARG;
        // a broadcast axis maps several grad_out elements to one grad_inp element: a reduction, not a scatter
        if (!FWD && shape[a] > 1 && strides[a] == 0) broadcast = true;
        total *= shape[a];
    }
    if (total == 0) return DFDX_ROCM_OK;
    if (!src || !dst) return DFDX_ROCM_ERR_INVALID_ARG;
    if (dtype < DFDX_ROCM_F32 || dtype > DFDX_ROCM_F64) return DFDX_ROCM_ERR_UNSUPPORTED;
    // Deferred zero fills: the contiguous side covers total elements; the strided side covers its buffer when the view
    // is a permutation of a contiguous layout (a backward through such a view then stores 0 + value).
    const size_t es = dtype == DFDX_ROCM_F64 ? 8 : dtype == DFDX_ROCM_F32 ? 4 : 2;
    bool fresh = false;
    if (int e = settle(ctx, src)) return e;
    if (int e = settle_output(ctx, dst, FWD ? (size_t)total * es : dense_bytes(rank, shape, strides, es), !FWD, broadcast ? nullptr : &fresh))
        return e;
    if (broadcast) {
        switch (dtype) {
        case DFDX_ROCM_F64: return launch_reduce<double>(ctx, rank, shape, strides, src, dst);
        case DFDX_ROCM_F32: return launch_reduce<float>(ctx, rank, shape, strides, src, dst);
        case DFDX_ROCM_F16: return launch_reduce<_Float16>(ctx, rank, shape, strides, src, dst);
        case DFDX_ROCM_BF16: return launch_reduce<__bf16>(ctx, rank, shape, strides, src, dst);
        default: return DFDX_ROCM_ERR_UNSUPPORTED;
        }
    }
    switch (dtype) {
    case DFDX_ROCM_F64: return launch_t<double, FWD>(ctx, rank, shape, strides, src, dst, fresh);
    case DFDX_ROCM_F32: return launch_t<float, FWD>(ctx, rank, shape, strides, src, dst, fresh);
    case DFDX_ROCM_F16: return launch_t<_Float16, FWD>(ctx, rank, shape, strides, src, dst, fresh);
    case DFDX_ROCM_BF16: return launch_t<__bf16, FWD>(ctx, rank, shape, strides, src, dst, fresh);
    default: return DFDX_ROCM_ERR_UNSUPPORTED;
    }
}

}  // namespace
}  // namespace dfdx_rocm

extern "C" {

int dfdx_rocm_reshape_forward(dfdx_rocm_ctx *ctx, int dtype, int rank, const int64_t *shape, const int64_t *inp_strides,
                              const void *inp, void *out) {
    return dfdx_rocm::dispatch<true>(ctx, dtype, rank, shape, inp_strides, inp, out);
}

int dfdx_rocm_reshape_backward(dfdx_rocm_ctx *ctx, int dtype, int rank, const int64_t *shape, const int64_t *inp_strides,
                               void *grad_inp, const void *grad_out) {
    return dfdx_rocm::dispatch<false>(ctx, dtype, rank, shape, inp_strides, grad_out, grad_inp);
}

}  // extern "C"
