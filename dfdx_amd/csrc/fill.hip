// Zero fill of device storage (`Storage::try_alloc_len` must return zeros, tensor/cuda/device.rs:259-266; every
// gradient buffer starts as one, tensor/gradients.rs:53-58).  A kernel rather than hipMemsetAsync: it is an ordinary
// launch on the context's stream (safe to record into a HIP graph) and it writes whole 128 B lines, 1 KB per wave
// instruction, which is the pattern the memory system of this chip accepts at its full write rate.
#include "ctx_internal.h"

namespace dfdx_rocm {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int FILL_THREADS = 256;
constexpr int FILL_UNROLL = 4;
constexpr int64_t FILL_CHUNK = (int64_t)FILL_THREADS * 16 * FILL_UNROLL;   // bytes one workgroup clears per step

// `body` = 16 B pieces from the first 16 B-aligned address; the bytes in front of it (`head` < 16) and behind it
// (`tail` < 16) are cleared bytewise by the first workgroup.
__global__ __launch_bounds__(FILL_THREADS) void zero_fill_kernel(uint8_t *ptr, int head, int64_t body, int tail) {
    u32x4 *dst = (u32x4 *)(ptr + head);
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int64_t pieces_per_chunk = FILL_CHUNK / 16;
    const int64_t chunks = (body + pieces_per_chunk - 1) / pieces_per_chunk;
    for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
        const int64_t first = c * pieces_per_chunk + threadIdx.x;
        if (first + (FILL_UNROLL - 1) * FILL_THREADS < body) {   // a whole chunk: no checks
#pragma unroll
            for (int u = 0; u < FILL_UNROLL; u++) dst[first + u * FILL_THREADS] = zero;
        } else {
#pragma unroll
            for (int u = 0; u < FILL_UNROLL; u++)
                if (first + u * FILL_THREADS < body) dst[first + u * FILL_THREADS] = zero;
        }
    }
    if (blockIdx.x == 0) {
        if ((int)threadIdx.x < head) ptr[threadIdx.x] = 0;
        if ((int)threadIdx.x >= 64 && (int)threadIdx.x - 64 < tail) ptr[head + body * 16 + (threadIdx.x - 64)] = 0;
    }
}

}  // namespace

hipError_t launch_zero_fill(void *ptr, size_t bytes, int compute_units, hipStream_t stream) {
    if (bytes == 0) return hipSuccess;
    const uintptr_t addr = (uintptr_t)ptr;
    size_t head = (16 - addr % 16) % 16;
    if (head > bytes) head = bytes;
    const int64_t body = (int64_t)((bytes - head) / 16);
    const int tail = (int)((bytes - head) % 16);
    const int64_t chunks = (body * 16 + FILL_CHUNK - 1) / FILL_CHUNK;
    const int64_t cap = (int64_t)(compute_units > 0 ? compute_units : 256) * 16;   // 8 waves x 8 workgroups per CU at most
    const int grid = (int)(chunks < 1 ? 1 : (chunks < cap ? chunks : cap));
    hipLaunchKernelGGL(zero_fill_kernel, dim3(grid), dim3(FILL_THREADS), 0, stream, (uint8_t *)ptr, (int)head, body, tail);
    return hipGetLastError();
}

}  // namespace dfdx_rocm
