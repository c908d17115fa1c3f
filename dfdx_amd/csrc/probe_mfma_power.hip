// Stand-alone measurement aid, not part of libdfdx_rocm.so: what the matrix cores alone sustain on this chip.
//
// Each launch issues exactly the MFMA instructions of a 4096^3 f16 GEMM tiled like gemm_mfma16_dma_kernel (256
// workgroups of 8 waves, wave tile 128 x 64, 128 k steps of 32), but on operands that stay in registers: no global
// loads, no LDS, no barrier, no stores.  It is run on all-zero operands and on U(-1,1) operands, with the
// 16x16x32 and the 32x32x16 instruction.  The difference between the two operand sets is what the chip's power
// limit costs the matrix cores on real data, and the U(-1,1) figure is the ceiling any f16 GEMM kernel on
// such data can approach.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
    fprintf(stderr, "probe_mfma_power: %s (line %d)\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

static constexpr int SRC_VECS = 1 << 20;   // 16 B vectors in the operand pool

// 16x16x32: per k step of 32, 8 A fragments x 4 B fragments; consecutive MFMAs share the first operand.
__global__ __launch_bounds__(512, 2) void mfma_only_16x16x32(const h8 *src, float *out, int steps) {
    const int t = threadIdx.x + blockIdx.x * 512;
    h8 a[2][8], b[2][4];
    for (int s = 0; s < 2; s++) {
        for (int i = 0; i < 8; i++) a[s][i] = src[(t * 24 + s * 12 + i) % SRC_VECS];
        for (int j = 0; j < 4; j++) b[s][j] = src[(t * 24 + s * 12 + 8 + j) % SRC_VECS];
    }
    f4 acc[8][4];
    for (int i = 0; i < 8; i++) for (int j = 0; j < 4; j++) acc[i][j] = f4{0, 0, 0, 0};
    for (int it = 0; it < steps; it += 2) {
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 8; i++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[s][j], a[s][i], acc[i][j], 0, 0, 0);
    }
    f4 r = f4{0, 0, 0, 0};
    for (int i = 0; i < 8; i++) for (int j = 0; j < 4; j++) r += acc[i][j];
    if (r[0] + r[1] + r[2] + r[3] == 12345.678f) out[t] = r[0];   // keeps the loop alive; never true in practice
}

// 32x32x16: per k step of 32, two halves of 16, each 4 A fragments x 2 B fragments.
__global__ __launch_bounds__(512, 2) void mfma_only_32x32x16(const h8 *src, float *out, int steps) {
    const int t = threadIdx.x + blockIdx.x * 512;
    h8 a[2][2][4], b[2][2][2];
    for (int s = 0; s < 2; s++)
        for (int h = 0; h < 2; h++) {
            for (int i = 0; i < 4; i++) a[s][h][i] = src[(t * 24 + s * 12 + h * 6 + i) % SRC_VECS];
            for (int j = 0; j < 2; j++) b[s][h][j] = src[(t * 24 + s * 12 + h * 6 + 4 + j) % SRC_VECS];
        }
    f16v acc[4][2];
    for (int i = 0; i < 4; i++) for (int j = 0; j < 2; j++) for (int e = 0; e < 16; e++) acc[i][j][e] = 0;
    for (int it = 0; it < steps; it += 2) {
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[s][h][j], a[s][h][i], acc[i][j], 0, 0, 0);
    }
    float r = 0;
    for (int i = 0; i < 4; i++) for (int j = 0; j < 2; j++) for (int e = 0; e < 16; e++) r += acc[i][j][e];
    if (r == 12345.678f) out[t] = r;
}

int main() {
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) { fprintf(stderr, "probe_mfma_power: no HIP device\n"); return 2; }
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int steps = 4096 / 32;
    std::vector<_Float16> host((size_t)SRC_VECS * 8);
    uint64_t s = 88172645463325252ull;   // xorshift64
    for (auto &v : host) {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        v = (_Float16)(((double)(s >> 11) / (double)(1ull << 53)) * 2.0 - 1.0);
    }
    h8 *d_rand, *d_zero;
    float *out;
    CK(hipMalloc(&d_rand, host.size() * 2));
    CK(hipMalloc(&d_zero, host.size() * 2));
    CK(hipMalloc(&out, (size_t)256 * 512 * sizeof(float)));
    CK(hipMemcpy(d_rand, host.data(), host.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemset(d_zero, 0, host.size() * 2));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    printf("device: %s, %d CUs\n", prop.gcnArchName, prop.multiProcessorCount);
    auto run = [&](const char *name, bool wide, const h8 *src) {
        const int warm = 3000, timed = 1000;   // ~0.25 s of load before the timed launches: sustained clock
        for (int r = 0; r < warm + timed; r++) {
            if (r == warm) CK(hipEventRecord(e0));
            if (wide) hipLaunchKernelGGL(mfma_only_32x32x16, dim3(256), dim3(512), 0, 0, src, out, steps);
            else hipLaunchKernelGGL(mfma_only_16x16x32, dim3(256), dim3(512), 0, 0, src, out, steps);
        }
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        CK(hipGetLastError());
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        const double flop = 2.0 * 4096 * 4096 * 4096;
        printf("%-28s %8.2f us/launch  %8.1f TFLOP/s  %5.1f %% of 2500\n", name, ms * 1e3 / timed,
               flop * timed / (ms * 1e-3) / 1e12, flop * timed / (ms * 1e-3) / 1e12 / 25.0);
        fflush(stdout);
    };
    for (int pass = 0; pass < 2; pass++) {
        run("16x16x32 zero operands", false, d_zero);
        run("32x32x16 zero operands", true, d_zero);
        run("16x16x32 U(-1,1) operands", false, d_rand);
        run("32x32x16 U(-1,1) operands", true, d_rand);
    }
    return 0;
}
