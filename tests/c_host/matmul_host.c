/* A plain-C host of libdfdx_rocm.so: what the Rust `Rocm` device's `Storage` and `MatMatKernel` impls would do,
 * call for call, without Python or torch in the process.
 *
 *   create -> alloc (zeroed) -> h2d -> matmat_forward -> d2h -> compare
 *          -> alloc gradients (zeroed / zero-deferred) -> matmat_backward -> d2h -> compare
 *          -> cache: enable, free, allocate again (the same buffer comes back, zero-filled again), empty, disable
 *          -> error paths: strerror of every code, a null descriptor, an unknown dtype
 *          -> destroy
 *
 * Values: the literals of the reference's `test_matmul_normal` (dfdx-core/src/tensor_ops/matmul/mod.rs:368-410): a
 * 4x3 by 3x2 product, loss = mean(exp(r)), so grad_out = exp(r) / 8; tolerance 1e-6 as `assert_close_to_literal!`
 * uses (f32), every return code checked.  Exit status 0 = all checks passed; the failing check is named on stderr.
 * Built by tests/c_host/Makefile with gcc against include/dfdx_rocm.h. */
#include "dfdx_rocm.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int failures = 0;

#define CHECK(cond, ...)                                      \
    do {                                                      \
        if (!(cond)) {                                        \
            fprintf(stderr, "FAILED %s:%d: ", __FILE__, __LINE__); \
            fprintf(stderr, __VA_ARGS__);                     \
            fprintf(stderr, "\n");                            \
            failures++;                                       \
        }                                                     \
    } while (0)

#define OK(call)                                                                          \
    do {                                                                                  \
        int rc_ = (call);                                                                 \
        if (rc_ != DFDX_ROCM_OK) {                                                        \
            fprintf(stderr, "FAILED %s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, dfdx_rocm_strerror(rc_)); \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)

static const float A[4 * 3] = {0.5086f, 0.5234f, 0.2684f, 0.8075f, 0.8437f, 0.9951f,
                               0.0774f, 0.7539f, 0.8894f, 0.8119f, 0.2693f, 0.7249f};
static const float B[3 * 2] = {0.4651f, 0.9106f, 0.3360f, 0.5534f, 0.8092f, 0.3827f};
static const float R[4 * 2] = {0.62960154f, 0.8554974f, 1.4642863f, 1.5830379f, 1.0090116f, 0.82806206f, 1.0546886f, 1.165766f};
static const float GA[4 * 3] = {0.37689444f, 0.24156547f, 0.30238447f, 0.80570966f, 0.5184905f, 0.6703743f,
                                0.4199963f, 0.2735345f, 0.38693744f, 0.5321113f, 0.34252504f, 0.4438907f};
static const float GB[3 * 2] = {0.8737376f, 0.9888564f, 0.9339924f, 0.991189f, 1.1659734f, 1.2298465f};

static void compare(const char *what, const float *got, const float *want, int n, float tol) {
    for (int i = 0; i < n; i++)
        CHECK(fabsf(got[i] - want[i]) <= tol, "%s[%d] = %.9g, literal %.9g", what, i, got[i], want[i]);
}

int main(void) {
    dfdx_rocm_ctx *ctx = NULL;
    int rc = dfdx_rocm_create(0, NULL, &ctx);
    if (rc != DFDX_ROCM_OK) {
        fprintf(stderr, "dfdx_rocm_create: %d (%s)\n", rc, dfdx_rocm_strerror(rc));
        return 2;
    }
    char name[128];
    int cus = 0, mhz = 0;
    OK(dfdx_rocm_device_info(ctx, name, sizeof name, &cus, &mhz));
    printf("device: %s, %d compute units, %d MHz\n", name, cus, mhz);
    CHECK(cus > 0 && strstr(name, "gfx950") != NULL, "device info: %s / %d", name, cus);

    /* Storage::try_alloc_len + copy in (tensor/cuda/device.rs:259-266, tensor_from_vec) */
    void *a = NULL, *b = NULL, *r = NULL;
    OK(dfdx_rocm_alloc(ctx, sizeof A, 1, &a));
    OK(dfdx_rocm_alloc(ctx, sizeof B, 1, &b));
    OK(dfdx_rocm_alloc(ctx, sizeof R, 0, &r));   /* a forward output is overwritten: no fill (cuda_kernel.rs:253) */
    float zero_check[12];
    memset(zero_check, 0x7f, sizeof zero_check);
    OK(dfdx_rocm_copy_d2h(ctx, zero_check, a, sizeof A));
    for (int i = 0; i < 12; i++) CHECK(zero_check[i] == 0.0f, "alloc(zeroed) byte run %d not zero", i);
    OK(dfdx_rocm_copy_h2d(ctx, a, A, sizeof A));
    OK(dfdx_rocm_copy_h2d(ctx, b, B, sizeof B));

    /* MatMatKernel::forward (cpu_kernel.rs:235-254) */
    const int64_t ls[2] = {3, 1}, rs[2] = {2, 1};
    OK(dfdx_rocm_matmat_forward(ctx, DFDX_ROCM_F32, 4, 3, 2, a, ls, b, rs, r));
    float out[8];
    OK(dfdx_rocm_copy_d2h(ctx, out, r, sizeof out));
    compare("out", out, R, 8, 1e-6f);

    /* r.exp().mean().backward(): grad_out = exp(r) / 8, then MatMatKernel::backward (cpu_kernel.rs:255-287) into
       gradients that start as zeros -- one filled eagerly, one only declared zero */
    float go_h[8];
    for (int i = 0; i < 8; i++) go_h[i] = expf(out[i]) / 8.0f;
    void *go = NULL, *ga = NULL, *gb = NULL;
    OK(dfdx_rocm_alloc(ctx, sizeof go_h, 0, &go));
    OK(dfdx_rocm_copy_h2d(ctx, go, go_h, sizeof go_h));
    OK(dfdx_rocm_alloc(ctx, sizeof A, 1, &ga));
    OK(dfdx_rocm_alloc(ctx, sizeof B, DFDX_ROCM_ZERO_DEFERRED, &gb));
    OK(dfdx_rocm_matmat_backward(ctx, DFDX_ROCM_F32, 4, 3, 2, a, ls, ga, b, rs, gb, go));
    float ga_h[12], gb_h[6];
    OK(dfdx_rocm_copy_d2h(ctx, ga_h, ga, sizeof ga_h));
    OK(dfdx_rocm_copy_d2h(ctx, gb_h, gb, sizeof gb_h));
    compare("grad_a", ga_h, GA, 12, 1e-6f);
    compare("grad_b", gb_h, GB, 6, 1e-6f);
    /* gradients accumulate: a second backward doubles them */
    OK(dfdx_rocm_matmat_backward(ctx, DFDX_ROCM_F32, 4, 3, 2, a, ls, ga, b, rs, gb, go));
    OK(dfdx_rocm_synchronize(ctx));
    OK(dfdx_rocm_copy_d2h(ctx, ga_h, ga, sizeof ga_h));
    for (int i = 0; i < 12; i++) CHECK(fabsf(ga_h[i] - 2.0f * GA[i]) <= 2e-6f, "second backward: grad_a[%d] = %.9g", i, ga_h[i]);

    /* the same product through the descriptor entry, and the planner's answer for it */
    dfdx_rocm_gemm_desc d;
    memset(&d, 0, sizeof d);
    d.dtype = DFDX_ROCM_F32;
    d.m = 4; d.k = 3; d.n = 2;
    d.batch1 = d.batch2 = 1;
    d.a = a; d.a_rs = 3; d.a_cs = 1;
    d.b = b; d.b_rs = 2; d.b_cs = 1;
    d.c = r; d.c_rs = 2; d.c_cs = 1;
    int kernel = -1, variant = -1;
    char plan[96];
    OK(dfdx_rocm_gemm_plan(ctx, &d, &kernel, &variant, plan, sizeof plan));
    printf("plan for 4x3x2 f32: %s\n", plan);
    OK(dfdx_rocm_gemm(ctx, &d));
    OK(dfdx_rocm_gemm_noalloc(ctx, &d));
    OK(dfdx_rocm_copy_d2h(ctx, out, r, sizeof out));
    compare("out (descriptor entry)", out, R, 8, 1e-6f);

    /* Cache (tensor/storage_traits.rs:41-77): a freed buffer is kept and comes back for the same size */
    size_t held = 99, held_bytes = 99;
    OK(dfdx_rocm_enable_cache(ctx));
    OK(dfdx_rocm_free(ctx, ga));
    OK(dfdx_rocm_cache_stats(ctx, &held, &held_bytes));
    CHECK(held == 1 && held_bytes == sizeof A, "cache after one free: %zu buffers, %zu bytes", held, held_bytes);
    void *again = NULL;
    OK(dfdx_rocm_alloc(ctx, sizeof A, 1, &again));
    CHECK(again == ga, "the cached buffer did not come back (%p vs %p)", again, ga);
    OK(dfdx_rocm_copy_d2h(ctx, ga_h, again, sizeof ga_h));
    for (int i = 0; i < 12; i++) CHECK(ga_h[i] == 0.0f, "recycled buffer not zero-filled again at %d", i);
    OK(dfdx_rocm_free(ctx, again));
    OK(dfdx_rocm_empty_cache(ctx));
    OK(dfdx_rocm_cache_stats(ctx, &held, &held_bytes));
    CHECK(held == 0 && held_bytes == 0, "cache after empty: %zu buffers", held);
    OK(dfdx_rocm_disable_cache(ctx));

    /* error model: codes, not aborts */
    CHECK(dfdx_rocm_gemm(ctx, NULL) == DFDX_ROCM_ERR_INVALID_ARG, "null descriptor");
    d.dtype = 17;
    CHECK(dfdx_rocm_gemm(ctx, &d) == DFDX_ROCM_ERR_INVALID_ARG, "unknown dtype");
    d.dtype = DFDX_ROCM_F32;
    d.c_b1 = 0; d.batch1 = 2;
    CHECK(dfdx_rocm_gemm(ctx, &d) == DFDX_ROCM_ERR_ALIASED_OUTPUT, "zero batch stride of C");
    CHECK(dfdx_rocm_matmat_forward(ctx, DFDX_ROCM_F32, 4, 3, 2, NULL, ls, b, rs, r) == DFDX_ROCM_ERR_INVALID_ARG, "null lhs");
    const int codes[] = {DFDX_ROCM_OK, DFDX_ROCM_ERR_INVALID_ARG, DFDX_ROCM_ERR_UNSUPPORTED, DFDX_ROCM_ERR_NO_DEVICE,
                         DFDX_ROCM_ERR_ALIASED_OUTPUT, DFDX_ROCM_ERR_SCRATCH_TOO_SMALL, 2 /* a HIP code */, -99};
    for (size_t i = 0; i < sizeof codes / sizeof codes[0]; i++) {
        const char *msg = dfdx_rocm_strerror(codes[i]);
        CHECK(msg != NULL && msg[0] != '\0', "strerror(%d)", codes[i]);
    }
    dfdx_rocm_ctx *none = NULL;
    CHECK(dfdx_rocm_create(4096, NULL, &none) == DFDX_ROCM_ERR_NO_DEVICE && none == NULL, "create on a device that does not exist");

    OK(dfdx_rocm_free(ctx, a));
    OK(dfdx_rocm_free(ctx, b));
    OK(dfdx_rocm_free(ctx, r));
    OK(dfdx_rocm_free(ctx, go));
    OK(dfdx_rocm_free(ctx, gb));
    OK(dfdx_rocm_free(ctx, NULL));
    OK(dfdx_rocm_destroy(ctx));
    OK(dfdx_rocm_destroy(NULL));
    if (failures) {
        fprintf(stderr, "%d check(s) failed\n", failures);
        return 1;
    }
    printf("c host ok\n");
    return 0;
}
