/* A host program in plain C on the C ABI of libluxhip: the known answers that the reference's own
 * layer tests hold, computed through the library without any other host layer.
 *   Dense(10 => 2) with ones, x = ones(10, 3), bias = ones(2): every output is 11
 *       (test/core_layers/dense_tests.jl, "ones" known answers)
 *   BatchNorm(2) in training mode on x = [1 3 5; 2 4 6]: y = +-1.22474 and 0, running mean 0.3 / 0.4,
 *       running variance 1.3 (test/core_layers/normalize_tests.jl:25-49)
 * Prints OK and returns 0 when both hold. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "luxhip.h"

#define CHECK(call)                                                                   \
    do {                                                                              \
        int rc_ = (call);                                                             \
        if (rc_ != LUXHIP_OK) {                                                       \
            fprintf(stderr, "%s -> %d: %s\n", #call, rc_, luxhip_last_error());       \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

static int upload(void** dev, const float* host, size_t n, luxhip_stream_t s) {
    int rc = luxhip_malloc(dev, n * sizeof(float));
    return rc != LUXHIP_OK ? rc : luxhip_memcpy_h2d(*dev, host, n * sizeof(float), s);
}

int main(void) {
    CHECK(luxhip_init(0));
    luxhip_stream_t s;
    CHECK(luxhip_stream_create(&s));

    /* dense: y (2 x 3) = W (2 x 10) * x (10 x 3) .+ b, identity */
    float W[20], x[30], b[2] = {1.0f, 1.0f}, y[6];
    for (int i = 0; i < 20; ++i) W[i] = 1.0f;
    for (int i = 0; i < 30; ++i) x[i] = 1.0f;
    void *dW, *dx, *db, *dy;
    CHECK(upload(&dW, W, 20, s));
    CHECK(upload(&dx, x, 30, s));
    CHECK(upload(&db, b, 2, s));
    CHECK(luxhip_malloc(&dy, sizeof(y)));
    CHECK(luxhip_fused_dense_fwd(s, LUXHIP_F32, LUXHIP_ACT_IDENTITY, 2, 10, 3, dW, 2, dx, 10, db, dy, 2, NULL));
    CHECK(luxhip_memcpy_d2h(y, dy, sizeof(y), s));
    for (int i = 0; i < 6; ++i)
        if (fabsf(y[i] - 11.0f) > 1e-5f) { fprintf(stderr, "dense: y[%d] = %g, expected 11\n", i, y[i]); return 1; }

    /* batchnorm: x (2 features x 3 samples, column-major) = [1 3 5; 2 4 6] */
    float bx[6] = {1, 2, 3, 4, 5, 6}, rm[2] = {0, 0}, rv[2] = {1, 1}, by[6], rm2[2], rv2[2];
    void *dbx, *drm, *drv, *dby, *drm2, *drv2;
    CHECK(upload(&dbx, bx, 6, s));
    CHECK(upload(&drm, rm, 2, s));
    CHECK(upload(&drv, rv, 2, s));
    CHECK(luxhip_malloc(&dby, sizeof(by)));
    CHECK(luxhip_malloc(&drm2, sizeof(rm2)));
    CHECK(luxhip_malloc(&drv2, sizeof(rv2)));
    /* (I, C, N) = (1, 2, 3); no scale / bias; momentum 0.1, eps 1e-5 */
    CHECK(luxhip_batchnorm_fwd(s, LUXHIP_F32, LUXHIP_ACT_IDENTITY, 1, 2, 3, dbx, NULL, NULL, drm, drv, 1, 0.1, 1e-5, dby, drm2,
                               drv2, NULL, NULL));
    CHECK(luxhip_memcpy_d2h(by, dby, sizeof(by), s));
    CHECK(luxhip_memcpy_d2h(rm2, drm2, sizeof(rm2), s));
    CHECK(luxhip_memcpy_d2h(rv2, drv2, sizeof(rv2), s));
    const float want[6] = {-1.22474f, -1.22474f, 0.0f, 0.0f, 1.22474f, 1.22474f};
    for (int i = 0; i < 6; ++i)
        if (fabsf(by[i] - want[i]) > 1e-4f) { fprintf(stderr, "batchnorm: y[%d] = %g, expected %g\n", i, by[i], want[i]); return 1; }
    if (fabsf(rm2[0] - 0.3f) > 1e-5f || fabsf(rm2[1] - 0.4f) > 1e-5f || fabsf(rv2[0] - 1.3f) > 1e-5f || fabsf(rv2[1] - 1.3f) > 1e-5f) {
        fprintf(stderr, "batchnorm: running statistics %g %g %g %g\n", rm2[0], rm2[1], rv2[0], rv2[1]);
        return 1;
    }

    void* all[] = {dW, dx, db, dy, dbx, drm, drv, dby, drm2, drv2};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); ++i) CHECK(luxhip_free(all[i]));
    CHECK(luxhip_stream_destroy(s));
    CHECK(luxhip_shutdown());
    printf("OK\n");
    return 0;
}
