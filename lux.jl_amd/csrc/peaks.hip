// Achievable peaks of the device, measured with the simplest kernels that reach them: a streaming copy
// (HBM) and register-only MFMA loops (matrix pipes).  The benchmark reports them next to the published
// figures that its roofline fractions divide by.
#include <stdint.h>

#include "common.h"

namespace luxhip {
namespace {

typedef __bf16 bf16x8_p __attribute__((ext_vector_type(8)));
typedef float f32x4_p __attribute__((ext_vector_type(4)));
typedef float f32x16_p __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void peak_copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = src[min(i + (size_t)u * 256, n - 1)];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (i + (size_t)u * 256 < n) dst[i + (size_t)u * 256] = v[u];
}

// Operands: pseudo-random values in (-1, 1) (the rate the matrix pipes sustain depends on how many bits
// toggle: all-equal operands run about 10 % faster than random ones at the same power limit).
__global__ __launch_bounds__(512) void peak_mfma_bf16_kernel(float* out, int iters) {
    f32x4_p acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = f32x4_p{0.f, 0.f, 0.f, 0.f};
    bf16x8_p a, b;
    uint32_t st = threadIdx.x * 7919u + blockIdx.x * 104729u + 1u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        st = st * 1664525u + 1013904223u;
        a[i] = (__bf16)(((int)(st >> 8) % 2001 - 1000) * 0.001f);
        st = st * 1664525u + 1013904223u;
        b[i] = (__bf16)(((int)(st >> 8) % 2001 - 1000) * 0.001f);
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (sum == 12345.678f) out[0] = sum;
}

__global__ __launch_bounds__(512) void peak_mfma_f32_kernel(float* out, int iters) {
    f32x16_p acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    uint32_t st = threadIdx.x * 7919u + blockIdx.x * 104729u + 1u;
    st = st * 1664525u + 1013904223u;
    const float a = ((int)(st >> 8) % 2001 - 1000) * 0.001f;
    st = st * 1664525u + 1013904223u;
    const float b = ((int)(st >> 8) % 2001 - 1000) * 0.001f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += acc[i][r];
    if (sum == 12345.678f) out[0] = sum;
}

template <typename Launch>
int time_ms(hipStream_t s, int warm, int reps, Launch&& launch, float* ms) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err == hipSuccess) {
        for (int i = 0; i < warm; ++i) launch();
        err = hipEventRecord(e0, s);
    }
    if (err == hipSuccess) {
        for (int i = 0; i < reps; ++i) launch();
        err = hipEventRecord(e1, s);
    }
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    if (err == hipSuccess) err = hipEventElapsedTime(ms, e0, e1);
    if (err == hipSuccess) err = hipGetLastError();
    if (e0) (void)hipEventDestroy(e0);       // on every path
    if (e1) (void)hipEventDestroy(e1);
    LUX_CHECK_HIP(err);
    *ms /= (float)reps;
    return LUXHIP_OK;
}

}  // namespace
}  // namespace luxhip

using namespace luxhip;

extern "C" int luxhip_measure_peaks(luxhip_stream_t stream, double* copy_GBps, double* mfma_bf16_TFLOPs, double* mfma_f32_TFLOPs) {
    LUX_REQUIRE_INIT();
    hipStream_t s = (hipStream_t)stream;
    const int cus = num_cus() > 0 ? num_cus() : 256;
    float ms = 0.f;
    int rc;
    if (copy_GBps) {
        // 1 GiB moved per launch (512 MiB read + 512 MiB written): twice the size of the Infinity Cache
        const size_t bytes = size_t(512) << 20, n = bytes / 16;
        // through the pooled allocator: it gives its free blocks back to the driver and retries when memory is short
        void *a = nullptr, *b = nullptr;
        if ((rc = luxhip_malloc(&a, bytes)) != LUXHIP_OK) return rc;
        if ((rc = luxhip_malloc(&b, bytes)) != LUXHIP_OK) { (void)luxhip_free(a); return rc; }
        (void)hipMemsetAsync(a, 0x11, bytes, s);
        rc = time_ms(s, 3, 10, [&] {
            peak_copy_kernel<<<dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, s>>>((const float4*)a, (float4*)b, n);
        }, &ms);
        (void)luxhip_free(a);
        (void)luxhip_free(b);
        if (rc != LUXHIP_OK) return rc;
        *copy_GBps = 2.0 * (double)bytes / (ms * 1e-3) / 1e9;
    }
    float* out = nullptr;
    LUX_CHECK_HIP(hipMalloc((void**)&out, 64));
    if (mfma_bf16_TFLOPs) {
        // 8 waves per compute unit; about 0.3 s of warm-up: the clocks settle under the load
        const int iters = 4000;
        rc = time_ms(s, 60, 10, [&] { peak_mfma_bf16_kernel<<<dim3((unsigned)cus), dim3(512), 0, s>>>(out, iters); }, &ms);
        if (rc != LUXHIP_OK) { (void)hipFree(out); return rc; }
        *mfma_bf16_TFLOPs = (double)iters * 32 * 8 * cus * (2.0 * 16 * 16 * 32) / (ms * 1e-3) / 1e12;
    }
    if (mfma_f32_TFLOPs) {
        const int iters = 2000;
        rc = time_ms(s, 10, 5, [&] { peak_mfma_f32_kernel<<<dim3((unsigned)cus), dim3(512), 0, s>>>(out, iters); }, &ms);
        if (rc != LUXHIP_OK) { (void)hipFree(out); return rc; }
        *mfma_f32_TFLOPs = (double)iters * 16 * 8 * cus * (2.0 * 32 * 32 * 2) / (ms * 1e-3) / 1e12;
    }
    (void)hipFree(out);
    return LUXHIP_OK;
}
