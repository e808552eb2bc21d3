// Convolutions with three spatial dims, reduced to the two-dimensional kernels.
//
// x (W, H, D, C, N) is unfolded along the depth: xu (W, H, KD*C, Dout*N) holds, for output depth
// od and depth tap kd, the depth slice od*sd + kd*dd - pd of x (zeros outside), as channel
// kd' + KD*c of sample od + Dout*n.  The weight (kW, kH, KD, C/groups, Cout) read as
// (kW, kH, KD*C/groups, Cout) has exactly that channel order, so the three-dimensional problem
// is the two-dimensional one on xu with the same memory for the weight and its gradient; the
// groups stay contiguous.  True convolution pairs weight index kd' with tap KD-1-kd',
// cross-correlation with kd'.
//   conv_depth_unfold  x  -> xu                (reads x once, writes KD times its size)
//   conv_depth_fold    dxu -> dx               (the adjoint: every dx element gathers its <= KD terms)
//   swap_middle_dims   (inner, A, B, outer) -> (inner, B, A, outer): y (OW*OH, Cout, Dout, N) of the
//                      two-dimensional problem <-> (OW*OH, Dout, Cout, N) of the caller
// All three are HBM copies: lanes run along the contiguous plane (16-byte units when the plane
// and the pointers allow), rows are decoded once per thread.
#include <algorithm>

#include "common.h"

namespace luxhip {

constexpr int kDepthThreads = 256;

struct DepthGeom {
    uint32_t PU;            // units per (w, h) plane
    uint32_t D, C, N, KD, Dout;
    int32_t sd, pd, dd;
    uint32_t flipkernel;
    uint32_t rows;          // rows of the output of the kernel
};

template <typename U>
__device__ __forceinline__ U zero_unit() {
    if constexpr (sizeof(U) == 16) return make_uint4(0, 0, 0, 0);
    else return (U)0;
}

template <typename U>
__global__ __launch_bounds__(kDepthThreads) void conv_depth_unfold_kernel(const U* __restrict__ x, U* __restrict__ xu, DepthGeom g) {
    const uint32_t pu = blockIdx.x * kDepthThreads + threadIdx.x;
    if (pu >= g.PU) return;
    const uint32_t J = g.KD * g.C;
    for (uint32_t row = blockIdx.y; row < g.rows; row += gridDim.y) {       // row = (j, od, n), j fastest
        const uint32_t j = row % J, r = row / J;
        const uint32_t od = r % g.Dout, n = r / g.Dout;
        const uint32_t kdw = j % g.KD, c = j / g.KD;
        const uint32_t kd = g.flipkernel ? kdw : g.KD - 1 - kdw;
        const int32_t id = (int32_t)od * g.sd + (int32_t)kd * g.dd - g.pd;
        U v = zero_unit<U>();
        if (id >= 0 && id < (int32_t)g.D) v = x[(((size_t)n * g.C + c) * g.D + (uint32_t)id) * g.PU + pu];
        xu[(size_t)row * g.PU + pu] = v;
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kDepthThreads) void conv_depth_fold_kernel(const T* __restrict__ dxu, T* __restrict__ dx, DepthGeom g) {
    const uint32_t pu = blockIdx.x * kDepthThreads + threadIdx.x;
    if (pu >= g.PU) return;
    const uint32_t J = g.KD * g.C;
    for (uint32_t row = blockIdx.y; row < g.rows; row += gridDim.y) {       // row = (id, c, n), id fastest
        const uint32_t id = row % g.D, r = row / g.D;
        const uint32_t c = r % g.C, n = r / g.C;
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
        for (uint32_t kd = 0; kd < g.KD; ++kd) {                             // fixed order: deterministic sums
            const int32_t t = (int32_t)id + g.pd - (int32_t)kd * g.dd;
            if (t < 0 || t % g.sd != 0) continue;
            const uint32_t od = (uint32_t)(t / g.sd);
            if (od >= g.Dout) continue;
            const uint32_t kdw = g.flipkernel ? kd : g.KD - 1 - kd;
            const size_t off = ((((size_t)n * g.Dout + od) * J) + kdw + (size_t)g.KD * c) * g.PU * VEC + (size_t)pu * VEC;
            float v[VEC];
            if constexpr (VEC == 1) v[0] = ld(dxu + off);
            else Vec<T>::load(dxu + off, v);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += v[e];
        }
        const size_t o = ((size_t)row * g.PU + pu) * VEC;
        if constexpr (VEC == 1) st(dx + o, acc[0]);
        else Vec<T>::store(dx + o, acc);
    }
}

template <typename U>
__global__ __launch_bounds__(kDepthThreads) void swap_middle_dims_kernel(const U* __restrict__ in, U* __restrict__ out, uint32_t IU,
                                                                        uint32_t A, uint32_t B, uint32_t rows) {
    const uint32_t i = blockIdx.x * kDepthThreads + threadIdx.x;
    if (i >= IU) return;
    for (uint32_t row = blockIdx.y; row < rows; row += gridDim.y) {          // output row = (b, a, o), b fastest
        const uint32_t b = row % B, r = row / B;
        const uint32_t a = r % A, o = r / A;
        out[(size_t)row * IU + i] = in[(((size_t)o * B + b) * A + a) * IU + i];
    }
}

static dim3 depth_grid(uint32_t units, uint32_t rows) {
    return dim3((units + kDepthThreads - 1) / kDepthThreads, std::min<uint32_t>(rows, 65535u));
}

static int depth_check(int dtype, int64_t plane, int64_t D, int64_t C, int64_t N, int64_t KD, int64_t Dout, int64_t sd,
                       int64_t pd, int64_t dd, DepthGeom* g, int64_t out_rows) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(plane < 0 || D < 0 || C < 0 || N < 0 || KD <= 0 || Dout < 0 || sd <= 0 || dd <= 0 || pd < 0,
                   "conv depth transform: invalid dimension");
    const long double big = 2147483648.0L;
    LUX_UNSUPPORTED_IF((long double)plane * D * C * std::max<int64_t>(N, 1) >= big ||
                           (long double)plane * KD * C * Dout * std::max<int64_t>(N, 1) >= big || (long double)out_rows >= big,
                       "conv depth transform: tensors of 2^31 or more elements are not supported");
    g->D = (uint32_t)D; g->C = (uint32_t)C; g->N = (uint32_t)N; g->KD = (uint32_t)KD; g->Dout = (uint32_t)Dout;
    g->sd = (int32_t)sd; g->pd = (int32_t)pd; g->dd = (int32_t)dd;
    g->rows = (uint32_t)out_rows;
    return LUXHIP_OK;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_conv_depth_unfold(luxhip_stream_t s, int dtype, int64_t plane, int64_t D, int64_t C, int64_t N, int64_t KD,
                             int64_t Dout, int64_t stride_d, int64_t pad_d_lo, int64_t dil_d, int flipkernel, const void* x,
                             void* xu) {
    LUX_REQUIRE_INIT();
    DepthGeom g{};
    int rc = depth_check(dtype, plane, D, C, N, KD, Dout, stride_d, pad_d_lo, dil_d, &g, KD * C * Dout * N);
    if (rc != LUXHIP_OK) return rc;
    g.flipkernel = flipkernel ? 1u : 0u;
    if (plane == 0 || g.rows == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || xu == nullptr, "conv_depth_unfold: x and xu must not be NULL");
    const size_t esize = dtype == LUXHIP_F32 ? 4 : 2;
    ProfScope ps("conv_depth_unfold_kernel", (hipStream_t)s);
    if ((plane * esize) % 16 == 0 && aligned16(x) && aligned16(xu)) {
        g.PU = (uint32_t)(plane * esize / 16);
        conv_depth_unfold_kernel<uint4><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, (hipStream_t)s>>>((const uint4*)x, (uint4*)xu, g);
    } else if (dtype == LUXHIP_F32) {
        g.PU = (uint32_t)plane;
        conv_depth_unfold_kernel<uint32_t><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, (hipStream_t)s>>>((const uint32_t*)x, (uint32_t*)xu, g);
    } else {
        g.PU = (uint32_t)plane;
        conv_depth_unfold_kernel<uint16_t><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, (hipStream_t)s>>>((const uint16_t*)x, (uint16_t*)xu, g);
    }
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

int luxhip_conv_depth_fold(luxhip_stream_t s, int dtype, int64_t plane, int64_t D, int64_t C, int64_t N, int64_t KD,
                           int64_t Dout, int64_t stride_d, int64_t pad_d_lo, int64_t dil_d, int flipkernel, const void* dxu,
                           void* dx) {
    LUX_REQUIRE_INIT();
    DepthGeom g{};
    int rc = depth_check(dtype, plane, D, C, N, KD, Dout, stride_d, pad_d_lo, dil_d, &g, D * C * N);
    if (rc != LUXHIP_OK) return rc;
    g.flipkernel = flipkernel ? 1u : 0u;
    if (plane == 0 || g.rows == 0) return LUXHIP_OK;
    LUX_INVALID_IF(dx == nullptr || (dxu == nullptr && Dout > 0), "conv_depth_fold: dxu and dx must not be NULL");
    const hipStream_t st = (hipStream_t)s;
    ProfScope ps("conv_depth_fold_kernel", st);
    if (dtype == LUXHIP_F32) {
        if (plane % 4 == 0 && aligned16(dxu) && aligned16(dx)) {
            g.PU = (uint32_t)(plane / 4);
            conv_depth_fold_kernel<float, 4><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, st>>>((const float*)dxu, (float*)dx, g);
        } else {
            g.PU = (uint32_t)plane;
            conv_depth_fold_kernel<float, 1><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, st>>>((const float*)dxu, (float*)dx, g);
        }
    } else {
        if (plane % 8 == 0 && aligned16(dxu) && aligned16(dx)) {
            g.PU = (uint32_t)(plane / 8);
            conv_depth_fold_kernel<bf16_t, 8><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, st>>>((const bf16_t*)dxu, (bf16_t*)dx, g);
        } else {
            g.PU = (uint32_t)plane;
            conv_depth_fold_kernel<bf16_t, 1><<<depth_grid(g.PU, g.rows), kDepthThreads, 0, st>>>((const bf16_t*)dxu, (bf16_t*)dx, g);
        }
    }
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

int luxhip_swap_middle_dims(luxhip_stream_t s, int dtype, int64_t inner, int64_t A, int64_t B, int64_t outer, const void* in,
                            void* out) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(inner < 0 || A < 0 || B < 0 || outer < 0, "swap_middle_dims: negative dimension");
    LUX_UNSUPPORTED_IF((long double)inner * A * B * std::max<int64_t>(outer, 1) >= 2147483648.0L,
                       "swap_middle_dims: tensors of 2^31 or more elements are not supported");
    if (inner * A * B * outer == 0) return LUXHIP_OK;
    LUX_INVALID_IF(in == nullptr || out == nullptr || in == out, "swap_middle_dims: in and out must be distinct buffers");
    const size_t esize = dtype == LUXHIP_F32 ? 4 : 2;
    const uint32_t rows = (uint32_t)(A * B * outer);
    const hipStream_t st = (hipStream_t)s;
    ProfScope ps("swap_middle_dims_kernel", st);
    if ((inner * esize) % 16 == 0 && aligned16(in) && aligned16(out)) {
        const uint32_t IU = (uint32_t)(inner * esize / 16);
        swap_middle_dims_kernel<uint4><<<depth_grid(IU, rows), kDepthThreads, 0, st>>>((const uint4*)in, (uint4*)out, IU, (uint32_t)A, (uint32_t)B, rows);
    } else if (dtype == LUXHIP_F32) {
        swap_middle_dims_kernel<uint32_t><<<depth_grid((uint32_t)inner, rows), kDepthThreads, 0, st>>>((const uint32_t*)in, (uint32_t*)out, (uint32_t)inner, (uint32_t)A, (uint32_t)B, rows);
    } else {
        swap_middle_dims_kernel<uint16_t><<<depth_grid((uint32_t)inner, rows), kDepthThreads, 0, st>>>((const uint16_t*)in, (uint16_t*)out, (uint32_t)inner, (uint32_t)A, (uint32_t)B, rows);
    }
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

}  // extern "C"
