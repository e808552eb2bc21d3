// wgrad implicit-GEMM kernels, storage type bf16: tile selection + instantiation.
#include "conv_kernels.h"
namespace luxhip {
template <>
int launch_conv_wgrad_any<bf16_t>(hipStream_t s, ConvWgradArgs<bf16_t>& a, int slices, bool small) {
    if (small) return launch_conv_wgrad<bf16_t, 1, 1>(s, a, slices);
    return launch_conv_wgrad<bf16_t, 2, 2>(s, a, slices);
}
// 128 x 128 tiles on 4 waves, 4 LDS stages (two workgroups per compute unit)
int launch_conv_wgrad_direct(hipStream_t s, ConvWgradDirectArgs& a, int slices) {
    using ML = GemmMainloop<bf16_t, 2, 2, false, true, true, 2, 4, 2>;
    a.tiles_m = (int)ceil_div(a.A.Mrows, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.B.Ncols, ML::TILE_N);
    auto kernel = conv_wgrad_direct_kernel<2, 2, 2, 4, 2>;
    static ResidentOnce ro;   // here only the one-time raise of the dynamic LDS limit
    ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return 1;
    });
    LUX_CHECK_HIP(ro.error);
    ProfScope ps("conv_wgrad_kernel<bf16>", s);
    a.slices = slices;
    kernel<<<dim3((unsigned)(a.tiles_m * a.tiles_n * slices)), dim3(ML::THREADS), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}
}  // namespace luxhip
