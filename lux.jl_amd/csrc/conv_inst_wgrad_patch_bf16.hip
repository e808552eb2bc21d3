// filter gradient with the input window of a tile held in LDS (bf16): launch.
#define LUXHIP_CONV_WGRAD_PATCH_KERNEL
#include "conv_wgrad_patch.h"
namespace luxhip {
namespace wpatch {
int launch(hipStream_t s, const Problem& p) {
    static ResidentOnce ro;   // here only the one-time raise of the dynamic LDS limit
    ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(conv_wgrad_patch_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)LDS_BYTES);
        return 1;
    });
    LUX_CHECK_HIP(ro.error);
    Args a;
    a.src = p.src; a.dz = p.dz; a.partial = p.partial; a.zero = p.zero;
    a.Ctot = p.Ctot; a.Cg = p.Cg; a.Cout = p.Cout; a.Ncols = p.Ncols;
    a.P = p.P; a.Q = p.Q; a.PQ = p.P * p.Q; a.N = p.N;
    a.pad_w = p.pad_w; a.pad_h = p.pad_h; a.pitch = p.P + 2;
    a.H = p.Cg / 64; a.CB = (p.Ncols + 63) / 64;
    a.lanes = image_lanes(p.N, a.H * a.CB, num_cus() > 0 ? num_cus() : 256);
    a.divP = FastDiv((uint32_t)a.P); a.divPitch = FastDiv((uint32_t)a.pitch);
    ProfScope ps("conv_wgrad_kernel<bf16>", s);
    conv_wgrad_patch_kernel<<<dim3((unsigned)(((a.lanes + 7) / 8) * 8 * a.H * a.CB)), dim3(THREADS), LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}
}  // namespace wpatch
}  // namespace luxhip
