// fprop / dgrad with the input window of a tile held in LDS (bf16): launch.
#define LUXHIP_CONV_PATCH_KERNEL
#include "conv_patch.h"
#include "conv_patch_narrow.h"
namespace luxhip {
namespace cpatch {
int launch(hipStream_t s, const Problem& p) {
    static ResidentOnce ro;   // here only the one-time raise of the dynamic LDS limit
    ro.get([&](hipError_t& err) {
        const void* kernels[4] = {reinterpret_cast<const void*>(conv_patch_kernel<false>), reinterpret_cast<const void*>(conv_patch_kernel<true>),
                                  reinterpret_cast<const void*>(conv_patch_narrow_kernel<false>),
                                  reinterpret_cast<const void*>(conv_patch_narrow_kernel<true>)};
        err = hipSuccess;
        for (const void* k : kernels)
            if (err == hipSuccess) err = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
        return 1;
    });
    LUX_CHECK_HIP(ro.error);
    Args a;
    a.src = p.src; a.wm = p.wm; a.bias = p.bias; a.out = p.out; a.pre = p.pre; a.zero = p.zero;
    a.Ctot = p.Ctot; a.Cg = p.Cg;
    a.P = p.P; a.Q = p.Q; a.NQ = p.N * p.Q; a.PQ = p.P * p.Q; a.M = a.PQ * p.N;
    a.kW = p.kW; a.kH = p.kH; a.H = p.Cg / 64;
    a.rev = p.dgrad ? 1 : 0;
    a.hlo = p.dgrad ? p.kW - 1 - p.pad_w : p.pad_w;
    a.dq_min = p.dgrad ? p.pad_h - (p.kH - 1) : -p.pad_h;
    a.pitch = p.P + p.kW - 1;
    a.Ncols = p.Ncols; a.col_off = p.col_off; a.Ctot_out = p.Ctot_out; a.act = p.act;
    // at most 64 output channels: the kernel whose eight waves share 64 columns (the one for 128 would leave half of
    // its waves multiplying columns that are never stored); the option forces either (1: tiles of 64, 2: of 128)
    const int64_t forced = option_conv_tile();
    const bool narrow = forced == 1 || (forced != 2 && a.Ncols <= 64);
    a.tiles_n = (int)ceil_div(a.Ncols, narrow ? 64 : TILE_N);
    a.frags = (int)ceil_div(a.M, 16);
    a.staged = a.PQ % 8 == 0 && a.pre == nullptr && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0;
    a.divP = FastDiv((uint32_t)a.P); a.divQ = FastDiv((uint32_t)a.Q); a.divPQ = FastDiv((uint32_t)a.PQ);
    a.divPitch = FastDiv((uint32_t)a.pitch);
    // the LDS holds one workgroup per compute unit: as many workgroups as compute units share the fragments evenly
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    a.groups_m = (int)std::max<int64_t>(1, std::min<int64_t>(cus / a.tiles_n, ceil_div(a.frags, 16)));
    const int grid = a.groups_m * a.tiles_n;
    ProfScope ps(p.dgrad ? "conv_dgrad_kernel<bf16>" : "conv_fprop_kernel<bf16>", s);
    // identity and relu have a kernel of their own, a few times smaller than the one with every activation inlined
    const bool any_act = a.act != LUXHIP_ACT_IDENTITY && a.act != LUXHIP_ACT_RELU;
    const dim3 g((unsigned)grid), b(THREADS);
    if (narrow) {
        if (any_act) conv_patch_narrow_kernel<true><<<g, b, LDS_BYTES, s>>>(a);
        else conv_patch_narrow_kernel<false><<<g, b, LDS_BYTES, s>>>(a);
    } else {
        if (any_act) conv_patch_kernel<true><<<g, b, LDS_BYTES, s>>>(a);
        else conv_patch_kernel<false><<<g, b, LDS_BYTES, s>>>(a);
    }
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}
}  // namespace cpatch
}  // namespace luxhip
