// fprop / dgrad implicit-GEMM kernels, storage type bf16: tile selection + instantiation.
#include "conv_kernels.h"
namespace luxhip {
template <>
int launch_conv_gemm_any<bf16_t>(hipStream_t s, ConvGemmArgs<bf16_t>& a) {
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    if (a.Ncols > 64 && ceil_div(a.gather.M, 256) * ceil_div(a.Ncols, 128) >= cus) return launch_conv_gemm<bf16_t, 4, 2>(s, a);
    if (a.Ncols > 64 && a.gather.M > 64) return launch_conv_gemm<bf16_t, 2, 2>(s, a);
    return launch_conv_gemm<bf16_t, 1, 1>(s, a);
}
// whole-tap stages: 256 x 256 tiles on 8 waves when there are that many output columns, else
// 256 x 128 on 4 waves with 3 LDS stages (two workgroups per compute unit)
template <>
int launch_conv_tap_any<bf16_t>(hipStream_t s, ConvTapArgs<bf16_t>& a) {
    if (a.Ncols > 128) return launch_conv_tap<bf16_t, 4, 2, 4, 4>(s, a);
    return launch_conv_tap<bf16_t, 4, 2, 2, 3>(s, a);
}
}  // namespace luxhip
