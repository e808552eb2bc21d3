// fprop / dgrad implicit-GEMM kernels, storage type f32: tile selection + instantiation.
#include "conv_kernels.h"
namespace luxhip {
template <>
int launch_conv_gemm_any<float>(hipStream_t s, ConvGemmArgs<float>& a) {
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    if (a.Ncols > 64 && ceil_div(a.gather.M, 256) * ceil_div(a.Ncols, 128) >= cus) return launch_conv_gemm<float, 4, 2>(s, a);
    if (a.Ncols > 64 && a.gather.M > 64) return launch_conv_gemm<float, 2, 2>(s, a);
    return launch_conv_gemm<float, 1, 1>(s, a);
}
// whole-tap stages through registers: 128 x 128 tiles (two workgroups per compute unit)
template <>
int launch_conv_tap_any<float>(hipStream_t s, ConvTapArgs<float>& a) {
    return launch_conv_tap<float, 2, 2, 2, 0>(s, a);
}
}  // namespace luxhip
