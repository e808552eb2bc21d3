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
// whole-tap stages, 8 waves of 128 x 64 each: 256 x 256 tiles when there are that many output
// columns, else 512 x 128 (4 x 2 waves); small problems take 256 x 128 on 4 waves
template <>
int launch_conv_tap_any<bf16_t>(hipStream_t s, ConvTapArgs<bf16_t>& a) {
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    const int tile = (int)option_conv_tile();
    if (tile == 82 || (tile == 0 && a.Ncols > 128)) return launch_conv_tap<bf16_t, 4, 2, 4, 4>(s, a);
    if (tile == 84 || (tile == 0 && ceil_div(a.tap.M, 512) >= cus)) return launch_conv_tap<bf16_t, 4, 2, 2, 4, 4>(s, a);
    if (tile == 83) return launch_conv_tap<bf16_t, 4, 2, 2, 3, 4>(s, a);
    return launch_conv_tap<bf16_t, 4, 2, 2, 3>(s, a);
}
}  // namespace luxhip
