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
// whole-tap stages through registers: 128 x 128 tiles (two workgroups per compute unit).  The
// tiles run in rounds of `resident` workgroups; a last round with only a few tiles (at most 10 %
// of all) would cost a whole tile time for little work, so those rows go to 64 x 64 tiles.
template <>
int launch_conv_tap_any<float>(hipStream_t s, ConvTapArgs<float>& a) {
    const int64_t resident = conv_tap_resident<float, 2, 2, 2, 0>();
    const int64_t tiles_m = ceil_div(a.tap.M, 128);
    if (resident > 0 && a.Ncols <= 128 && tiles_m > resident) {
        const int64_t rem = tiles_m % resident;
        if (rem != 0 && rem * 10 <= tiles_m) {
            ConvTapArgs<float> big = a, rest = a;
            big.tap.M = (int)((tiles_m - rem) * 128);    // rows past this belong to the second launch
            rest.m_begin = big.tap.M;
            int rc = launch_conv_tap<float, 2, 2, 2, 0>(s, big);
            if (rc != LUXHIP_OK) return rc;
            return launch_conv_tap<float, 1, 1, 2, 0>(s, rest);
        }
    }
    return launch_conv_tap<float, 2, 2, 2, 0>(s, a);
}
}  // namespace luxhip
