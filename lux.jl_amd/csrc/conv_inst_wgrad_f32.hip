// wgrad implicit-GEMM kernels, storage type f32: tile selection + instantiation.
#include "conv_kernels.h"
namespace luxhip {
template <>
int launch_conv_wgrad_any<float>(hipStream_t s, ConvWgradArgs<float>& a, int slices, bool small) {
    if (small) return launch_conv_wgrad<float, 1, 1>(s, a, slices);
    return launch_conv_wgrad<float, 2, 2>(s, a, slices);
}
}  // namespace luxhip
