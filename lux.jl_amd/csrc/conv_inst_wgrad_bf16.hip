// wgrad implicit-GEMM kernels, storage type bf16: tile selection + instantiation.
#include "conv_kernels.h"
namespace luxhip {
template <>
int launch_conv_wgrad_any<bf16_t>(hipStream_t s, ConvWgradArgs<bf16_t>& a, int slices, bool small) {
    if (small) return launch_conv_wgrad<bf16_t, 1, 1>(s, a, slices);
    return launch_conv_wgrad<bf16_t, 2, 2>(s, a, slices);
}
}  // namespace luxhip
