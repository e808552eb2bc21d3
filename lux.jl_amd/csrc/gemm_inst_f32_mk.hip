// Explicit instantiation: storage f32, A M-major, B K-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<float, false, true>(hipStream_t, DenseArgs<float>&);
template int launch_batched_layout<float, false, true>(hipStream_t, DenseArgs<float>&);
}
