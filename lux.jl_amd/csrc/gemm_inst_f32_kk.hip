// Explicit instantiation: storage f32, A K-major, B K-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<float, true, true>(hipStream_t, DenseArgs<float>&);
template int launch_batched_layout<float, true, true>(hipStream_t, DenseArgs<float>&);
}
