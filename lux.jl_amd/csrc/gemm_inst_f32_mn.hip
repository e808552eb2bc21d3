// Explicit instantiation: storage f32, A M-major, B N-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<float, false, false>(hipStream_t, DenseArgs<float>&);
template int launch_batched_layout<float, false, false>(hipStream_t, DenseArgs<float>&);
}
