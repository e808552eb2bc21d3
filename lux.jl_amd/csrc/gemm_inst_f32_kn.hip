// Explicit instantiation: storage f32, A K-major, B N-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<float, true, false>(hipStream_t, DenseArgs<float>&);
template int launch_batched_layout<float, true, false>(hipStream_t, DenseArgs<float>&);
}
