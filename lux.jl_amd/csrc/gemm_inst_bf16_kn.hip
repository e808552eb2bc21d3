// Explicit instantiation: storage bf16, A K-major, B N-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<bf16_t, true, false>(hipStream_t, DenseArgs<bf16_t>&);
template int launch_batched_layout<bf16_t, true, false>(hipStream_t, DenseArgs<bf16_t>&);
}
