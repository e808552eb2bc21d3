// Explicit instantiation: storage bf16, A M-major, B K-major.
#include "gemm_dense.h"
namespace luxhip {
template int launch_layout<bf16_t, false, true>(hipStream_t, DenseArgs<bf16_t>&);
template int launch_batched_layout<bf16_t, false, true>(hipStream_t, DenseArgs<bf16_t>&);
}
