// Explicit instantiation: storage bf16, A K-major, B K-major; and the 256 x 256 kernel of gemm_kk256.h.
#include "gemm_dense.h"
#include "gemm_kk256.h"
namespace luxhip {
bool launch_kk256_if_applicable(hipStream_t s, DenseArgs<bf16_t>& a, int* rc) {
    if (!kk256::applicable(a)) return false;
    *rc = kk256::launch(s, a);
    return true;
}
template int launch_layout<bf16_t, true, true>(hipStream_t, DenseArgs<bf16_t>&);
template int launch_batched_layout<bf16_t, true, true>(hipStream_t, DenseArgs<bf16_t>&);
}
