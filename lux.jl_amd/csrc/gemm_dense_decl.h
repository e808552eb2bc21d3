// Declarations shared by gemm.hip (dispatch) and gemm_inst_*.hip (kernel instantiations).
#pragma once

#include "common.h"
#include "gemm_core.h"

namespace luxhip {

template <typename T>
struct DenseArgs {
    Operand<T> A, B;
    int M, N, K;
    T* C;
    int64_t ldc;
    const T* bias;   // per m, may be null
    T* pre;          // same layout as C, may be null
    int act;
    int tiles_m, tiles_n;
    // batched products: matrix b of each operand starts b * stride elements after the first (0: shared)
    int batch = 1;
    int64_t bsA = 0, bsB = 0, bsC = 0;
};

template <typename T, bool A_KMAJOR, bool B_KMAJOR>
int launch_layout(hipStream_t s, DenseArgs<T>& a);

template <typename T, bool A_KMAJOR, bool B_KMAJOR>
int launch_batched_layout(hipStream_t s, DenseArgs<T>& a);

}  // namespace luxhip
