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
    int c_vec = 0;   // C and pre allow 8-byte stores at every (m multiple of 4, n): aligned base, ldc a multiple of 4
    int tail = 0;    // this launch finishes the rows or columns of another one (profile name "...+tail")
    int c_f32 = 0;   // batched products of bf16 operands only: C points to fp32 values (same ldc and strides, in elements)
    // batched products only: the softmax rule as the epilogue (attention pullback).  ep_probs != null: with acc = the
    // cotangent of the weights, C = ep_scale * probs .* (acc - ep_d[column]); probs lies as C does (same ldc and
    // strides), ep_d holds one value per column of every product: product b's N values from ep_d + b * N on
    const T* ep_probs = nullptr;
    const float* ep_d = nullptr;
    float ep_scale = 0.0f;
    // batched products: the batch index runs over up to three nested dims (bdim[0] innermost); along
    // dim d the matrices of an operand lie stride[d] elements apart (0: one matrix shared by all)
    int batch = 1;
    int bdim[3] = {1, 1, 1};
    int64_t bsA[3] = {0, 0, 0}, bsB[3] = {0, 0, 0}, bsC[3] = {0, 0, 0};
    // batched products with a triangular operand or result (causal attention), see luxhip_batched_matmul_strided:
    // 0 none; 1 tiles of C with every m > n are left untouched; 2 op(B)[k, n] = 0 for k > n: the
    // contraction stops at the tile's last column; 3 op(B)[k, n] = 0 for k < n: it starts at the tile's first column
    int structure = 0;
};

template <typename T, bool A_KMAJOR, bool B_KMAJOR>
int launch_layout(hipStream_t s, DenseArgs<T>& a);

template <typename T, bool A_KMAJOR, bool B_KMAJOR>
int launch_batched_layout(hipStream_t s, DenseArgs<T>& a);

}  // namespace luxhip
