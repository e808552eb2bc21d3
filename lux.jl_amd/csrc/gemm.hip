// Dense layer entry points: matmul / matmuladd, fused_dense forward and pullback, on the MFMA
// mainloop of gemm_core.h with a fused bias + activation (+ pre-activation) epilogue.
#include <stdlib.h>

#include <algorithm>

#include "common.h"
#include "gemm_dense_decl.h"

namespace luxhip {

int bias_act_bwd_dispatch(hipStream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* delta,
                          const void* out, const void* pre, void* dx, void* dbias);   // elementwise.hip

int gemm_tile_override() { return (int)option_gemm_tile(); }

template <typename T>
static int gemm_impl(hipStream_t s, int transA, int transB, int64_t M, int64_t N, int64_t K, const T* A, int64_t lda,
                     const T* B, int64_t ldb, const T* bias, T* C, int64_t ldc, T* pre, int act) {
    DenseArgs<T> a;
    const bool a_kmajor = transA != 0, b_kmajor = transB == 0;
    a.A.p = A;
    a.A.sr = a_kmajor ? lda : 1;
    a.A.sk = a_kmajor ? 1 : lda;
    a.A.rows = (int)M;
    a.A.vec_ok = aligned16(A) && (lda * sizeof(T)) % 16 == 0;
    a.B.p = B;
    a.B.sr = b_kmajor ? ldb : 1;
    a.B.sk = b_kmajor ? 1 : ldb;
    a.B.rows = (int)N;
    a.B.vec_ok = aligned16(B) && (ldb * sizeof(T)) % 16 == 0;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.C = C; a.ldc = ldc; a.bias = bias; a.pre = pre; a.act = act;
    if (a_kmajor && b_kmajor) return launch_layout<T, true, true>(s, a);
    if (a_kmajor) return launch_layout<T, true, false>(s, a);
    if (b_kmajor) return launch_layout<T, false, true>(s, a);
    return launch_layout<T, false, false>(s, a);
}

static int gemm_check(int dtype, int act, int64_t M, int64_t N, int64_t K) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    LUX_INVALID_IF(M < 0 || N < 0 || K < 0, "negative dimension");
    LUX_UNSUPPORTED_IF(M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31), "dimension of 2^31 or more");
    return LUXHIP_OK;
}

static int gemm_dispatch(hipStream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K, const void* A,
                         int64_t lda, const void* B, int64_t ldb, const void* bias, void* C, int64_t ldc, void* pre,
                         int act) {
    if (M == 0 || N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(C == nullptr, "matmul: C must not be NULL");
    LUX_INVALID_IF(K > 0 && (A == nullptr || B == nullptr), "matmul: A and B must not be NULL");
    LUX_INVALID_IF(lda < (transA ? K : M) || ldb < (transB ? N : K) || ldc < M, "matmul: leading dimension too small");
    if (dtype == LUXHIP_F32)
        return gemm_impl<float>(s, transA, transB, M, N, K, (const float*)A, lda, (const float*)B, ldb, (const float*)bias,
                                (float*)C, ldc, (float*)pre, act);
    return gemm_impl<bf16_t>(s, transA, transB, M, N, K, (const bf16_t*)A, lda, (const bf16_t*)B, ldb, (const bf16_t*)bias,
                             (bf16_t*)C, ldc, (bf16_t*)pre, act);
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_matmul(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K, const void* A,
                  int64_t lda, const void* B, int64_t ldb, const void* bias, void* C, int64_t ldc) {
    LUX_REQUIRE_INIT();
    int rc = gemm_check(dtype, 0, M, N, K);
    if (rc != LUXHIP_OK) return rc;
    return gemm_dispatch((hipStream_t)s, dtype, transA, transB, M, N, K, A, lda, B, ldb, bias, C, ldc, nullptr,
                         LUXHIP_ACT_IDENTITY);
}

int luxhip_fused_dense_fwd(luxhip_stream_t s, int dtype, int act, int64_t M, int64_t K, int64_t N, const void* W,
                           int64_t ldw, const void* x, int64_t ldx, const void* bias, void* y, int64_t ldy, void* pre) {
    LUX_REQUIRE_INIT();
    int rc = gemm_check(dtype, act, M, N, K);
    if (rc != LUXHIP_OK) return rc;
    return gemm_dispatch((hipStream_t)s, dtype, 0, 0, M, N, K, W, ldw, x, ldx, bias, y, ldy, pre, act);
}

int luxhip_fused_dense_bwd(luxhip_stream_t s, int dtype, int act, int64_t M, int64_t K, int64_t N, const void* delta,
                           const void* y, const void* pre, const void* W, int64_t ldw, const void* x, int64_t ldx,
                           void* dz, void* dW, void* dx, void* dbias) {
    LUX_REQUIRE_INIT();
    int rc = gemm_check(dtype, act, M, N, K);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF(M * N > 0 && delta == nullptr, "fused_dense_bwd: delta must not be NULL");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && M * N > 0 && dz == nullptr, "fused_dense_bwd: dz scratch is required");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && !act_needs_pre(act) && y == nullptr, "fused_dense_bwd: activation %d needs y", act);
    LUX_INVALID_IF(act_needs_pre(act) && pre == nullptr, "fused_dense_bwd: activation %d needs the pre-activation", act);
    const void* dzp = delta;
    if (act != LUXHIP_ACT_IDENTITY || dbias != nullptr) {
        // dz = delta .* act'(y, pre) and dbias = sum over the batch, one pass (dense layout: I = 1)
        void* dz_out = act == LUXHIP_ACT_IDENTITY ? nullptr : dz;
        rc = bias_act_bwd_dispatch((hipStream_t)s, dtype, act, 1, M, N, delta, y, pre, dz_out, dbias);
        if (rc != LUXHIP_OK) return rc;
        if (dz_out) dzp = dz_out;
    }
    if (dW != nullptr) {   // dW (M x K) = dz (M x N) * x' (N x K);  x is stored K x N
        rc = gemm_dispatch((hipStream_t)s, dtype, 0, 1, M, K, N, dzp, std::max<int64_t>(M, 1), x, ldx, nullptr, dW,
                           std::max<int64_t>(M, 1), nullptr, LUXHIP_ACT_IDENTITY);
        if (rc != LUXHIP_OK) return rc;
    }
    if (dx != nullptr) {   // dx (K x N) = W' (K x M) * dz (M x N);  W is stored M x K
        rc = gemm_dispatch((hipStream_t)s, dtype, 1, 0, K, N, M, W, ldw, dzp, std::max<int64_t>(M, 1), nullptr, dx,
                           std::max<int64_t>(K, 1), nullptr, LUXHIP_ACT_IDENTITY);
        if (rc != LUXHIP_OK) return rc;
    }
    return LUXHIP_OK;
}

}  // extern "C"
