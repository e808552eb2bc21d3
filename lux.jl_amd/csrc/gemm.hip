// Dense layer entry points: matmul / matmuladd, fused_dense forward and pullback, on the MFMA
// mainloop of gemm_core.h with a fused bias + activation (+ pre-activation) epilogue.
#include <stdlib.h>

#include <algorithm>

#include "common.h"
#include "gemm_dense_decl.h"

namespace luxhip {

int bias_act_bwd_dispatch(hipStream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* delta,
                          const void* out, const void* pre, void* dx, void* dbias);   // elementwise.hip

int transpose_matrix_bf16(hipStream_t s, const bf16_t* in, bf16_t* out, int64_t P, int64_t C);   // conv.hip
int dense_dz_transposed(hipStream_t s, int act, int64_t M, int64_t N, const bf16_t* delta, const bf16_t* out, const bf16_t* pre,
                        bf16_t* dz, bf16_t* dzT, float* partial, bf16_t* dbias);                 // elementwise.hip

int gemm_tile_override() { return (int)option_gemm_tile(); }
static inline size_t align256(size_t b) { return (b + 255) & ~size_t(255); }
// The 256 x 256 bf16 kernel reads K-major operands from LDS at twice the rate of M/N-major ones
// (plain 16-byte reads against transposing reads): 1090-1190 TFLOP/s against 800-950 measured on
// 4096..11008-sized problems.  A large M/N-major operand is therefore copied into the K-major
// layout first (a pass at HBM rate: 90 MB in ~37 us, against ~200 us saved), when the other
// dimension is long enough for the copy to pay (threshold from those measurements).
template <typename T>
static bool pretranspose_pays(int64_t M, int64_t N, int64_t K, int64_t other, int64_t ld, int64_t rows, const T* p) {
    if constexpr (sizeof(T) != 2) return false;
    return option_gemm_pretranspose() != 0 && gemm_tile_override() == 0 && M % 256 == 0 && N % 256 == 0 && K % 32 == 0 &&
           (M / 256) * (N / 256) >= 128 && K >= 1024 && other >= 4096 && ld == rows && aligned16(p);
}

// ws_front: bytes at the start of the stream's workspace that the caller is using (operand copies go behind them)
template <typename T>
static int gemm_impl(hipStream_t s, int transA, int transB, int64_t M, int64_t N, int64_t K, const T* A, int64_t lda,
                     const T* B, int64_t ldb, const T* bias, T* C, int64_t ldc, T* pre, int act, size_t ws_front = 0) {
    DenseArgs<T> a;
    bool a_kmajor = transA != 0, b_kmajor = transB == 0;
    if constexpr (sizeof(T) == 2) {
        bool ta = !a_kmajor && pretranspose_pays<T>(M, N, K, N, lda, M, A);
        bool tb = !b_kmajor && pretranspose_pays<T>(M, N, K, M, ldb, N, B);
        // only the kernel with both operands K-major is faster (a mixed pair is not), and two copies
        // need a longer K to pay than one (measured: 4096 x 4096 x 1024 loses, x 4096 wins)
        if (!((a_kmajor || ta) && (b_kmajor || tb)) || (ta && tb && K < 2048)) ta = tb = false;
        if (ta || tb) {
            const size_t ab = ta ? (((size_t)M * K * sizeof(T) + 255) & ~size_t(255)) : 0;
            const size_t bb = tb ? (size_t)N * K * sizeof(T) : 0;
            Workspace ws;
            int rc = get_workspace(s, ws_front + ab + bb, &ws);
            if (rc != LUXHIP_OK) return rc;
            ws.data += ws_front;
            if (ta) {
                T* At = reinterpret_cast<T*>(ws.data);
                if ((rc = transpose_matrix_bf16(s, A, At, M, K)) != LUXHIP_OK) return rc;
                A = At; lda = K; a_kmajor = true;
            }
            if (tb) {
                T* Bt = reinterpret_cast<T*>(ws.data + ab);
                if ((rc = transpose_matrix_bf16(s, B, Bt, N, K)) != LUXHIP_OK) return rc;
                B = Bt; ldb = K; b_kmajor = true;
            }
        }
    }
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
    a.c_vec = (reinterpret_cast<uintptr_t>(C) & 7u) == 0 && (reinterpret_cast<uintptr_t>(pre) & 7u) == 0 && ldc % 4 == 0;
    if (a_kmajor && b_kmajor) return launch_layout<T, true, true>(s, a);
    if (a_kmajor) return launch_layout<T, true, false>(s, a);
    if (b_kmajor) return launch_layout<T, false, true>(s, a);
    return launch_layout<T, false, false>(s, a);
}

// C_b = op(A_b) op(B_b) over up to three nested batch dims; a stride of 0 shares one matrix
template <typename T>
static int batched_impl(hipStream_t s, int transA, int transB, int64_t M, int64_t N, int64_t K, const int64_t* bdim, const T* A,
                        int64_t lda, const int64_t* sA, const T* B, int64_t ldb, const int64_t* sB, T* C, int64_t ldc,
                        const int64_t* sC, int structure, int c_f32 = 0, const T* ep_probs = nullptr, const float* ep_d = nullptr,
                        float ep_scale = 0.0f) {
    DenseArgs<T> a;
    a.structure = structure;
    a.c_f32 = c_f32;
    a.ep_probs = ep_probs;
    a.ep_d = ep_d;
    a.ep_scale = ep_scale;
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
    a.batch = 1;
    for (int d = 0; d < 3; ++d) {
        a.bdim[d] = (int)bdim[d];
        a.batch *= (int)bdim[d];
        a.bsA[d] = sA[d]; a.bsB[d] = sB[d]; a.bsC[d] = sC[d];
        a.A.vec_ok = a.A.vec_ok && (sA[d] * sizeof(T)) % 16 == 0;
        a.B.vec_ok = a.B.vec_ok && (sB[d] * sizeof(T)) % 16 == 0;
    }
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.C = C; a.ldc = ldc; a.bias = nullptr; a.pre = nullptr; a.act = LUXHIP_ACT_IDENTITY;
    a.c_vec = (reinterpret_cast<uintptr_t>(C) & 7u) == 0 && ldc % 4 == 0 && sC[0] % 4 == 0 && sC[1] % 4 == 0 && sC[2] % 4 == 0;
    if (a_kmajor && b_kmajor) return launch_batched_layout<T, true, true>(s, a);
    if (a_kmajor) return launch_batched_layout<T, true, false>(s, a);
    if (b_kmajor) return launch_batched_layout<T, false, true>(s, a);
    return launch_batched_layout<T, false, false>(s, a);
}

static int batched_dispatch(hipStream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                            const int64_t* bdim, const void* A, int64_t lda, const int64_t* sA, const void* B, int64_t ldb,
                            const int64_t* sB, void* C, int64_t ldc, const int64_t* sC, int structure) {
    LUX_INVALID_IF(structure < 0 || structure > 3, "batched_matmul: structure must be 0..3");
    int64_t batch = 1;
    for (int d = 0; d < 3; ++d) {
        LUX_INVALID_IF(bdim[d] < 0 || sA[d] < 0 || sB[d] < 0 || sC[d] < 0, "batched_matmul: negative batch extent or stride");
        batch *= bdim[d];
        LUX_UNSUPPORTED_IF(batch >= (1ll << 31), "batched_matmul: batch of 2^31 or more");
    }
    if (M == 0 || N == 0 || batch == 0) return LUXHIP_OK;
    LUX_INVALID_IF(C == nullptr, "batched_matmul: C must not be NULL");
    LUX_INVALID_IF(K > 0 && (A == nullptr || B == nullptr), "batched_matmul: A and B must not be NULL");
    LUX_INVALID_IF(lda < (transA ? K : M) || ldb < (transB ? N : K) || ldc < M, "batched_matmul: leading dimension too small");
    if (dtype == LUXHIP_F32)
        return batched_impl<float>(s, transA, transB, M, N, K, bdim, (const float*)A, lda, sA, (const float*)B, ldb, sB, (float*)C,
                                   ldc, sC, structure);
    return batched_impl<bf16_t>(s, transA, transB, M, N, K, bdim, (const bf16_t*)A, lda, sA, (const bf16_t*)B, ldb, sB,
                                (bf16_t*)C, ldc, sC, structure, dtype == LUXHIP_BF16_WIDE ? 1 : 0);
}

// out[i] = sum_b in[i + b n]: `sum(tmp; dims=3)` of a stack of matrices, accumulated in fp32 in batch order
template <typename T, int VEC>
__global__ __launch_bounds__(256) void batch_sum_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t n, int batch,
                                                        int64_t first, int64_t nvec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        const int64_t e = first + i * VEC;
        float acc[VEC] = {};
        for (int b = 0; b < batch; ++b) {
            float v[VEC];
            if constexpr (VEC == 1) v[0] = ld(in + e + (int64_t)b * n);
            else Vec<T>::load(in + e + (int64_t)b * n, v);
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] += v[k];
        }
        if constexpr (VEC == 1) st(out + e, acc[0]);
        else Vec<T>::store(out + e, acc);
    }
}

template <typename T>
static int batch_sum_impl(hipStream_t s, int64_t n, int64_t batch, const T* in, T* out) {
    constexpr int V = Vec<T>::N;
    const bool vec = aligned16(in) && aligned16(out) && (n * sizeof(T)) % 16 == 0;
    const int64_t nvec = vec ? n / V : 0;
    ProfScope ps("batch_sum_kernel", s);
    const unsigned cap = (unsigned)(num_cus() > 0 ? num_cus() : 256) * 16;
    if (nvec > 0) {
        batch_sum_kernel<T, V><<<std::min((unsigned)ceil_div(nvec, 256), cap), 256, 0, s>>>(in, out, n, (int)batch, 0, nvec);
        LUX_CHECK_LAUNCH();
    }
    if (nvec * V < n) {
        const int64_t rest = n - nvec * V;
        batch_sum_kernel<T, 1><<<std::min((unsigned)ceil_div(rest, 256), cap), 256, 0, s>>>(in, out, n, (int)batch, nvec * V, rest);
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

// d[b * N + n] = sum_e dO[e, n] O[e, n] of product b (both E x N with leading dimension ldo and the given batch strides):
// one wavefront per column, fp32.  This is sum_s probs[s, n] dprobs[s, n], the inner product that the softmax rule needs,
// without the cotangent of the weights -- exactly so only for the unrounded O = V probs, which is why bf16 storage
// hands O over in fp32 (TO = float): an O rounded to bf16 shifts a whole column of the result by probs times the
// rounding error.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void attn_rowdot_kernel(const T* __restrict__ dO, const TO* __restrict__ O, float* __restrict__ d, int E,
                                                          int N, int64_t ldo, int bd0, int bd1, int64_t s0, int64_t s1, int64_t s2,
                                                          int64_t cols) {
    const int64_t col = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (col >= cols) return;
    const int lane = threadIdx.x & 63;
    const int64_t b = col / N;
    const int n = (int)(col - b * N);
    const int i0 = (int)(b % bd0), i1 = (int)((b / bd0) % bd1);
    const int64_t i2 = b / ((int64_t)bd0 * bd1);
    const int64_t off = i0 * s0 + i1 * s1 + i2 * s2 + (int64_t)n * ldo;
    float acc = 0.0f;
    for (int e = lane; e < E; e += 64) acc = fmaf(ld(dO + off + e), ld(O + off + e), acc);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) acc += __shfl_xor(acc, o);
    if (lane == 0) d[col] = acc;
}
// Columns whose length, leading dimension and strides are multiples of 4 elements (aligned accordingly): sixteen lanes per
// column (four columns per wave), four consecutive elements per lane and trip, so that a wave's loads are 8- or 16-byte
// vectors that cover whole cache lines of four columns.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void attn_rowdot_quad_kernel(const T* __restrict__ dO, const TO* __restrict__ O, float* __restrict__ d, int E,
                                                               int N, int64_t ldo, int bd0, int bd1, int64_t s0, int64_t s1, int64_t s2,
                                                               int64_t cols) {
    const int64_t col = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int sub = threadIdx.x & 15;
    float acc = 0.0f;
    if (col < cols) {
        const int64_t b = col / N;
        const int n = (int)(col - b * N);
        const int i0 = (int)(b % bd0), i1 = (int)((b / bd0) % bd1);
        const int64_t i2 = b / ((int64_t)bd0 * bd1);
        const int64_t off = i0 * s0 + i1 * s1 + i2 * s2 + (int64_t)n * ldo;
        for (int e = sub * 4; e < E; e += 64) {
            float a[4], o[4];
            if constexpr (sizeof(T) == 2) {
                const uint2 w = *reinterpret_cast<const uint2*>(dO + off + e);
                a[0] = __uint_as_float(w.x << 16); a[1] = __uint_as_float(w.x & 0xffff0000u);
                a[2] = __uint_as_float(w.y << 16); a[3] = __uint_as_float(w.y & 0xffff0000u);
            } else {
                const float4 w = *reinterpret_cast<const float4*>(dO + off + e);
                a[0] = w.x; a[1] = w.y; a[2] = w.z; a[3] = w.w;
            }
            if constexpr (sizeof(TO) == 2) {
                const uint2 w = *reinterpret_cast<const uint2*>(O + off + e);
                o[0] = __uint_as_float(w.x << 16); o[1] = __uint_as_float(w.x & 0xffff0000u);
                o[2] = __uint_as_float(w.y << 16); o[3] = __uint_as_float(w.y & 0xffff0000u);
            } else {
                const float4 w = *reinterpret_cast<const float4*>(O + off + e);
                o[0] = w.x; o[1] = w.y; o[2] = w.z; o[3] = w.w;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = fmaf(a[i], o[i], acc);
        }
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) acc += __shfl_xor(acc, o);      // within the sixteen lanes of a column
    if (sub == 0 && col < cols) d[col] = acc;
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
                         int act, size_t ws_front = 0) {
    if (M == 0 || N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(C == nullptr, "matmul: C must not be NULL");
    LUX_INVALID_IF(K > 0 && (A == nullptr || B == nullptr), "matmul: A and B must not be NULL");
    LUX_INVALID_IF(lda < (transA ? K : M) || ldb < (transB ? N : K) || ldc < M, "matmul: leading dimension too small");
    if (dtype == LUXHIP_F32)
        return gemm_impl<float>(s, transA, transB, M, N, K, (const float*)A, lda, (const float*)B, ldb, (const float*)bias,
                                (float*)C, ldc, (float*)pre, act);
    return gemm_impl<bf16_t>(s, transA, transB, M, N, K, (const bf16_t*)A, lda, (const bf16_t*)B, ldb, (const bf16_t*)bias,
                             (bf16_t*)C, ldc, (bf16_t*)pre, act, ws_front);
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

int luxhip_batched_matmul(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                          int64_t batch, const void* A, int64_t lda, int64_t strideA, const void* B, int64_t ldb,
                          int64_t strideB, void* C, int64_t ldc, int64_t strideC) {
    LUX_REQUIRE_INIT();
    int rc = gemm_check(dtype, 0, M, N, K);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF(batch > 1 && M > 0 && N > 0 && strideC < ldc * (N - 1) + M, "batched_matmul: the results would overlap");
    const int64_t bdim[3] = {batch, 1, 1}, sA[3] = {strideA, 0, 0}, sB[3] = {strideB, 0, 0}, sC[3] = {strideC, 0, 0};
    return batched_dispatch((hipStream_t)s, dtype, transA, transB, M, N, K, bdim, A, lda, sA, B, ldb, sB, C, ldc, sC, 0);
}

int luxhip_batched_matmul_strided(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                                  const int64_t* batch_dims, const void* A, int64_t lda, const int64_t* stridesA, const void* B,
                                  int64_t ldb, const int64_t* stridesB, void* C, int64_t ldc, const int64_t* stridesC,
                                  int structure) {
    LUX_REQUIRE_INIT();
    int rc = gemm_check(dtype == LUXHIP_BF16_WIDE ? LUXHIP_BF16 : dtype, 0, M, N, K);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF(batch_dims == nullptr || stridesA == nullptr || stridesB == nullptr || stridesC == nullptr,
                   "batched_matmul_strided: batch extents and strides must not be NULL");
    return batched_dispatch((hipStream_t)s, dtype, transA, transB, M, N, K, batch_dims, A, lda, stridesA, B, ldb, stridesB, C, ldc,
                            stridesC, structure);
}

int luxhip_attention_weights_pullback(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t Ev, const int64_t* batch_dims,
                                      const void* v, int64_t ldv, const int64_t* strides_v, const void* d_out, const void* out,
                                      int64_t ldo, const int64_t* strides_o, const void* probs, double scale, void* dlogits,
                                      int64_t ldc, const int64_t* strides_c, int structure) {
    LUX_REQUIRE_INIT();
    const bool wide = dtype == LUXHIP_BF16_WIDE;
    if (wide) dtype = LUXHIP_BF16;
    int rc = gemm_check(dtype, 0, S, L, Ev);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF(batch_dims == nullptr || strides_v == nullptr || strides_o == nullptr || strides_c == nullptr,
                   "attention_weights_pullback: batch extents and strides must not be NULL");
    LUX_INVALID_IF(structure != 0 && structure != 1, "attention_weights_pullback: structure must be 0 or 1");
    int64_t batch = 1;
    for (int d = 0; d < 3; ++d) {
        LUX_INVALID_IF(batch_dims[d] < 0 || strides_v[d] < 0 || strides_o[d] < 0 || strides_c[d] < 0,
                       "attention_weights_pullback: negative batch extent or stride");
        batch *= batch_dims[d];
        LUX_UNSUPPORTED_IF(batch >= (1ll << 31), "attention_weights_pullback: batch of 2^31 or more");
    }
    if (S == 0 || L == 0 || batch == 0) return LUXHIP_OK;
    LUX_INVALID_IF(v == nullptr || d_out == nullptr || out == nullptr || probs == nullptr || dlogits == nullptr,
                   "attention_weights_pullback: null operand");
    LUX_INVALID_IF(ldv < Ev || ldo < Ev || ldc < S, "attention_weights_pullback: leading dimension too small");
    const int64_t cols = batch * L;
    Workspace ws;
    rc = get_workspace((hipStream_t)s, (size_t)cols * sizeof(float), &ws);
    if (rc != LUXHIP_OK) return rc;
    float* d = reinterpret_cast<float*>(ws.data);
    {
        ProfScope ps("attn_rowdot_kernel", (hipStream_t)s);
        const int b0 = (int)batch_dims[0], b1 = (int)batch_dims[1];
        const int64_t* so = strides_o;
        const size_t eo = dtype == LUXHIP_F32 || wide ? 4 : 2, ed = dtype == LUXHIP_F32 ? 4 : 2;      // element sizes of out and d_out
        const bool quad = Ev % 4 == 0 && ldo % 4 == 0 && so[0] % 4 == 0 && so[1] % 4 == 0 && so[2] % 4 == 0 &&
                          reinterpret_cast<uintptr_t>(d_out) % (4 * ed) == 0 && reinterpret_cast<uintptr_t>(out) % (4 * eo) == 0;
        const unsigned grid = (unsigned)ceil_div(cols, quad ? 16 : 4);
#define ROWDOT(T, TO)                                                                                                                   \
    do {                                                                                                                                \
        if (quad) attn_rowdot_quad_kernel<T, TO><<<grid, 256, 0, (hipStream_t)s>>>((const T*)d_out, (const TO*)out, d, (int)Ev, (int)L, ldo, \
                                                                                   b0, b1, so[0], so[1], so[2], cols);                  \
        else attn_rowdot_kernel<T, TO><<<grid, 256, 0, (hipStream_t)s>>>((const T*)d_out, (const TO*)out, d, (int)Ev, (int)L, ldo, b0, b1, \
                                                                         so[0], so[1], so[2], cols);                                   \
    } while (0)
        if (dtype == LUXHIP_F32) ROWDOT(float, float);
        else if (wide) ROWDOT(bf16_t, float);
        else ROWDOT(bf16_t, bf16_t);
#undef ROWDOT
        LUX_CHECK_LAUNCH();
    }
    // dprobs (S x L) = v' (S x Ev) * d_out (Ev x L), with the softmax rule as its epilogue
    if (dtype == LUXHIP_F32)
        return batched_impl<float>((hipStream_t)s, 1, 0, S, L, Ev, batch_dims, (const float*)v, ldv, strides_v, (const float*)d_out, ldo,
                                   strides_o, (float*)dlogits, ldc, strides_c, structure, 0, (const float*)probs, d, (float)scale);
    return batched_impl<bf16_t>((hipStream_t)s, 1, 0, S, L, Ev, batch_dims, (const bf16_t*)v, ldv, strides_v, (const bf16_t*)d_out, ldo,
                                strides_o, (bf16_t*)dlogits, ldc, strides_c, structure, 0, (const bf16_t*)probs, d, (float)scale);
}

int luxhip_batch_sum(luxhip_stream_t s, int dtype, int64_t n, int64_t batch, const void* in, void* out) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(n < 0 || batch < 1, "batch_sum: invalid extent");
    LUX_UNSUPPORTED_IF(batch >= (1ll << 31), "batch_sum: batch of 2^31 or more");
    if (n == 0) return LUXHIP_OK;
    LUX_INVALID_IF(in == nullptr || out == nullptr, "batch_sum: in and out must not be NULL");
    if (dtype == LUXHIP_F32) return batch_sum_impl<float>((hipStream_t)s, n, batch, (const float*)in, (float*)out);
    return batch_sum_impl<bf16_t>((hipStream_t)s, n, batch, (const bf16_t*)in, (bf16_t*)out);
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
    // Large bf16 layers: the weight-gradient product reads dz along n, so it would copy dz into that layout first
    // (pretranspose_pays); the pass that computes dz writes that copy as well, and the bias gradient's partial sums,
    // instead of a pass for dz / dbias followed by a transposing copy.
    const int64_t ldxe = std::max<int64_t>(ldx, 1);
    const bool dz_both = dtype == LUXHIP_BF16 && dW != nullptr && M % 64 == 0 && N % 64 == 0 && N / 64 <= 65535 && N >= 2048 &&
                         pretranspose_pays<bf16_t>(M, K, N, K, M, M, (const bf16_t*)delta) &&
                         pretranspose_pays<bf16_t>(M, K, N, M, ldxe, K, (const bf16_t*)x) && aligned16(y) && aligned16(pre) &&
                         aligned16(dz) && M * N < (int64_t(1) << 31);
    if (dz_both) {
        const size_t tb = align256((size_t)M * N * 2), pb = dbias != nullptr ? align256((size_t)(N / 64) * M * sizeof(float)) : 0;
        const size_t xb = align256((size_t)K * N * 2);          // the product's own copy of x, behind ours
        Workspace ws;
        rc = get_workspace((hipStream_t)s, tb + pb + xb, &ws);
        if (rc != LUXHIP_OK) return rc;
        bf16_t* dzT = reinterpret_cast<bf16_t*>(ws.data);
        void* dz_out = act == LUXHIP_ACT_IDENTITY ? nullptr : dz;
        rc = dense_dz_transposed((hipStream_t)s, act, M, N, (const bf16_t*)delta, (const bf16_t*)y, (const bf16_t*)pre, (bf16_t*)dz_out,
                                 dzT, reinterpret_cast<float*>(ws.data + tb), (bf16_t*)dbias);
        if (rc != LUXHIP_OK) return rc;
        if (dz_out) dzp = dz_out;
        // dW (M x K) = dz (M x N) * x' (N x K) with dz given as its transpose (N contiguous)
        rc = gemm_dispatch((hipStream_t)s, dtype, 1, 1, M, K, N, dzT, N, x, ldx, nullptr, dW, std::max<int64_t>(M, 1), nullptr,
                           LUXHIP_ACT_IDENTITY, tb + pb);
        if (rc != LUXHIP_OK) return rc;
    } else {
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
    }
    if (dx != nullptr) {   // dx (K x N) = W' (K x M) * dz (M x N);  W is stored M x K
        rc = gemm_dispatch((hipStream_t)s, dtype, 1, 0, K, N, M, W, ldw, dzp, std::max<int64_t>(M, 1), nullptr, dx,
                           std::max<int64_t>(K, 1), nullptr, LUXHIP_ACT_IDENTITY);
        if (rc != LUXHIP_OK) return rc;
    }
    return LUXHIP_OK;
}

}  // extern "C"
