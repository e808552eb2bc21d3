// batchnorm forward (statistics + running-stat update + normalise/activate) and the complete
// pullback, as HBM-bound streaming kernels over the (I, C, N) view.
//
// Channel c owns the rows (n*C + c)*I .. +I for every n.  Reduction kernels use a (S, C)
// grid: workgroup (s, c) streams a contiguous slice of channel c's I*N elements and writes one
// partial; a one-wave-per-channel finalize kernel combines the S partials in a fixed order
// (deterministic, no floating-point atomics, no device-wide fences inside the streaming
// kernels: an agent-scope fence per workgroup writes back the L2 and costs far more than the
// extra launch) and writes the per-channel results.
//
//   forward, training : bn_stats_kernel (read x) -> partials
//                       bn_stats_finalize_kernel -> mean, invstd, scale, shift, running stats
//                       bn_apply_kernel  (read x, write y)
//   forward, inference: bn_infer_prep_kernel (C threads) -> scale, shift
//                       bn_apply_kernel
//   pullback          : bn_bwd_reduce_kernel (read delta, x) -> partials
//                       bn_bwd_finalize_kernel -> dgamma, dbeta, per-channel coefficients
//                       bn_bwd_apply_kernel  (read delta, x, write dx)
#include <algorithm>

#include "common.h"

namespace luxhip {

constexpr int kBnThreads = 256;
constexpr int kBnUnroll = 1;  // one 16-byte vector per thread and a huge grid streams fastest on MI355X

struct ChanGeom {
    uint32_t nq;           // vectors per channel = I*N / VEC
    uint32_t chunk;        // vectors per workgroup slice
    uint32_t vec_per_row;  // I / VEC
    uint32_t C;
    FastDiv rowdiv;        // / vec_per_row
    __device__ __forceinline__ size_t offset(uint32_t q, uint32_t c, int vec) const {
        const uint32_t n = rowdiv.div(q);
        return ((size_t)q + (size_t)vec_per_row * ((size_t)n * (C - 1) + c)) * vec;
    }
};

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T* p, size_t off, float (&v)[VEC]) {
    if constexpr (VEC == 1) v[0] = ld(p + off);
    else Vec<T>::load(p + off, v);
}
template <typename T, int VEC>
__device__ __forceinline__ void store_vecn(T* p, size_t off, const float (&v)[VEC]) {
    if constexpr (VEC == 1) st(p + off, v[0]);
    else Vec<T>::store(p + off, v);
}

// Chan et al. pairwise combination of (count, mean, M2).
__device__ __forceinline__ void chan_merge(float& n, float& mean, float& m2, float nb, float meanb, float m2b) {
    const float nn = n + nb;
    if (nn == 0.0f) return;
    const float delta = meanb - mean;
    const float f = nb / nn;
    mean += delta * f;
    m2 += m2b + delta * delta * n * f;
    n = nn;
}

// ------------------------------------------------------------------------------- statistics
// Partial (count, mean, M2) of slice s of channel c -> partial[(c*S + s)*3 ..].  A workgroup
// keeps its slice (up to kStatVecs vectors per thread) in registers and makes two passes over
// the registers: workgroup mean, then the sum of squared deviations from it (exact two-pass
// statistics per slice; slices are combined with Chan's formula by the finalize kernel).
constexpr int kStatVecs = 4;
template <typename T, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_stats_kernel(const T* __restrict__ x, float* partial, ChanGeom g) {
    __shared__ float sm[kBnThreads / 64];
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const uint32_t q0 = s * g.chunk, q1 = min(q0 + g.chunk, g.nq);
    const float cnt = (float)((q1 - q0) * VEC);
    float n = 0.0f, mean = 0.0f, m2 = 0.0f;   // running (count, mean, M2) over the passes of the outer loop
    for (uint32_t base = q0; base < q1; base += kBnThreads * kStatVecs) {
        float v[kStatVecs][VEC];
        bool ok[kStatVecs];
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < kStatVecs; ++u) {
            const uint32_t q = base + u * kBnThreads + threadIdx.x;
            ok[u] = q < q1;
            if (ok[u]) load_vec<T, VEC>(x, g.offset(q, c, VEC), v[u]);
        }
#pragma unroll
        for (int u = 0; u < kStatVecs; ++u)
            if (ok[u]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) sum += v[u][k];
            }
        const uint32_t nvec = min(q1 - base, (uint32_t)(kBnThreads * kStatVecs));
        const float nb = (float)(nvec * VEC);
        const float mb = block_sum(sum, sm) / nb;
        float dev = 0.0f;
#pragma unroll
        for (int u = 0; u < kStatVecs; ++u)
            if (ok[u]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) dev = fmaf(v[u][k] - mb, v[u][k] - mb, dev);
            }
        const float m2b = block_sum(dev, sm);
        chan_merge(n, mean, m2, nb, mb, m2b);
    }
    (void)cnt;
    if (threadIdx.x == 0) {
        float* p = partial + ((size_t)c * S + s) * 3;
        p[0] = n; p[1] = mean; p[2] = m2;
    }
}

// One wave per channel merges the S partials (fixed tree order) and writes every per-channel
// result of the forward pass.  S <= kBnThreads.
template <typename T>
__global__ __launch_bounds__(kWave) void bn_stats_finalize_kernel(
    const float* __restrict__ partial, uint32_t S, const T* __restrict__ gamma, const T* __restrict__ beta,
    const T* __restrict__ rmean, const T* __restrict__ rvar, T* rmean_out, T* rvar_out, float* save_mean,
    float* save_invstd, float* scale, float* shift, float count, float momentum, float eps) {
    const uint32_t c = blockIdx.x;
    const float* p = partial + (size_t)c * S * 3;
    float n = 0.0f, mean = 0.0f, m2 = 0.0f;
    for (uint32_t i = threadIdx.x; i < S; i += kWave) chan_merge(n, mean, m2, p[3 * i], p[3 * i + 1], p[3 * i + 2]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float nb = __shfl_xor(n, off, kWave), mb = __shfl_xor(mean, off, kWave), qb = __shfl_xor(m2, off, kWave);
        chan_merge(n, mean, m2, nb, mb, qb);
    }
    if (threadIdx.x == 0) {
        const float var = m2 / count;
        const float invstd = 1.0f / sqrtf(var + eps);
        const float gm = gamma ? ld(gamma + c) : 1.0f;
        const float bt = beta ? ld(beta + c) : 0.0f;
        const float sc = gm * invstd;
        scale[c] = sc;
        shift[c] = fmaf(-mean, sc, bt);
        if (save_mean) save_mean[c] = mean;
        if (save_invstd) save_invstd[c] = invstd;
        if (rmean_out) {
            const float m1 = momentum, m3 = 1.0f - momentum;
            const float m2c = momentum * count / (count - 1.0f);
            st(rmean_out + c, m3 * ld(rmean + c) + m1 * mean);
            st(rvar_out + c, m3 * ld(rvar + c) + m2c * var);
        }
    }
}

template <typename T>
__global__ void bn_infer_prep_kernel(const T* __restrict__ gamma, const T* __restrict__ beta,
                                     const T* __restrict__ rmean, const T* __restrict__ rvar, float* save_mean,
                                     float* save_invstd, float* scale, float* shift, uint32_t C, float eps) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const float mean = ld(rmean + c), var = ld(rvar + c);
    const float invstd = 1.0f / sqrtf(var + eps);
    const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
    scale[c] = sc;
    shift[c] = fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
    if (save_mean) save_mean[c] = mean;
    if (save_invstd) save_invstd[c] = invstd;
}

// ------------------------------------------------------------------------------- normalise
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_apply_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                              const float* __restrict__ shift, T* y,
                                                              uint32_t total_vec, FastDiv rowdiv, FastDiv cdiv,
                                                              uint32_t C) {
    for (uint32_t base = blockIdx.x * (kBnThreads * kBnUnroll); base < total_vec;
         base += gridDim.x * (kBnThreads * kBnUnroll)) {
        float v[kBnUnroll][VEC];
        uint32_t idx[kBnUnroll];
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) {
            idx[u] = base + u * kBnThreads + threadIdx.x;
            if (idx[u] < total_vec) load_vec<T, VEC>(x, (size_t)idx[u] * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) {
            if (idx[u] < total_vec) {
                const uint32_t row = rowdiv.div(idx[u]);
                const uint32_t c = row - cdiv.div(row) * C;
                const float sc = scale[c], sh = shift[c];
                float o[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) o[k] = Act<ACT>::f(fmaf(v[u][k], sc, sh));
                store_vecn<T, VEC>(y, (size_t)idx[u] * VEC, o);
            }
        }
    }
}

// ------------------------------------------------------------------------------- pullback
// Partials of s1 = sum dy and s2 = sum dy * (x - mean) * invstd, dy = delta * act'(recomputed).
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_reduce_kernel(
    const T* __restrict__ delta, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
    const float* __restrict__ save_mean, const float* __restrict__ save_invstd, float* partial, ChanGeom g) {
    __shared__ float sm[kBnThreads / 64];
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const uint32_t q0 = s * g.chunk, q1 = min(q0 + g.chunk, g.nq);
    const float mean = save_mean[c], invstd = save_invstd[c];
    const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
    const float sh = fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
    float s1 = 0.0f, s2 = 0.0f;
    for (uint32_t base = q0; base < q1; base += kBnThreads * kStatVecs) {
        float d[kStatVecs][VEC], v[kStatVecs][VEC];
        bool ok[kStatVecs];
#pragma unroll
        for (int u = 0; u < kStatVecs; ++u) {
            const uint32_t q = base + u * kBnThreads + threadIdx.x;
            ok[u] = q < q1;
            if (ok[u]) {
                const size_t off = g.offset(q, c, VEC);
                load_vec<T, VEC>(delta, off, d[u]);
                load_vec<T, VEC>(x, off, v[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kStatVecs; ++u)
            if (ok[u]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float dy = d[u][k];
                    if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                        const float pre = fmaf(v[u][k], sc, sh);
                        dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
                    }
                    s1 += dy;
                    s2 = fmaf(dy, (v[u][k] - mean) * invstd, s2);
                }
            }
    }
    s1 = block_sum(s1, sm);
    s2 = block_sum(s2, sm);
    if (threadIdx.x == 0) {
        partial[((size_t)c * S + s) * 2] = s1;
        partial[((size_t)c * S + s) * 2 + 1] = s2;
    }
}

// One wave per channel: dgamma, dbeta and the coefficients of dx = A*dy + B*(x - mean) + D.
template <typename T>
__global__ __launch_bounds__(kWave) void bn_bwd_finalize_kernel(const float* __restrict__ partial, uint32_t S,
                                                                const T* __restrict__ gamma,
                                                                const float* __restrict__ save_invstd, T* dgamma,
                                                                T* dbeta, float* coef, uint32_t C, float inv_count,
                                                                int stats_from_batch) {
    const uint32_t c = blockIdx.x;
    const float* p = partial + (size_t)c * S * 2;
    float t1 = 0.0f, t2 = 0.0f;
    for (uint32_t i = threadIdx.x; i < S; i += kWave) { t1 += p[2 * i]; t2 += p[2 * i + 1]; }
    t1 = wave_sum(t1);
    t2 = wave_sum(t2);
    if (threadIdx.x == 0) {
        const float invstd = save_invstd[c];
        const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
        if (dgamma) st(dgamma + c, t2);
        if (dbeta) st(dbeta + c, t1);
        coef[c] = sc;
        coef[C + c] = stats_from_batch ? -sc * invstd * t2 * inv_count : 0.0f;
        coef[2 * C + c] = stats_from_batch ? -sc * t1 * inv_count : 0.0f;
    }
}

template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_apply_kernel(const T* __restrict__ delta, const T* __restrict__ x,
                                                                  const T* __restrict__ beta,
                                                                  const float* __restrict__ save_mean,
                                                                  const float* __restrict__ coef, T* dx,
                                                                  uint32_t total_vec, FastDiv rowdiv, FastDiv cdiv,
                                                                  uint32_t C) {
    for (uint32_t base = blockIdx.x * (kBnThreads * kBnUnroll); base < total_vec;
         base += gridDim.x * (kBnThreads * kBnUnroll)) {
        float d[kBnUnroll][VEC], v[kBnUnroll][VEC];
        uint32_t idx[kBnUnroll];
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) {
            idx[u] = base + u * kBnThreads + threadIdx.x;
            if (idx[u] < total_vec) {
                load_vec<T, VEC>(delta, (size_t)idx[u] * VEC, d[u]);
                load_vec<T, VEC>(x, (size_t)idx[u] * VEC, v[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u) {
            if (idx[u] < total_vec) {
                const uint32_t row = rowdiv.div(idx[u]);
                const uint32_t c = row - cdiv.div(row) * C;
                const float A = coef[c], B = coef[C + c], D = coef[2 * C + c], mean = save_mean[c];
                float sh = 0.0f;
                if constexpr (ACT != LUXHIP_ACT_IDENTITY) sh = fmaf(-mean, A, beta ? ld(beta + c) : 0.0f);
                float o[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float dy = d[u][k];
                    if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                        const float pre = fmaf(v[u][k], A, sh);
                        dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
                    }
                    o[k] = fmaf(A, dy, fmaf(B, v[u][k] - mean, D));
                }
                store_vecn<T, VEC>(dx, (size_t)idx[u] * VEC, o);
            }
        }
    }
}

// ------------------------------------------------------------------------------- host side
static ChanGeom make_geom(int64_t I, int64_t C, int64_t N, int vec, int64_t* S_out) {
    ChanGeom g;
    g.nq = (uint32_t)(I * N / vec);
    g.vec_per_row = (uint32_t)(I / vec);
    g.C = (uint32_t)C;
    g.rowdiv = FastDiv(g.vec_per_row);
    // kStatVecs vectors per thread where possible (amortises the workgroup reduction), at most
    // 256 slices per channel and about 16K workgroups in all
    int64_t S = ceil_div(g.nq, kBnThreads * kStatVecs);
    const int64_t smax = std::min<int64_t>(256, std::max<int64_t>(1, 16384 / C));
    S = std::max<int64_t>(1, std::min(S, smax));
    g.chunk = (uint32_t)ceil_div(g.nq, S);
    *S_out = ceil_div(g.nq, g.chunk);
    return g;
}

static int bn_check(int dtype, int act, int64_t I, int64_t C, int64_t N) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    LUX_INVALID_IF(I < 0 || C < 0 || N < 0, "negative dimension");
    if (I > 0 && C > 0 && N > 0) {
        const long double tot = (long double)I * (long double)C * (long double)N;
        LUX_UNSUPPORTED_IF(tot >= 2147483648.0L, "tensors of 2^31 or more elements are not supported");
    }
    LUX_UNSUPPORTED_IF(C > 65535, "more than 65535 channels are not supported");
    return LUXHIP_OK;
}

static inline unsigned flat_grid(uint32_t total_vec) { return (unsigned)ceil_div(total_vec, kBnThreads * kBnUnroll); }

template <typename T>
static int bn_fwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t N, const T* x, const T* gamma,
                       const T* beta, const T* rmean, const T* rvar, int training, float momentum, float eps, T* y,
                       T* rmean_out, T* rvar_out, float* save_mean, float* save_invstd) {
    constexpr int V = Vec<T>::N;
    const bool vec = aligned16(x) && aligned16(y) && I % V == 0;
    const int vv = vec ? V : 1;
    const bool batch_stats = training || rmean == nullptr;
    int64_t S = 1;
    ChanGeom g = make_geom(I, C, N, vv, &S);
    Workspace ws;
    int rc = get_workspace(s, (size_t)C * (2 + 3 * S) * sizeof(float), &ws);  // scale, shift, partials
    if (rc != LUXHIP_OK) return rc;
    float* scale = reinterpret_cast<float*>(ws.data);
    float* shift = scale + C;
    float* partial = shift + C;
    if (batch_stats) {
        const bool upd = training && rmean != nullptr;
        dim3 grid((unsigned)S, (unsigned)C);
        {
            ProfScope ps("bn_stats_kernel", s);
            if (vec) bn_stats_kernel<T, V><<<grid, kBnThreads, 0, s>>>(x, partial, g);
            else bn_stats_kernel<T, 1><<<grid, kBnThreads, 0, s>>>(x, partial, g);
        }
        LUX_CHECK_LAUNCH();
        ProfScope ps("bn_stats_finalize_kernel", s);
        bn_stats_finalize_kernel<T><<<(unsigned)C, kWave, 0, s>>>(partial, (uint32_t)S, gamma, beta, rmean, rvar,
                                                                 upd ? rmean_out : nullptr, upd ? rvar_out : nullptr,
                                                                 save_mean, save_invstd, scale, shift, (float)(I * N),
                                                                 momentum, eps);
    } else {
        ProfScope ps("bn_infer_prep_kernel", s);
        bn_infer_prep_kernel<T><<<(unsigned)ceil_div(C, 256), 256, 0, s>>>(gamma, beta, rmean, rvar, save_mean,
                                                                           save_invstd, scale, shift, (uint32_t)C, eps);
    }
    LUX_CHECK_LAUNCH();
    const uint32_t tv = (uint32_t)(I * C * N / vv);
    const FastDiv rowdiv((uint32_t)(I / vv)), cdiv((uint32_t)C);
#define LAUNCH_APPLY(A)                                                                                             \
    do {                                                                                                            \
        if (vec) bn_apply_kernel<T, A, V><<<flat_grid(tv), kBnThreads, 0, s>>>(x, scale, shift, y, tv, rowdiv, cdiv, (uint32_t)C); \
        else bn_apply_kernel<T, A, 1><<<flat_grid(tv), kBnThreads, 0, s>>>(x, scale, shift, y, tv, rowdiv, cdiv, (uint32_t)C);     \
    } while (0)
    {
        ProfScope ps("bn_apply_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_APPLY);
    }
#undef LAUNCH_APPLY
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
static int bn_bwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t N, const T* delta, const T* x,
                       const T* gamma, const T* beta, const float* save_mean, const float* save_invstd,
                       int stats_from_batch, T* dx, T* dgamma, T* dbeta) {
    constexpr int V = Vec<T>::N;
    const bool vec = aligned16(x) && aligned16(delta) && aligned16(dx) && I % V == 0;
    const int vv = vec ? V : 1;
    int64_t S = 1;
    ChanGeom g = make_geom(I, C, N, vv, &S);
    Workspace ws;
    int rc = get_workspace(s, (size_t)C * (3 + 2 * S) * sizeof(float), &ws);
    if (rc != LUXHIP_OK) return rc;
    float* coef = reinterpret_cast<float*>(ws.data);
    float* partial = coef + 3 * C;
    const float inv_count = 1.0f / (float)(I * N);
    dim3 grid((unsigned)S, (unsigned)C);
    const uint32_t tv = (uint32_t)(I * C * N / vv);
    const FastDiv rowdiv((uint32_t)(I / vv)), cdiv((uint32_t)C);
#define LAUNCH_REDUCE(A)                                                                                            \
    do {                                                                                                            \
        if (vec) bn_bwd_reduce_kernel<T, A, V><<<grid, kBnThreads, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, partial, g); \
        else bn_bwd_reduce_kernel<T, A, 1><<<grid, kBnThreads, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, partial, g);     \
    } while (0)
#define LAUNCH_BWD_APPLY(A)                                                                                         \
    do {                                                                                                            \
        if (vec) bn_bwd_apply_kernel<T, A, V><<<flat_grid(tv), kBnThreads, 0, s>>>(delta, x, beta, save_mean, coef, dx, tv, rowdiv, cdiv, (uint32_t)C); \
        else bn_bwd_apply_kernel<T, A, 1><<<flat_grid(tv), kBnThreads, 0, s>>>(delta, x, beta, save_mean, coef, dx, tv, rowdiv, cdiv, (uint32_t)C);     \
    } while (0)
    {
        ProfScope ps("bn_bwd_reduce_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_REDUCE);
    }
    LUX_CHECK_LAUNCH();
    {
        ProfScope ps("bn_bwd_finalize_kernel", s);
        bn_bwd_finalize_kernel<T><<<(unsigned)C, kWave, 0, s>>>(partial, (uint32_t)S, gamma, save_invstd, dgamma, dbeta, coef,
                                                               (uint32_t)C, inv_count, stats_from_batch);
    }
    LUX_CHECK_LAUNCH();
    {
        ProfScope ps("bn_bwd_apply_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_BWD_APPLY);
    }
#undef LAUNCH_REDUCE
#undef LAUNCH_BWD_APPLY
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_batchnorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* x,
                         const void* gamma, const void* beta, const void* rmean, const void* rvar, int training,
                         double momentum, double eps, void* y, void* rmean_out, void* rvar_out, float* save_mean,
                         float* save_invstd) {
    LUX_REQUIRE_INIT();
    int rc = bn_check(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "batchnorm_fwd: gamma and beta must be given together");
    LUX_INVALID_IF((rmean == nullptr) != (rvar == nullptr), "batchnorm_fwd: running mean and variance must be given together");
    LUX_INVALID_IF(training && rmean != nullptr && (rmean_out == nullptr || rvar_out == nullptr),
                   "batchnorm_fwd: training with running statistics needs rmean_out and rvar_out");
    if (I * C * N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || y == nullptr, "batchnorm_fwd: x and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return bn_fwd_impl<float>((hipStream_t)s, act, I, C, N, (const float*)x, (const float*)gamma, (const float*)beta,
                                  (const float*)rmean, (const float*)rvar, training, (float)momentum, (float)eps,
                                  (float*)y, (float*)rmean_out, (float*)rvar_out, save_mean, save_invstd);
    return bn_fwd_impl<bf16_t>((hipStream_t)s, act, I, C, N, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta,
                               (const bf16_t*)rmean, (const bf16_t*)rvar, training, (float)momentum, (float)eps,
                               (bf16_t*)y, (bf16_t*)rmean_out, (bf16_t*)rvar_out, save_mean, save_invstd);
}

int luxhip_batchnorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* delta,
                         const void* x, const void* gamma, const void* beta, const float* save_mean,
                         const float* save_invstd, int stats_from_batch, void* dx, void* dgamma, void* dbeta) {
    LUX_REQUIRE_INIT();
    int rc = bn_check(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "batchnorm_bwd: gamma and beta must be given together");
    if (I * C * N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(delta == nullptr || x == nullptr || dx == nullptr || save_mean == nullptr || save_invstd == nullptr,
                   "batchnorm_bwd: delta, x, dx, save_mean and save_invstd must not be NULL");
    if (dtype == LUXHIP_F32)
        return bn_bwd_impl<float>((hipStream_t)s, act, I, C, N, (const float*)delta, (const float*)x, (const float*)gamma,
                                  (const float*)beta, save_mean, save_invstd, stats_from_batch, (float*)dx,
                                  (float*)dgamma, (float*)dbeta);
    return bn_bwd_impl<bf16_t>((hipStream_t)s, act, I, C, N, (const bf16_t*)delta, (const bf16_t*)x, (const bf16_t*)gamma,
                               (const bf16_t*)beta, save_mean, save_invstd, stats_from_batch, (bf16_t*)dx,
                               (bf16_t*)dgamma, (bf16_t*)dbeta);
}

}  // extern "C"
