// layernorm forward and pullback over an (L, R) view: each of the R columns (L contiguous
// elements) is normalised on its own; gamma/beta (optional) are indexed by the position l.
//
//   forward : one wave (L small) or one workgroup per column keeps the column in registers:
//             mean, variance about the mean and the normalised output from one HBM read.
//   pullback: ln_bwd_dx_kernel, same ownership, delta and x in registers:
//               g = gamma*dy, dx = invstd*(g - mean(g) - xhat*mean(g*xhat))
//             ln_param_grad_kernel: dgamma[l] = sum_r dy*xhat, dbeta[l] = sum_r dy as a column
//             reduction (threads along l, coalesced; R split into slices, partials combined
//             in a fixed order by ln_param_finalize_kernel).
//             ln_bwd_fused_kernel: both in one pass for columns that one wavefront holds.
#include <algorithm>

#include "common.h"

namespace luxhip {

constexpr int kLnCache = 8;   // vectors per thread kept in registers

template <typename T, int VEC>
__device__ __forceinline__ void ln_load(const T* p, size_t off, float (&v)[VEC]) {
    if constexpr (VEC == 1) v[0] = ld(p + off);
    else Vec<T>::load(p + off, v);
}
template <typename T, int VEC>
__device__ __forceinline__ void ln_store(T* p, size_t off, const float (&v)[VEC]) {
    if constexpr (VEC == 1) st(p + off, v[0]);
    else Vec<T>::store(p + off, v);
}

// Sum over the threads that share a column: the wave (WAVE) or the workgroup.
template <bool WAVE>
__device__ __forceinline__ float col_sum(float v, float* sm) {
    if constexpr (WAVE) return wave_sum(v);
    else return block_sum(v, sm);
}

// ------------------------------------------------------------------------------- forward
template <typename T, int ACT, int VEC, bool WAVE, bool CACHED>
__global__ __launch_bounds__(WAVE ? 256 : 1024) void ln_fwd_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta, T* y,
                              float* save_mean, float* save_invstd, uint32_t nvec, uint32_t R, float inv_L, float eps) {
    __shared__ float sm[16];
    const uint32_t tpc = WAVE ? 64u : blockDim.x;                       // threads per column
    const uint32_t t = WAVE ? (threadIdx.x & 63u) : threadIdx.x;
    const uint32_t r = WAVE ? blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6) : blockIdx.x;
    if (r >= R) return;                                                 // whole waves / workgroups only
    const size_t base = (size_t)r * nvec * VEC;
    using K = Kept<T, VEC>;
    typename K::type kv[CACHED ? kLnCache : 1];   // cached: the column; loads past its end re-read the last vector
    float v[1][VEC];
    float sum = 0.0f;
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) kv[u] = K::load(x, base + (size_t)min(u * tpc + t, nvec - 1) * VEC);
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const uint32_t q = u * tpc + t;
            if (q < nvec) {
                K::get(kv[u], v[0]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) sum += v[0][e];
            }
        }
    } else {
        for (uint32_t q = t; q < nvec; q += tpc) {
            ln_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) sum += v[0][e];
        }
    }
    const float mean = col_sum<WAVE>(sum, sm) * inv_L;
    float dev = 0.0f;
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const uint32_t q = u * tpc + t;
            if (q < nvec) {
                K::get(kv[u], v[0]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) dev = fmaf(v[0][e] - mean, v[0][e] - mean, dev);
            }
        }
    } else {
        for (uint32_t q = t; q < nvec; q += tpc) {
            ln_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) dev = fmaf(v[0][e] - mean, v[0][e] - mean, dev);
        }
    }
    const float var = col_sum<WAVE>(dev, sm) * inv_L;
    const float invstd = 1.0f / sqrtf(var + eps);
    if (t == 0) {
        if (save_mean) save_mean[r] = mean;
        if (save_invstd) save_invstd[r] = invstd;
    }
    auto emit = [&](uint32_t q, const float (&xv)[VEC]) {
        float gm[VEC], bt[VEC], o[VEC];
        if (gamma) {
            ln_load<T, VEC>(gamma, (size_t)q * VEC, gm);
            ln_load<T, VEC>(beta, (size_t)q * VEC, bt);
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float sc = (gamma ? gm[e] : 1.0f) * invstd;
            const float sh = fmaf(-mean, sc, gamma ? bt[e] : 0.0f);
            o[e] = Act<ACT>::f(fmaf(xv[e], sc, sh));
        }
        ln_store<T, VEC>(y, base + (size_t)q * VEC, o);
    };
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const uint32_t q = u * tpc + t;
            if (q < nvec) {
                K::get(kv[u], v[0]);
                emit(q, v[0]);
            }
        }
    } else {
        for (uint32_t q = t; q < nvec; q += tpc) {
            ln_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
            emit(q, v[0]);
        }
    }
}

// ------------------------------------------------------------------------------- pullback: dx
// dy for one vector, given the column statistics and the affine parameters at its positions.
template <typename T, int ACT, int VEC>
__device__ __forceinline__ void ln_dy(const T* gamma, const T* beta, uint32_t q, float mean, float invstd,
                                      const float (&dv)[VEC], const float (&xv)[VEC], float (&dy)[VEC],
                                      float (&gm)[VEC]) {
    float bt[VEC];
    if (gamma) {
        ln_load<T, VEC>(gamma, (size_t)q * VEC, gm);
        if constexpr (ACT != LUXHIP_ACT_IDENTITY) ln_load<T, VEC>(beta, (size_t)q * VEC, bt);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) { gm[e] = 1.0f; bt[e] = 0.0f; }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        dy[e] = dv[e];
        if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
            const float sc = gm[e] * invstd;
            const float pre = fmaf(xv[e], sc, fmaf(-mean, sc, bt[e]));
            dy[e] *= Act<ACT>::d(Act<ACT>::f(pre), pre);
        }
    }
}

// the same with the parameters already in registers
template <int ACT, int VEC>
__device__ __forceinline__ void ln_dy_regs(const float (&gm)[VEC], const float (&bt)[VEC], float mean, float invstd,
                                           const float (&dv)[VEC], const float (&xv)[VEC], float (&dy)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        dy[e] = dv[e];
        if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
            const float sc = gm[e] * invstd;
            const float pre = fmaf(xv[e], sc, fmaf(-mean, sc, bt[e]));
            dy[e] *= Act<ACT>::d(Act<ACT>::f(pre), pre);
        }
    }
}

template <typename T, int ACT, int VEC, bool WAVE, bool CACHED>
__global__ __launch_bounds__(WAVE ? 256 : 1024) void ln_bwd_dx_kernel(const T* __restrict__ delta, const T* __restrict__ x, const T* __restrict__ gamma,
                                 const T* __restrict__ beta, const float* __restrict__ save_mean,
                                 const float* __restrict__ save_invstd, T* dx, uint32_t nvec, uint32_t R, float inv_L) {
    __shared__ float sm[16];
    const uint32_t tpc = WAVE ? 64u : blockDim.x;
    const uint32_t t = WAVE ? (threadIdx.x & 63u) : threadIdx.x;
    const uint32_t r = WAVE ? blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6) : blockIdx.x;
    if (r >= R) return;
    const size_t base = (size_t)r * nvec * VEC;
    const float mean = save_mean[r], invstd = save_invstd[r];
    using K = Kept<T, VEC>;
    typename K::type kd[CACHED ? kLnCache : 1], kv[CACHED ? kLnCache : 1];
    float d[1][VEC], v[1][VEC];
    float s1 = 0.0f, s2 = 0.0f;
    auto accumulate = [&](uint32_t q, const float (&dv)[VEC], const float (&xv)[VEC]) {
        float dy[VEC], gm[VEC];
        ln_dy<T, ACT, VEC>(gamma, beta, q, mean, invstd, dv, xv, dy, gm);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float g = gm[e] * dy[e];
            s1 += g;
            s2 = fmaf(g, (xv[e] - mean) * invstd, s2);
        }
    };
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const size_t off = base + (size_t)min(u * tpc + t, nvec - 1) * VEC;   // past the end: re-read the last vector
            kd[u] = K::load(delta, off);
            kv[u] = K::load(x, off);
        }
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const uint32_t q = u * tpc + t;
            if (q < nvec) {
                K::get(kd[u], d[0]);
                K::get(kv[u], v[0]);
                accumulate(q, d[0], v[0]);
            }
        }
    } else {
        for (uint32_t q = t; q < nvec; q += tpc) {
            ln_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
            ln_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
            accumulate(q, d[0], v[0]);
        }
    }
    s1 = col_sum<WAVE>(s1, sm) * inv_L;
    s2 = col_sum<WAVE>(s2, sm) * inv_L;
    auto emit = [&](uint32_t q, const float (&dv)[VEC], const float (&xv)[VEC]) {
        float dy[VEC], gm[VEC], o[VEC];
        ln_dy<T, ACT, VEC>(gamma, beta, q, mean, invstd, dv, xv, dy, gm);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float xh = (xv[e] - mean) * invstd;
            o[e] = invstd * (gm[e] * dy[e] - s1 - xh * s2);
        }
        ln_store<T, VEC>(dx, base + (size_t)q * VEC, o);
    };
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kLnCache; ++u) {
            const uint32_t q = u * tpc + t;
            if (q < nvec) {
                K::get(kd[u], d[0]);
                K::get(kv[u], v[0]);
                emit(q, d[0], v[0]);
            }
        }
    } else {
        for (uint32_t q = t; q < nvec; q += tpc) {
            ln_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
            ln_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
            emit(q, d[0], v[0]);
        }
    }
}

// ------------------------------------------------------------------------------- pullback: dx, dgamma, dbeta in one pass
// Columns of up to 64 * kLnCache vectors with affine parameters.  Two wavefronts share a column
// (half of its vectors each, so that the per-position sums fit the register file next to the
// column itself); a pair walks over columns r = pair, pair + P, ... (P pairs in the grid) with
// delta and x of the current column in registers, as ln_bwd_dx_kernel does, and keeps dy * xhat
// and dy of its positions l summed over its columns.  The two pairs of a workgroup add their sums
// in pair order through LDS; row `blockIdx.x` of pg / pb receives the result and
// ln_param_finalize_kernel adds the rows in order.  delta and x are read once.
constexpr int kLnFusedCache = kLnCache / 2;
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(256) void ln_bwd_fused_kernel(const T* __restrict__ delta, const T* __restrict__ x,
                                                           const T* __restrict__ gamma, const T* __restrict__ beta,
                                                           const float* __restrict__ save_mean,
                                                           const float* __restrict__ save_invstd, T* dx, float* pg, float* pb,
                                                           uint32_t nvec, uint32_t R, float inv_L) {
    __shared__ float red[2][2][128 * VEC];
    __shared__ float colsum[2][2][2];                  // [pair][wave of the pair][s1, s2]
    const uint32_t w = threadIdx.x >> 6, pair = w >> 1, half = w & 1u;
    const uint32_t t = half * 64u + (threadIdx.x & 63u);          // 0..127 inside the pair
    const uint32_t pairs = gridDim.x * 2u;
    using K = Kept<T, VEC>;
    float ag[kLnFusedCache][VEC], ab[kLnFusedCache][VEC];
#pragma unroll
    for (int u = 0; u < kLnFusedCache; ++u)
#pragma unroll
        for (int e = 0; e < VEC; ++e) { ag[u][e] = 0.0f; ab[u][e] = 0.0f; }
    // The affine parameters at this thread's positions are the same for every column: read once and kept as they lie
    // in memory.  (Read inside the second pass they would sit between the dx stores, and a wave's memory operations
    // complete in the order of their issue: every such load would wait for the store before it.)
    typename K::type kgm[kLnFusedCache], kbt[kLnFusedCache];
    const bool affine = gamma != nullptr;
    if (affine) {
#pragma unroll
        for (int u = 0; u < kLnFusedCache; ++u) {
            const size_t off = (size_t)min(u * 128u + t, nvec - 1) * VEC;
            kgm[u] = K::load(gamma, off);
            if constexpr (ACT != LUXHIP_ACT_IDENTITY) kbt[u] = K::load(beta, off);
        }
    }
    auto params = [&](int u, float (&gm)[VEC], float (&bt)[VEC]) {
        if (affine) {
            K::get(kgm[u], gm);
            if constexpr (ACT != LUXHIP_ACT_IDENTITY) K::get(kbt[u], bt);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { gm[e] = 1.0f; bt[e] = 0.0f; }
        }
    };
    const uint32_t rounds = (R + pairs - 1) / pairs;              // the same for every wavefront: barriers inside
    for (uint32_t it = 0; it < rounds; ++it) {
        const uint32_t r = it * pairs + blockIdx.x * 2u + pair;
        const bool live = r < R;                                  // uniform per wavefront
        const uint32_t rc = live ? r : R - 1;
        const size_t base = (size_t)rc * nvec * VEC;
        const float mean = save_mean[rc], invstd = save_invstd[rc];
        typename K::type kd[kLnFusedCache], kv[kLnFusedCache];
#pragma unroll
        for (int u = 0; u < kLnFusedCache; ++u) {
            const size_t off = base + (size_t)min(u * 128u + t, nvec - 1) * VEC;   // past the end: the last vector again
            kd[u] = K::load(delta, off);
            kv[u] = K::load(x, off);
        }
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int u = 0; u < kLnFusedCache; ++u) {
            const uint32_t q = u * 128u + t;
            if (q < nvec && live) {
                float d[VEC], v[VEC], dy[VEC], gm[VEC], bt[VEC];
                K::get(kd[u], d);
                K::get(kv[u], v);
                params(u, gm, bt);
                ln_dy_regs<ACT, VEC>(gm, bt, mean, invstd, d, v, dy);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xh = (v[e] - mean) * invstd;
                    const float g = gm[e] * dy[e];
                    s1 += g;
                    s2 = fmaf(g, xh, s2);
                    ag[u][e] = fmaf(dy[e], xh, ag[u][e]);
                    ab[u][e] += dy[e];
                }
            }
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        if ((threadIdx.x & 63u) == 0) { colsum[pair][half][0] = s1; colsum[pair][half][1] = s2; }
        __syncthreads();
        s1 = (colsum[pair][0][0] + colsum[pair][1][0]) * inv_L;
        s2 = (colsum[pair][0][1] + colsum[pair][1][1]) * inv_L;
        __syncthreads();                                          // colsum is rewritten in the next round
#pragma unroll
        for (int u = 0; u < kLnFusedCache; ++u) {
            const uint32_t q = u * 128u + t;
            if (q < nvec && live) {
                float d[VEC], v[VEC], dy[VEC], gm[VEC], bt[VEC], o[VEC];
                K::get(kd[u], d);
                K::get(kv[u], v);
                params(u, gm, bt);
                ln_dy_regs<ACT, VEC>(gm, bt, mean, invstd, d, v, dy);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xh = (v[e] - mean) * invstd;
                    o[e] = invstd * (gm[e] * dy[e] - s1 - xh * s2);
                }
                ln_store<T, VEC>(dx, base + (size_t)q * VEC, o);
            }
        }
    }
    // sums of the two pairs, in pair order, one cached vector at a time
    const size_t row = (size_t)blockIdx.x * nvec * VEC;
#pragma unroll
    for (int u = 0; u < kLnFusedCache; ++u) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            red[0][pair][t * VEC + e] = ag[u][e];
            red[1][pair][t * VEC + e] = ab[u][e];
        }
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < 128u * VEC; i += 256u) {
            const uint32_t l = u * 128u * VEC + i;
            if (l < nvec * VEC) {
                pg[row + l] = red[0][0][i] + red[0][1][i];
                pb[row + l] = red[1][0][i] + red[1][1][i];
            }
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------- pullback: dgamma, dbeta
// grid (ceil(nvec / 64), S): a thread owns one vector of positions l and walks over the
// columns of slice s; partial sums go to pg/pb[s][l].
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(64) void ln_param_grad_kernel(const T* __restrict__ delta, const T* __restrict__ x,
                                                           const T* __restrict__ gamma, const T* __restrict__ beta,
                                                           const float* __restrict__ save_mean,
                                                           const float* __restrict__ save_invstd, float* pg, float* pb,
                                                           uint32_t nvec, uint32_t R, uint32_t cols_per_slice) {
    const uint32_t q = blockIdx.x * 64 + threadIdx.x;
    if (q >= nvec) return;
    const uint32_t r0 = blockIdx.y * cols_per_slice, r1 = min(r0 + cols_per_slice, R);
    float gm[VEC], bt[VEC], ag[VEC], ab[VEC];
    if (gamma) {
        ln_load<T, VEC>(gamma, (size_t)q * VEC, gm);
        ln_load<T, VEC>(beta, (size_t)q * VEC, bt);
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        ag[e] = 0.0f; ab[e] = 0.0f;
        if (!gamma) { gm[e] = 1.0f; bt[e] = 0.0f; }
    }
    const size_t stride = (size_t)nvec * VEC;
#pragma unroll 4
    for (uint32_t r = r0; r < r1; ++r) {
        float dv[VEC], xv[VEC];
        ln_load<T, VEC>(delta, r * stride + (size_t)q * VEC, dv);
        ln_load<T, VEC>(x, r * stride + (size_t)q * VEC, xv);
        const float mean = save_mean[r], invstd = save_invstd[r];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float dy = dv[e];
            if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                const float sc = gm[e] * invstd;
                const float pre = fmaf(xv[e], sc, fmaf(-mean, sc, bt[e]));
                dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
            }
            ag[e] = fmaf(dy, (xv[e] - mean) * invstd, ag[e]);
            ab[e] += dy;
        }
    }
    const size_t o = (size_t)blockIdx.y * stride + (size_t)q * VEC;
#pragma unroll
    for (int e = 0; e < VEC; ++e) { pg[o + e] = ag[e]; pb[o + e] = ab[e]; }
}

// dgamma[l] = sum_s pg[s][l], dbeta likewise.  Workgroup of LW positions x (1024 / LW) slice groups:
// group g adds slices g, g + G, ... and the G group sums are added in group order.  LW = 32 gives
// L / 32 workgroups (128-byte row segments): enough of them to fill the device for L of a few thousand.
constexpr int kLnFinalizeWidth = 32;
template <typename T>
__global__ __launch_bounds__(1024) void ln_param_finalize_kernel(const float* __restrict__ pg, const float* __restrict__ pb,
                                                                 T* dgamma, T* dbeta, uint32_t L, uint32_t S) {
    constexpr int LW = kLnFinalizeWidth, G = 1024 / LW;
    __shared__ float sg[G][LW], sb[G][LW];
    const uint32_t lx = threadIdx.x % LW, grp = threadIdx.x / LW;
    const uint32_t l = blockIdx.x * LW + lx;
    float tg = 0.0f, tb = 0.0f;
    if (l < L) {
        uint32_t s = grp;
        for (; s + 3 * G < S; s += 4 * G) {          // four independent loads in flight
            const float g0 = pg[(size_t)s * L + l], g1 = pg[(size_t)(s + G) * L + l];
            const float g2 = pg[(size_t)(s + 2 * G) * L + l], g3 = pg[(size_t)(s + 3 * G) * L + l];
            const float b0 = pb[(size_t)s * L + l], b1 = pb[(size_t)(s + G) * L + l];
            const float b2 = pb[(size_t)(s + 2 * G) * L + l], b3 = pb[(size_t)(s + 3 * G) * L + l];
            tg = (((tg + g0) + g1) + g2) + g3;
            tb = (((tb + b0) + b1) + b2) + b3;
        }
        for (; s < S; s += G) {
            tg += pg[(size_t)s * L + l];
            tb += pb[(size_t)s * L + l];
        }
    }
    sg[grp][lx] = tg;
    sb[grp][lx] = tb;
    __syncthreads();
    if (grp == 0 && l < L) {
        tg = 0.0f; tb = 0.0f;
#pragma unroll
        for (int g = 0; g < G; ++g) { tg += sg[g][lx]; tb += sb[g][lx]; }
        if (dgamma) st(dgamma + l, tg);
        if (dbeta) st(dbeta + l, tb);
    }
}

// ------------------------------------------------------------------------------- host side
struct LnPlan {
    bool vec, wave, cached;
    uint32_t nvec;
    unsigned threads, blocks;
};

template <typename T>
static LnPlan ln_plan(int64_t L, int64_t R, bool ptr_ok) {
    constexpr int V = Vec<T>::N;
    LnPlan p;
    p.vec = ptr_ok && L % V == 0;
    p.nvec = (uint32_t)(L / (p.vec ? V : 1));
    p.wave = p.nvec <= 64u * kLnCache;
    if (p.wave) {
        p.cached = true;
        p.threads = 256;                                   // 4 columns per workgroup
        p.blocks = (unsigned)ceil_div(R, 4);
    } else {
        int64_t t = 256;
        while (t < 1024 && t * kLnCache < p.nvec) t <<= 1;
        p.threads = (unsigned)t;
        p.cached = (int64_t)p.nvec <= t * kLnCache;
        p.blocks = (unsigned)R;
    }
    return p;
}

static int ln_check(int dtype, int act, int64_t L, int64_t R) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    LUX_INVALID_IF(L < 0 || R < 0, "negative dimension");
    if (L > 0 && R > 0) {
        const long double tot = (long double)L * (long double)R;
        LUX_UNSUPPORTED_IF(tot >= 2147483648.0L, "tensors of 2^31 or more elements are not supported");
    }
    return LUXHIP_OK;
}

#define LN_VARIANTS(KERNEL, A, ...)                                                                     \
    do {                                                                                                \
        if (p.vec && p.wave) launch_exact(ps, KERNEL<T, A, V, true, true>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);   \
        else if (p.vec && p.cached) launch_exact(ps, KERNEL<T, A, V, false, true>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);  \
        else if (p.vec) launch_exact(ps, KERNEL<T, A, V, false, false>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);      \
        else if (p.wave) launch_exact(ps, KERNEL<T, A, 1, true, true>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);       \
        else if (p.cached) launch_exact(ps, KERNEL<T, A, 1, false, true>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);    \
        else launch_exact(ps, KERNEL<T, A, 1, false, false>, dim3(p.blocks), dim3(p.threads), 0, s, __VA_ARGS__);                 \
    } while (0)

template <typename T>
static int ln_fwd_impl(hipStream_t s, int act, int64_t L, int64_t R, const T* x, const T* gamma, const T* beta, float eps,
                       T* y, float* save_mean, float* save_invstd) {
    constexpr int V = Vec<T>::N;
    const bool ptr_ok = aligned16(x) && aligned16(y) && (gamma == nullptr || (aligned16(gamma) && aligned16(beta)));
    LnPlan p = ln_plan<T>(L, R, ptr_ok);
    const float inv_L = 1.0f / (float)L;
    ProfScope ps("ln_fwd_kernel", s, true);
#define LN_FWD(A) LN_VARIANTS(ln_fwd_kernel, A, x, gamma, beta, y, save_mean, save_invstd, p.nvec, (uint32_t)R, inv_L, eps)
    LUX_DISPATCH_ACT(act, LN_FWD);
#undef LN_FWD
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
static int ln_bwd_impl(hipStream_t s, int act, int64_t L, int64_t R, const T* delta, const T* x, const T* gamma,
                       const T* beta, const float* save_mean, const float* save_invstd, T* dx, T* dgamma, T* dbeta) {
    constexpr int V = Vec<T>::N;
    const bool ptr_ok = aligned16(x) && aligned16(delta) && aligned16(dx) &&
                        (gamma == nullptr || (aligned16(gamma) && aligned16(beta)));
    LnPlan p = ln_plan<T>(L, R, ptr_ok);
    const float inv_L = 1.0f / (float)L;
    if (p.vec && p.wave && gamma != nullptr && (dgamma != nullptr || dbeta != nullptr) && R >= 64) {
        // one pass over delta and x: dx and the per-position sums of every workgroup
        const int64_t blocks = std::min<int64_t>(ceil_div(R, 2), 3 * (int64_t)(num_cus() > 0 ? num_cus() : 256));
        Workspace ws;
        int rc = get_workspace(s, (size_t)2 * blocks * L * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        float* pg = reinterpret_cast<float*>(ws.data);
        float* pb = pg + (size_t)blocks * L;
        {
            ProfScope ps("ln_bwd_fused_kernel", s, true);
#define LN_FUSED(A) launch_exact(ps, ln_bwd_fused_kernel<T, A, V>, dim3((unsigned)blocks), dim3(256), 0, s, delta, x, gamma, beta, save_mean, save_invstd, dx, pg, pb, p.nvec, (uint32_t)R, inv_L)
            LUX_DISPATCH_ACT(act, LN_FUSED);
#undef LN_FUSED
        }
        LUX_CHECK_LAUNCH();
        ProfScope ps2("ln_param_finalize_kernel", s);
        ln_param_finalize_kernel<T><<<(unsigned)ceil_div(L, kLnFinalizeWidth), 1024, 0, s>>>(pg, pb, dgamma, dbeta, (uint32_t)L, (uint32_t)blocks);
        LUX_CHECK_LAUNCH();
        return LUXHIP_OK;
    }
    {
        ProfScope ps("ln_bwd_dx_kernel", s, true);
#define LN_BWD(A) LN_VARIANTS(ln_bwd_dx_kernel, A, delta, x, gamma, beta, save_mean, save_invstd, dx, p.nvec, (uint32_t)R, inv_L)
        LUX_DISPATCH_ACT(act, LN_BWD);
#undef LN_BWD
    }
    LUX_CHECK_LAUNCH();
    if (gamma != nullptr && (dgamma != nullptr || dbeta != nullptr)) {
        const int64_t gx = ceil_div(p.nvec, 64);
        int64_t S = std::max<int64_t>(1, std::min<int64_t>(ceil_div(R, 16), ceil_div(2048, gx)));
        const uint32_t cols = (uint32_t)ceil_div(R, S);
        S = ceil_div(R, cols);
        LUX_UNSUPPORTED_IF(S > 65535, "layernorm_bwd: column split too large");
        Workspace ws;
        int rc = get_workspace(s, (size_t)2 * S * L * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        float* pg = reinterpret_cast<float*>(ws.data);
        float* pb = pg + (size_t)S * L;
        dim3 grid((unsigned)gx, (unsigned)S);
        {
            ProfScope ps("ln_param_grad_kernel", s);
#define LN_PG(A)                                                                                                           \
    do {                                                                                                                   \
        if (p.vec) ln_param_grad_kernel<T, A, V><<<grid, 64, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, pg, pb, p.nvec, (uint32_t)R, cols); \
        else ln_param_grad_kernel<T, A, 1><<<grid, 64, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, pg, pb, p.nvec, (uint32_t)R, cols);       \
    } while (0)
            LUX_DISPATCH_ACT(act, LN_PG);
#undef LN_PG
        }
        LUX_CHECK_LAUNCH();
        ProfScope ps2("ln_param_finalize_kernel", s);
        ln_param_finalize_kernel<T><<<(unsigned)ceil_div(L, kLnFinalizeWidth), 1024, 0, s>>>(pg, pb, dgamma, dbeta, (uint32_t)L, (uint32_t)S);
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_layernorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t L, int64_t R, const void* x, const void* gamma,
                         const void* beta, double eps, void* y, float* save_mean, float* save_invstd) {
    LUX_REQUIRE_INIT();
    int rc = ln_check(dtype, act, L, R);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "layernorm_fwd: gamma and beta must be given together");
    if (L * R == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || y == nullptr, "layernorm_fwd: x and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return ln_fwd_impl<float>((hipStream_t)s, act, L, R, (const float*)x, (const float*)gamma, (const float*)beta,
                                  (float)eps, (float*)y, save_mean, save_invstd);
    return ln_fwd_impl<bf16_t>((hipStream_t)s, act, L, R, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta,
                               (float)eps, (bf16_t*)y, save_mean, save_invstd);
}

int luxhip_layernorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t L, int64_t R, const void* delta, const void* x,
                         const void* gamma, const void* beta, const float* save_mean, const float* save_invstd, void* dx,
                         void* dgamma, void* dbeta) {
    LUX_REQUIRE_INIT();
    int rc = ln_check(dtype, act, L, R);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "layernorm_bwd: gamma and beta must be given together");
    if (L * R == 0) {
        if (L > 0 && dgamma) { rc = luxhip_fill_zero(dgamma, (size_t)L * (dtype == LUXHIP_F32 ? 4 : 2), s); if (rc) return rc; }
        if (L > 0 && dbeta) { rc = luxhip_fill_zero(dbeta, (size_t)L * (dtype == LUXHIP_F32 ? 4 : 2), s); if (rc) return rc; }
        return LUXHIP_OK;
    }
    LUX_INVALID_IF(delta == nullptr || x == nullptr || dx == nullptr || save_mean == nullptr || save_invstd == nullptr,
                   "layernorm_bwd: delta, x, dx, save_mean and save_invstd must not be NULL");
    if (dtype == LUXHIP_F32)
        return ln_bwd_impl<float>((hipStream_t)s, act, L, R, (const float*)delta, (const float*)x, (const float*)gamma,
                                  (const float*)beta, save_mean, save_invstd, (float*)dx, (float*)dgamma, (float*)dbeta);
    return ln_bwd_impl<bf16_t>((hipStream_t)s, act, L, R, (const bf16_t*)delta, (const bf16_t*)x, (const bf16_t*)gamma,
                               (const bf16_t*)beta, save_mean, save_invstd, (bf16_t*)dx, (bf16_t*)dgamma, (bf16_t*)dbeta);
}

}  // extern "C"
