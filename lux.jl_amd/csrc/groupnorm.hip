// groupnorm forward and pullback.
//
// x is viewed as (I, C/G, G, N): the slice of group k and sample n is the contiguous run of
// m = I*C/G elements at ((n*G + k)*C/G)*I.  One workgroup owns one slice.
//   * cached kernels keep the slice (forward: x; pullback: delta and x) in registers, so HBM
//     sees every tensor once: statistics, normalisation and the input gradient all come from
//     the registers (slices of up to kGnCache vectors per thread x 1024 threads);
//   * a slice too long for a 512-thread workgroup is split between two of them (each owns whole
//     channels); the halves exchange their partial statistics as (value, epoch) words, with a
//     bounded wait after which a workgroup recomputes its peer's share from global memory;
//   * streaming kernels handle still larger slices with a second read of the slice.
// Per-channel gradients (dgamma, dbeta) are accumulated per wave in LDS in program order,
// combined across waves in a fixed order, published as [N][C] partials and added over N, in
// sample order, by the workgroup of each group that arrives last: deterministic, no
// floating-point atomics, no extra launch.
#include <algorithm>

#include "common.h"

namespace luxhip {

constexpr int kGnCache = 8;  // vectors per thread kept in registers

struct GnGeom {
    uint32_t I, Cg, G, C;
    uint32_t nvec;         // vectors per slice = I*Cg / VEC
    uint32_t parts, pvec;  // workgroups per slice (cached kernels; 1 otherwise) and vectors per part = nvec / parts
    FastDiv chdiv;         // vector index -> channel within group: / (I / VEC)   (VEC == 1: / I)
    float inv_m;           // 1 / (I*Cg)
};

template <typename T, int VEC>
__device__ __forceinline__ void gn_load(const T* p, size_t off, float (&v)[VEC]) {
    if constexpr (VEC == 1) v[0] = ld(p + off);
    else Vec<T>::load(p + off, v);
}
template <typename T, int VEC>
__device__ __forceinline__ void gn_store(T* p, size_t off, const float (&v)[VEC]) {
    if constexpr (VEC == 1) st(p + off, v[0]);
    else Vec<T>::store(p + off, v);
}

// ------------------------------------------------------------------------------- forward
// Exchange area of the split kernels: `epoch`-tagged words, K per part, parts of a slice adjacent.
struct GnExchange {
    uint64_t* words;
    uint32_t epoch, spin_limit;
};

// instancenorm's running statistics, updated by the forward kernel itself (G == C: slice = n*C + c): the
// workgroup of a channel that arrives last averages the channel's N slice statistics, in sample order.
// out_mean == nullptr: no update.
template <typename T>
struct InRunning {
    const T* rmean;
    const T* rvar;
    T* out_mean;
    T* out_var;
    uint32_t* counters;
    float* var;                    // (C, N) words of workspace: the slice variances themselves (1/invstd^2 - eps would
                                   // cancel for channels whose variance is far below eps)
    uint32_t cstride, N;
    float momentum, corrected;     // corrected = momentum * I / (I - 1)
};

template <typename T, int ACT, int VEC, bool CACHED>
__global__ void gn_fwd_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta, T* y,
                              float* save_mean, float* save_invstd, GnGeom g, float eps, InRunning<T> rs) {
    __shared__ float sm[16];
    __shared__ uint32_t last_flag;
    const uint32_t slice = blockIdx.x;              // = n*G + k
    const uint32_t k = slice % g.G;
    const size_t base = (size_t)slice * g.nvec * VEC;
    const uint32_t T_ = blockDim.x;
    using K = Kept<T, VEC>;
    typename K::type kv[CACHED ? kGnCache : 1];   // cached: the slice as it lies in memory; loads past its end re-read the last vector
    float v[1][VEC];

    // pass 1: mean
    float sum = 0.0f;
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) kv[u] = K::load(x, base + (size_t)min(u * T_ + threadIdx.x, g.nvec - 1) * VEC);
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            const uint32_t q = u * T_ + threadIdx.x;
            if (q < g.nvec) {
                K::get(kv[u], v[0]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) sum += v[0][e];
            }
        }
    } else {
        for (uint32_t q = threadIdx.x; q < g.nvec; q += T_) {
            gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) sum += v[0][e];
        }
    }
    const float mean = block_sum(sum, sm) * g.inv_m;
    // pass 2: variance about the mean
    float dev = 0.0f;
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            const uint32_t q = u * T_ + threadIdx.x;
            if (q < g.nvec) {
                K::get(kv[u], v[0]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) dev = fmaf(v[0][e] - mean, v[0][e] - mean, dev);
            }
        }
    } else {
        for (uint32_t q = threadIdx.x; q < g.nvec; q += T_) {
            gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) dev = fmaf(v[0][e] - mean, v[0][e] - mean, dev);
        }
    }
    const float var = block_sum(dev, sm) * g.inv_m;
    const float invstd = 1.0f / sqrtf(var + eps);
    if (rs.out_mean != nullptr) {                     // uniform over the grid
        if (threadIdx.x == 0) {
            publish(reinterpret_cast<uint32_t*>(save_mean + slice), __float_as_uint(mean));
            publish(reinterpret_cast<uint32_t*>(save_invstd + slice), __float_as_uint(invstd));
            publish(reinterpret_cast<uint32_t*>(rs.var + slice), __float_as_uint(var));
            publish_done();
        }
        if (arrive_last(rs.counters + (size_t)k * rs.cstride, rs.N, &last_flag)) {
            float tm = 0.0f, tv = 0.0f;
            for (uint32_t n = threadIdx.x; n < rs.N; n += T_) {
                tm += __uint_as_float(fetch(reinterpret_cast<const uint32_t*>(save_mean + k + (size_t)g.G * n)));
                tv += __uint_as_float(fetch(reinterpret_cast<const uint32_t*>(rs.var + k + (size_t)g.G * n)));
            }
            tm = block_sum(tm, sm);
            tv = block_sum(tv, sm);
            if (threadIdx.x == 0) {
                st<T>(rs.out_mean + k, (1.0f - rs.momentum) * ld<T>(rs.rmean + k) + rs.momentum * (tm / (float)rs.N));
                st<T>(rs.out_var + k, (1.0f - rs.momentum) * ld<T>(rs.rvar + k) + rs.corrected * (tv / (float)rs.N));
            }
        }
    } else if (threadIdx.x == 0) {
        if (save_mean) save_mean[slice] = mean;
        if (save_invstd) save_invstd[slice] = invstd;
    }
    // pass 3: normalise.  Scale and shift of the group's channels go through LDS (groups of up to 64 channels): read
    // from global memory per vector, the loads would sit between the stores of this pass, and a load waits for the
    // store before it (a wave's memory operations complete in the order of their issue).
    __shared__ float chan[2 * 64];
    const bool tabled = g.Cg <= 64;
    if (tabled) {
        if (threadIdx.x < g.Cg) {
            const uint32_t c = k * g.Cg + threadIdx.x;
            const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
            chan[2 * threadIdx.x] = sc;
            chan[2 * threadIdx.x + 1] = fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
        }
        __syncthreads();
    }
    auto emit = [&](uint32_t q, const float (&xv)[VEC]) {
        const uint32_t j = g.chdiv.div(q), c = k * g.Cg + j;
        const float sc = tabled ? chan[2 * j] : (gamma ? ld(gamma + c) : 1.0f) * invstd;
        const float sh = tabled ? chan[2 * j + 1] : fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
        float o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = Act<ACT>::f(fmaf(xv[e], sc, sh));
        gn_store<T, VEC>(y, base + (size_t)q * VEC, o);
    };
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            const uint32_t q = u * T_ + threadIdx.x;
            if (q < g.nvec) {
                K::get(kv[u], v[0]);
                emit(q, v[0]);
            }
        }
    } else {
        for (uint32_t q = threadIdx.x; q < g.nvec; q += T_) {
            gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
            emit(q, v[0]);
        }
    }
}

// ------------------------------------------------------------------------------- pullback
// Adds the per-lane contributions (a, b) of channel j to this wave's LDS accumulators.
// Lanes of a wave usually share j (rows are longer than a wave); otherwise the distinct
// channels present in the wave are handled one after the other.
__device__ __forceinline__ void wave_channel_accumulate(float* accg, float* accb, uint32_t j, float a, float b,
                                                        bool active) {
    const int lane = threadIdx.x & 63;
    unsigned long long todo = __ballot(active);
    while (todo) {
        const int first = __ffsll((long long)todo) - 1;
        const uint32_t j0 = (uint32_t)__builtin_amdgcn_readlane((int)j, first);   // first is uniform
        const bool sel = active && j == j0;
        const float ta = wave_sum(sel ? a : 0.0f);
        const float tb = wave_sum(sel ? b : 0.0f);
        if (lane == 0) {
            accg[j0] += ta;
            accb[j0] += tb;
        }
        todo &= ~__ballot(sel);
    }
}

template <typename T, int ACT, int VEC, bool CACHED, bool AFFINE>
__global__ void gn_bwd_kernel(const T* __restrict__ delta, const T* __restrict__ x, const T* __restrict__ gamma,
                              const T* __restrict__ beta, const float* __restrict__ save_mean,
                              const float* __restrict__ save_invstd, T* dx, float* pdg, float* pdb, T* dgamma,
                              T* dbeta, uint32_t* counters, uint32_t cstride, uint32_t N, GnGeom g, GnExchange ex) {
    extern __shared__ float lds[];                  // [16] reduction scratch, then [nw][Cg] x 2
    float* sm = lds;
    const uint32_t T_ = blockDim.x, nw = T_ >> 6, w = threadIdx.x >> 6;
    float* accg = lds + 16 + (size_t)w * g.Cg;
    float* accb = lds + 16 + (size_t)(nw + w) * g.Cg;
    __shared__ float pst[2 * 4 + 2];                // exchanged part sums (parts <= 4), then the slice totals
    const uint32_t parts = CACHED ? g.parts : 1u;
    const uint32_t slice = blockIdx.x / parts, part = blockIdx.x - slice * parts;
    const uint32_t k = slice % g.G, n = slice / g.G;
    const uint32_t qbeg = part * g.pvec, qend = CACHED ? qbeg + g.pvec : g.nvec;   // this workgroup's vectors of the slice
    const size_t base = (size_t)slice * g.nvec * VEC;
    const float mean = save_mean[slice], invstd = save_invstd[slice];
    // the normalised value: with 16-bit storage one fused multiply-add (x carries 8 bits, so the rounding of mean * invstd
    // does not show); fp32 storage subtracts first, which keeps every bit when x is close to the mean
    const float nmean = -mean * invstd;
    auto xhat = [&](float xe) { return sizeof(T) == 2 ? fmaf(xe, invstd, nmean) : (xe - mean) * invstd; };
    if constexpr (AFFINE) {
        for (uint32_t i = threadIdx.x; i < 2 * nw * g.Cg; i += T_) lds[16 + i] = 0.0f;
        __syncthreads();
    }
    using K = Kept<T, VEC>;
    typename K::type kd[CACHED ? kGnCache : 1], kv[CACHED ? kGnCache : 1];
    float d[1][VEC], v[1][VEC];
    // After the first pass kd holds g = dy * act'(y) * gamma, so the second pass needs neither the activation
    // derivative nor the parameters (whose loads, between the dx stores, would each wait for the stores before
    // them).  fp32 storage keeps g as it is; bf16 storage keeps it as eight fp16 values in the vector's four
    // registers (11 bits against the 8 that dx is rounded to anyway), scaled by a power of two that the thread
    // takes from its first vector (its largest |g| lands in [256, 512): cotangents of any magnitude keep their
    // bits, and later vectors may be 128 times larger).  A workgroup in which a value still leaves the fp16
    // range reads the cotangent and x from memory again and recomputes (the check below).
    // (identity and relu recompute their derivative in the second pass instead: cheaper than the packing)
    constexpr bool HALF_G = sizeof(T) == 2 && VEC == 8 && ACT != LUXHIP_ACT_IDENTITY && ACT != LUXHIP_ACT_RELU;
    constexpr bool KEEP_G = sizeof(T) == 4 || HALF_G;
    auto keep_half = [](const float (&gv)[VEC]) {
        raw16_t r;
        if constexpr (VEC == 8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const _Float16 lo = (_Float16)gv[2 * i];         // beyond the fp16 range: infinite, and the workgroup
                const _Float16 hi = (_Float16)gv[2 * i + 1];     // recomputes from memory (gmax below), never reading it
                r[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            }
        }
        return r;
    };
    auto get_half = [](const raw16_t& r, float (&gv)[VEC]) {
        if constexpr (VEC == 8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                gv[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r[i] & 0xffffu));
                gv[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r[i] >> 16));
            }
        }
    };
    float s1 = 0.0f, s2 = 0.0f;
    float gmax = 0.0f;                              // largest scaled |g| this thread has packed as fp16
    float gscale = 0.0f, gunscale = 0.0f;           // the thread's power of two and its inverse; 0: not chosen yet

    // gamma, scale and shift of the group's channels through LDS (groups of up to 64 channels): one global load per
    // workgroup and channel instead of two per vector, each with its own wait
    __shared__ float chan[3 * 64];
    const bool tabled = g.Cg <= 64;
    if (tabled) {
        if (threadIdx.x < g.Cg) {
            const uint32_t c = k * g.Cg + threadIdx.x;
            const float gm = gamma ? ld(gamma + c) : 1.0f;
            chan[3 * threadIdx.x] = gm;
            chan[3 * threadIdx.x + 1] = gm * invstd;
            chan[3 * threadIdx.x + 2] = fmaf(-mean, gm * invstd, beta ? ld(beta + c) : 0.0f);
        }
        __syncthreads();
    }
    // dy and g = dy * gamma for one vector; also returns the channel's parameters
    auto grad_terms = [&](uint32_t q, const float (&dv)[VEC], const float (&xv)[VEC], float (&gv)[VEC], float& a, float& b) {
        const uint32_t j = g.chdiv.div(q), c = k * g.Cg + j;
        const float gm = tabled ? chan[3 * j] : (gamma ? ld(gamma + c) : 1.0f);
        const float sc = tabled ? chan[3 * j + 1] : gm * invstd;
        const float sh = tabled ? chan[3 * j + 2] : fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
        a = 0.0f;
        b = 0.0f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float dy = dv[e];
            if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                const float pre = fmaf(xv[e], sc, sh);
                dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
            }
            const float xh = xhat(xv[e]);
            gv[e] = dy * gm;
            a = fmaf(dy, xh, a);
            b += dy;
        }
    };

    // Parameter-gradient terms of a lane stay in its registers while its vectors lie in one channel (rows are
    // usually many vectors long); the wave adds them up across lanes (DPP chain, LDS accumulators) only when a lane
    // moves on to another channel, and once at the end.  j = jc for a lane without a vector in this trip.
    constexpr uint32_t kNoChannel = 0xffffffffu;
    uint32_t jc = kNoChannel;
    float ac = 0.0f, bc = 0.0f;
    auto gather = [&](uint32_t j, float a, float b) {
        if (__any((int)(j != jc && jc != kNoChannel))) {       // uniform over the wave
            wave_channel_accumulate(accg, accb, jc, ac, bc, jc != kNoChannel);
            ac = 0.0f;
            bc = 0.0f;
        }
        jc = j;
        ac += a;
        bc += b;
    };

    const uint32_t iters = (qend - qbeg + T_ - 1) / T_;
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            const size_t off = base + (size_t)min(qbeg + u * T_ + threadIdx.x, qend - 1) * VEC;   // past the end: last vector again
            kd[u] = K::load(delta, off);
            kv[u] = K::load(x, off);
        }
    }
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            if ((uint32_t)u < iters) {              // uniform
                const uint32_t q = qbeg + u * T_ + threadIdx.x;
                const bool active = q < qend;
                float gv[VEC], a = 0.0f, b = 0.0f;
                if (active) {
                    K::get(kd[u], d[0]);
                    K::get(kv[u], v[0]);
                    grad_terms(q, d[0], v[0], gv, a, b);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float xh = xhat(v[0][e]);
                        s1 += gv[e];
                        s2 = fmaf(gv[e], xh, s2);
                    }
                    if constexpr (HALF_G) {
                        float m = 0.0f;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) m = fmaxf(m, fabsf(gv[e]));
                        if (gscale == 0.0f && m > 0.0f) {
                            if (m < 3.0e38f) {
                                const int ex = __builtin_amdgcn_frexp_expf(m);   // m = f * 2^ex, 0.5 <= f < 1
                                gscale = __builtin_ldexpf(1.0f, 9 - ex);
                                gunscale = __builtin_ldexpf(1.0f, ex - 9);
                            } else {
                                gmax = m;                                        // infinite: recompute from memory
                            }
                        }
                        float hv[VEC];
#pragma unroll
                        for (int e = 0; e < VEC; ++e) hv[e] = gv[e] * gscale;
                        gmax = fmaxf(gmax, m * gscale);
                        kd[u] = keep_half(hv);
                    } else if constexpr (KEEP_G) {
                        kd[u] = keep<T, VEC>(gv);
                    }
                }
                if constexpr (AFFINE) gather(active ? g.chdiv.div(q) : jc, a, b);
            }
        }
    } else {
        for (uint32_t u = 0; u < iters; ++u) {
            const uint32_t q = u * T_ + threadIdx.x;
            const bool active = q < g.nvec;
            float gv[VEC], a = 0.0f, b = 0.0f;
            if (active) {
                gn_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
                gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
                grad_terms(q, d[0], v[0], gv, a, b);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xh = xhat(v[0][e]);
                    s1 += gv[e];
                    s2 = fmaf(gv[e], xh, s2);
                }
            }
            if constexpr (AFFINE) gather(active ? g.chdiv.div(q) : jc, a, b);
        }
    }
    if constexpr (AFFINE) wave_channel_accumulate(accg, accb, jc, ac, bc, jc != kNoChannel);
    s1 = block_sum(s1, sm);
    s2 = block_sum(s2, sm);
    if (parts > 1) {
        // part sums -> the other workgroups of the slice; added in part order
        uint64_t* words = ex.words + (size_t)slice * parts * 2;
        if (threadIdx.x == 0) {
            publish_tagged(words + 2 * part, s1, ex.epoch);
            publish_tagged(words + 2 * part + 1, s2, ex.epoch);
        }
        if (!collect_tagged(words, 2 * parts, ex.epoch, ex.spin_limit, pst)) {
            // a peer did not show up in time: its sums are recomputed here from global memory
            for (uint32_t i = 0; i < parts; ++i) {
                float t1 = 0.0f, t2 = 0.0f;
                for (uint32_t q = i * g.pvec + threadIdx.x; q < (i + 1) * g.pvec; q += T_) {
                    float gv[VEC], a, b;
                    gn_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
                    gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
                    grad_terms(q, d[0], v[0], gv, a, b);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        t1 += gv[e];
                        t2 = fmaf(gv[e], xhat(v[0][e]), t2);
                    }
                }
                t1 = block_sum(t1, sm);
                t2 = block_sum(t2, sm);
                if (threadIdx.x == 0) { pst[2 * i] = t1; pst[2 * i + 1] = t2; }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) {
            float t1 = 0.0f, t2 = 0.0f;
            for (uint32_t i = 0; i < parts; ++i) { t1 += pst[2 * i]; t2 += pst[2 * i + 1]; }
            pst[8] = t1;
            pst[9] = t2;
        }
        __syncthreads();
        s1 = pst[8];
        s2 = pst[9];
    }
    s1 *= g.inv_m;
    s2 *= g.inv_m;

    // Parameter gradients first (they only need the first pass), so that their hand-off does not
    // wait for the dx stores below.
    if constexpr (AFFINE) {
        const uint32_t jbeg = part * (g.Cg / parts), jend = jbeg + g.Cg / parts;   // a part owns whole channels
        for (uint32_t j = jbeg + threadIdx.x; j < jend; j += T_) {
            float tg = 0.0f, tb = 0.0f;
            for (uint32_t ww = 0; ww < nw; ++ww) {
                tg += lds[16 + (size_t)ww * g.Cg + j];
                tb += lds[16 + (size_t)(nw + ww) * g.Cg + j];
            }
            publish(pdg + (size_t)n * g.C + k * g.Cg + j, tg);
            publish(pdb + (size_t)n * g.C + k * g.Cg + j, tb);
        }
        publish_done();
        // the workgroup of group k that arrives last (parts per sample) adds the N per-sample
        // partials of the group's channels in sample order
        uint32_t* last_flag = reinterpret_cast<uint32_t*>(lds + 15);   // a word of the reduction scratch that is free now
        if (arrive_last(counters + (size_t)k * cstride, N * parts, last_flag)) {
            for (uint32_t j = threadIdx.x; j < g.Cg; j += T_) {
                float tg = 0.0f, tb = 0.0f;
                for (uint32_t nn = 0; nn < N; ++nn) {
                    tg += fetch(pdg + (size_t)nn * g.C + k * g.Cg + j);
                    tb += fetch(pdb + (size_t)nn * g.C + k * g.Cg + j);
                }
                if (dgamma) st(dgamma + k * g.Cg + j, tg);
                if (dbeta) st(dbeta + k * g.Cg + j, tb);
            }
        }
    }

    // a scaled |g| beyond the fp16 range (a vector far larger than the thread's first one, or an infinite value) was
    // saturated in the registers: such a workgroup takes the cotangent and x from memory again and recomputes
    const bool refetch = HALF_G && __syncthreads_or(gmax > 65504.0f);
    auto emit = [&](uint32_t q, const float (&dv)[VEC], const float (&xv)[VEC]) {
        float gv[VEC], a, b, o[VEC];
        grad_terms(q, dv, xv, gv, a, b);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float xh = xhat(xv[e]);
            o[e] = invstd * (gv[e] - s1 - xh * s2);
        }
        gn_store<T, VEC>(dx, base + (size_t)q * VEC, o);
    };
    if constexpr (CACHED) {
#pragma unroll
        for (int u = 0; u < kGnCache; ++u) {
            const uint32_t q = qbeg + u * T_ + threadIdx.x;
            if (q < qend) {
                if (refetch) {
                    gn_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
                    gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
                    emit(q, d[0], v[0]);
                    continue;
                }
                if constexpr (HALF_G) get_half(kd[u], d[0]);
                else K::get(kd[u], d[0]);
                K::get(kv[u], v[0]);
                if constexpr (KEEP_G) {             // kd[u] holds dy * act' * gamma (HALF_G: times gscale)
                    // invstd * (g - s1 - xh * s2) as two fused multiply-adds per element
                    const float kg = HALF_G ? invstd * gunscale : invstd, k1 = -s1 * invstd, k2 = -s2 * invstd;
                    float o[VEC];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float xh = xhat(v[0][e]);
                        o[e] = fmaf(xh, k2, fmaf(d[0][e], kg, k1));
                    }
                    gn_store<T, VEC>(dx, base + (size_t)q * VEC, o);
                } else {
                    emit(q, d[0], v[0]);
                }
            }
        }
    } else {
        for (uint32_t q = threadIdx.x; q < g.nvec; q += T_) {
            gn_load<T, VEC>(delta, base + (size_t)q * VEC, d[0]);
            gn_load<T, VEC>(x, base + (size_t)q * VEC, v[0]);
            emit(q, d[0], v[0]);
        }
    }
}

// ------------------------------------------------------------------------------- host side
static int gn_check(int dtype, int act, int64_t I, int64_t C, int64_t G, int64_t N) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    LUX_INVALID_IF(I < 0 || C < 0 || N < 0 || G <= 0, "invalid dimension");
    LUX_INVALID_IF(C % G != 0, "number of channels %lld must be divisible by the number of groups %lld", (long long)C,
                   (long long)G);
    if (I > 0 && C > 0 && N > 0) {
        const long double tot = (long double)I * (long double)C * (long double)N;
        LUX_UNSUPPORTED_IF(tot >= 2147483648.0L, "tensors of 2^31 or more elements are not supported");
    }
    return LUXHIP_OK;
}

struct GnLaunch {
    GnGeom g;
    bool vec, cached;
    unsigned threads, blocks;
};

template <typename T>
static GnLaunch gn_plan(int64_t I, int64_t C, int64_t G, int64_t N, bool ptr_ok, bool allow_split) {
    constexpr int V = Vec<T>::N;
    GnLaunch L;
    const int64_t Cg = C / G, m = I * Cg;
    L.vec = ptr_ok && I % V == 0;
    const int vv = L.vec ? V : 1;
    L.g.I = (uint32_t)I; L.g.Cg = (uint32_t)Cg; L.g.G = (uint32_t)G; L.g.C = (uint32_t)C;
    L.g.nvec = (uint32_t)(m / vv);
    L.g.chdiv = FastDiv((uint32_t)(I / vv));
    L.g.inv_m = 1.0f / (float)m;
    // A slice that would need a 1024-thread workgroup can be split between two 512-thread
    // workgroups (each owns whole channels): two of them fit a compute unit even with the
    // pullback's register footprint, and one loads while the other computes or stores.  The halves
    // exchange their partial sums through tagged words.  Measured: 5 % faster for the pullback,
    // slower for the forward pass (which fits twice per compute unit anyway), so only the
    // pullback asks for it.
    L.g.parts = 1;
    if (allow_split && L.vec && (int64_t)L.g.nvec > 512 * kGnCache && (int64_t)L.g.nvec <= 2 * 512 * kGnCache && Cg % 2 == 0 &&
        (L.g.nvec / 2) % (uint32_t)(I / vv) == 0 && (size_t)(G * N) * 2 * 3 * 2 <= kWorkspaceFlags)
        L.g.parts = 2;
    L.g.pvec = L.g.nvec / L.g.parts;
    int64_t t = 64;
    while (t < 1024 && t * kGnCache < L.g.pvec) t <<= 1;
    L.threads = (unsigned)t;
    L.cached = (int64_t)L.g.pvec <= t * kGnCache;
    if (!L.cached) { L.g.parts = 1; L.g.pvec = L.g.nvec; }
    L.blocks = (unsigned)(G * N * L.g.parts);
    return L;
}

static int gn_exchange(hipStream_t s, GnExchange* ex) {
    Workspace ws;
    int rc = get_workspace(s, 0, &ws);
    if (rc != LUXHIP_OK) return rc;
    ex->words = reinterpret_cast<uint64_t*>(ws.flags);
    ex->epoch = ws.epoch;
    ex->spin_limit = (uint32_t)option_bn_spin_limit();
    return LUXHIP_OK;
}

template <typename T>
static int gn_fwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t G, int64_t N, const T* x, const T* gamma,
                       const T* beta, float eps, T* y, float* save_mean, float* save_invstd, InRunning<T> rs = InRunning<T>{}) {
    constexpr int V = Vec<T>::N;
    GnLaunch L = gn_plan<T>(I, C, G, N, aligned16(x) && aligned16(y), false);
    if (rs.out_mean != nullptr) {
        LUX_UNSUPPORTED_IF((size_t)C > kWorkspaceCounters, "instancenorm: more than %zu channels", kWorkspaceCounters);
        Workspace ws;
        int rc = get_workspace(s, (size_t)C * N * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        rs.counters = ws.counters;
        rs.var = reinterpret_cast<float*>(ws.data);
        rs.cstride = counter_stride(C);
        rs.N = (uint32_t)N;
    }
    ProfScope ps("gn_fwd_kernel", s, true);
#define GN_FWD(A)                                                                                                     \
    do {                                                                                                              \
        if (L.vec && L.cached) launch_exact(ps, gn_fwd_kernel<T, A, V, true>, dim3(L.blocks), dim3(L.threads), 0, s, x, gamma, beta, y, save_mean, save_invstd, L.g, eps, rs);   \
        else if (L.vec) launch_exact(ps, gn_fwd_kernel<T, A, V, false>, dim3(L.blocks), dim3(L.threads), 0, s, x, gamma, beta, y, save_mean, save_invstd, L.g, eps, rs);        \
        else if (L.cached) launch_exact(ps, gn_fwd_kernel<T, A, 1, true>, dim3(L.blocks), dim3(L.threads), 0, s, x, gamma, beta, y, save_mean, save_invstd, L.g, eps, rs);      \
        else launch_exact(ps, gn_fwd_kernel<T, A, 1, false>, dim3(L.blocks), dim3(L.threads), 0, s, x, gamma, beta, y, save_mean, save_invstd, L.g, eps, rs);                   \
    } while (0)
    LUX_DISPATCH_ACT(act, GN_FWD);
#undef GN_FWD
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
static int gn_bwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t G, int64_t N, const T* delta, const T* x,
                       const T* gamma, const T* beta, const float* save_mean, const float* save_invstd, T* dx,
                       T* dgamma, T* dbeta) {
    constexpr int V = Vec<T>::N;
    GnLaunch L = gn_plan<T>(I, C, G, N, aligned16(x) && aligned16(delta) && aligned16(dx), !stream_capturing(s));
    const bool affine = gamma != nullptr && (dgamma != nullptr || dbeta != nullptr);
    // LDS: 16 floats of reduction scratch + 2 * nw * Cg accumulators
    size_t lds_bytes = 64;
    if (affine) {
        while (L.threads > 64 && (16 + 2 * (size_t)(L.threads / 64) * L.g.Cg) * 4 > 60 * 1024) {
            L.threads >>= 1;
            L.cached = (int64_t)L.g.pvec <= (int64_t)L.threads * kGnCache;
        }
        if (!L.cached && L.g.parts > 1) {           // the streaming kernel works on whole slices
            L.g.parts = 1;
            L.g.pvec = L.g.nvec;
            L.blocks = (unsigned)(G * N);
        }
        lds_bytes = (16 + 2 * (size_t)(L.threads / 64) * L.g.Cg) * 4;
        LUX_UNSUPPORTED_IF(lds_bytes > 60 * 1024, "groupnorm_bwd: %u channels per group exceed the LDS accumulators", L.g.Cg);
    }
    float *pdg = nullptr, *pdb = nullptr;
    uint32_t* counters = nullptr;
    const uint32_t cstride = counter_stride(G);
    GnExchange ex;
    {
        int rc = gn_exchange(s, &ex);
        if (rc != LUXHIP_OK) return rc;
    }
    if (affine) {
        LUX_UNSUPPORTED_IF((size_t)G > kWorkspaceCounters, "groupnorm_bwd: more than %zu groups", kWorkspaceCounters);
        Workspace ws;
        int rc = get_workspace(s, (size_t)2 * N * C * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        pdg = reinterpret_cast<float*>(ws.data);
        pdb = pdg + (size_t)N * C;
        counters = ws.counters;
    }
    {
        ProfScope ps("gn_bwd_kernel", s, true);
#define GN_BWD_A(A, VV, CA)                                                                                           \
    do {                                                                                                              \
        if (affine) launch_exact(ps, gn_bwd_kernel<T, A, VV, CA, true>, dim3(L.blocks), dim3(L.threads), lds_bytes, s, delta, x, gamma, beta, save_mean, save_invstd, dx, pdg, pdb, dgamma, dbeta, counters, cstride, (uint32_t)N, L.g, ex); \
        else launch_exact(ps, gn_bwd_kernel<T, A, VV, CA, false>, dim3(L.blocks), dim3(L.threads), lds_bytes, s, delta, x, gamma, beta, save_mean, save_invstd, dx, pdg, pdb, dgamma, dbeta, counters, cstride, (uint32_t)N, L.g, ex);       \
    } while (0)
#define GN_BWD(A)                                                                                                     \
    do {                                                                                                              \
        if (L.vec && L.cached) GN_BWD_A(A, V, true);                                                                  \
        else if (L.vec) GN_BWD_A(A, V, false);                                                                        \
        else if (L.cached) GN_BWD_A(A, 1, true);                                                                      \
        else GN_BWD_A(A, 1, false);                                                                                   \
    } while (0)
        LUX_DISPATCH_ACT(act, GN_BWD);
#undef GN_BWD
#undef GN_BWD_A
    }
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// instancenorm's running statistics: the statistics of the (channel, sample) slices averaged over
// the batch, the variance with the n / (n - 1) correction of a slice of n = I values.
template <typename T>
__global__ __launch_bounds__(256) void in_running_stats_kernel(const float* __restrict__ mean, const float* __restrict__ invstd,
                                                               int C, int N, float eps, float momentum, float corrected,
                                                               const T* __restrict__ rmean, const T* __restrict__ rvar,
                                                               T* __restrict__ rmean_out, T* __restrict__ rvar_out) {
    // one wavefront per channel, the lanes stride over the samples
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c >= C) return;
    const int lane = threadIdx.x & 63;
    float sm = 0.f, sv = 0.f;
    for (int n = lane; n < N; n += 64) {
        const float is = invstd[c + (size_t)C * n];
        sm += mean[c + (size_t)C * n];
        sv += fmaxf(1.f / (is * is) - eps, 0.f);   // rounding can take the difference below zero when var << eps
    }
    sm = wave_sum(sm);
    sv = wave_sum(sv);
    if (lane == 0) {
        st<T>(rmean_out + c, (1.f - momentum) * ld<T>(rmean + c) + momentum * (sm / (float)N));
        st<T>(rvar_out + c, (1.f - momentum) * ld<T>(rvar + c) + corrected * (sv / (float)N));
    }
}

template <typename T>
static int in_running_stats_impl(hipStream_t s, int64_t I, int64_t C, int64_t N, const float* mean, const float* invstd,
                                 float eps, float momentum, const T* rmean, const T* rvar, T* rmean_out, T* rvar_out) {
    const float m = (float)I;
    const float corrected = momentum * m / (m - 1.f);            // update_normalization_statistics
    ProfScope ps("in_running_stats_kernel", s);
    in_running_stats_kernel<T><<<dim3((unsigned)ceil_div(C, 4)), dim3(256), 0, s>>>(mean, invstd, (int)C, (int)N, eps, momentum,
                                                                                      corrected, rmean, rvar, rmean_out, rvar_out);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
static int in_fwd_t(hipStream_t s, int act, int64_t I, int64_t C, int64_t N, const void* x, const void* gamma, const void* beta,
                    float eps, void* y, float* save_mean, float* save_invstd, float momentum, const void* rmean,
                    const void* rvar, void* rmean_out, void* rvar_out) {
    InRunning<T> rs{};
    rs.rmean = (const T*)rmean; rs.rvar = (const T*)rvar; rs.out_mean = (T*)rmean_out; rs.out_var = (T*)rvar_out;
    rs.momentum = momentum;
    rs.corrected = momentum * (float)I / ((float)I - 1.0f);        // update_normalization_statistics
    return gn_fwd_impl<T>(s, act, I, C, C, N, (const T*)x, (const T*)gamma, (const T*)beta, eps, (T*)y, save_mean, save_invstd, rs);
}

}  // namespace luxhip


using namespace luxhip;

extern "C" {

int luxhip_groupnorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t G, int64_t N, const void* x,
                         const void* gamma, const void* beta, double eps, void* y, float* save_mean,
                         float* save_invstd) {
    LUX_REQUIRE_INIT();
    int rc = gn_check(dtype, act, I, C, G, N);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "groupnorm_fwd: gamma and beta must be given together");
    if (I * C * N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || y == nullptr, "groupnorm_fwd: x and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return gn_fwd_impl<float>((hipStream_t)s, act, I, C, G, N, (const float*)x, (const float*)gamma, (const float*)beta,
                                  (float)eps, (float*)y, save_mean, save_invstd);
    return gn_fwd_impl<bf16_t>((hipStream_t)s, act, I, C, G, N, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta,
                               (float)eps, (bf16_t*)y, save_mean, save_invstd);
}

int luxhip_instancenorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* x,
                            const void* gamma, const void* beta, double eps, void* y, float* save_mean, float* save_invstd,
                            double momentum, const void* rmean, const void* rvar, void* rmean_out, void* rvar_out) {
    LUX_REQUIRE_INIT();
    int rc = gn_check(dtype, act, I, C, C > 0 ? C : 1, N);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "instancenorm_fwd: gamma and beta must be given together");
    if (I * C * N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || y == nullptr || save_mean == nullptr || save_invstd == nullptr || rmean == nullptr ||
                       rvar == nullptr || rmean_out == nullptr || rvar_out == nullptr,
                   "instancenorm_fwd: x, y, the saved statistics and the running statistics must not be NULL");
    if (dtype == LUXHIP_F32)
        return in_fwd_t<float>((hipStream_t)s, act, I, C, N, x, gamma, beta, (float)eps, y, save_mean, save_invstd, (float)momentum,
                               rmean, rvar, rmean_out, rvar_out);
    return in_fwd_t<bf16_t>((hipStream_t)s, act, I, C, N, x, gamma, beta, (float)eps, y, save_mean, save_invstd, (float)momentum,
                            rmean, rvar, rmean_out, rvar_out);
}

int luxhip_groupnorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t G, int64_t N,
                         const void* delta, const void* x, const void* gamma, const void* beta, const float* save_mean,
                         const float* save_invstd, void* dx, void* dgamma, void* dbeta) {
    LUX_REQUIRE_INIT();
    int rc = gn_check(dtype, act, I, C, G, N);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF((gamma == nullptr) != (beta == nullptr), "groupnorm_bwd: gamma and beta must be given together");
    if (I * C * N == 0) {   // nothing to read: the parameter gradients are empty sums
        const size_t bytes = (size_t)C * (dtype == LUXHIP_F32 ? 4 : 2);
        if (C > 0 && dgamma) { rc = luxhip_fill_zero(dgamma, bytes, s); if (rc) return rc; }
        if (C > 0 && dbeta) { rc = luxhip_fill_zero(dbeta, bytes, s); if (rc) return rc; }
        return LUXHIP_OK;
    }
    LUX_INVALID_IF(delta == nullptr || x == nullptr || dx == nullptr || save_mean == nullptr || save_invstd == nullptr,
                   "groupnorm_bwd: delta, x, dx, save_mean and save_invstd must not be NULL");
    if (dtype == LUXHIP_F32)
        return gn_bwd_impl<float>((hipStream_t)s, act, I, C, G, N, (const float*)delta, (const float*)x, (const float*)gamma,
                                  (const float*)beta, save_mean, save_invstd, (float*)dx, (float*)dgamma, (float*)dbeta);
    return gn_bwd_impl<bf16_t>((hipStream_t)s, act, I, C, G, N, (const bf16_t*)delta, (const bf16_t*)x, (const bf16_t*)gamma,
                               (const bf16_t*)beta, save_mean, save_invstd, (bf16_t*)dx, (bf16_t*)dgamma, (bf16_t*)dbeta);
}

int luxhip_instancenorm_running_stats(luxhip_stream_t s, int dtype, int64_t I, int64_t C, int64_t N, const float* save_mean,
                                      const float* save_invstd, double eps, double momentum, const void* rmean,
                                      const void* rvar, void* rmean_out, void* rvar_out) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(I < 0 || C < 0 || N < 0, "invalid dimension");
    if (C == 0) return LUXHIP_OK;
    LUX_INVALID_IF(I * N == 0, "instancenorm_running_stats: statistics of empty slices");
    LUX_UNSUPPORTED_IF(C * N >= 2147483648LL, "instancenorm_running_stats: too many slices");
    LUX_INVALID_IF(save_mean == nullptr || save_invstd == nullptr || rmean == nullptr || rvar == nullptr ||
                       rmean_out == nullptr || rvar_out == nullptr,
                   "instancenorm_running_stats: no argument may be NULL");
    if (dtype == LUXHIP_F32)
        return in_running_stats_impl<float>((hipStream_t)s, I, C, N, save_mean, save_invstd, (float)eps, (float)momentum,
                                            (const float*)rmean, (const float*)rvar, (float*)rmean_out, (float*)rvar_out);
    return in_running_stats_impl<bf16_t>((hipStream_t)s, I, C, N, save_mean, save_invstd, (float)eps, (float)momentum,
                                         (const bf16_t*)rmean, (const bf16_t*)rvar, (bf16_t*)rmean_out, (bf16_t*)rvar_out);
}

}  // extern "C"
