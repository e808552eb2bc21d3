// batchnorm forward (statistics + running-stat update + normalise/activate) and the complete
// pullback, as HBM-bound streaming kernels over the (I, C, N) view.
//
// Channel c owns the rows (n*C + c)*I .. +I for every n.  Reduction kernels use a (S, C)
// grid: workgroup (s, c) works on a contiguous slice of channel c's I*N elements and publishes
// one partial result; partials are always combined in slice order, so results do not depend on
// scheduling.  No floating-point atomics and no cache-wide fences (see common.h, cross-workgroup
// hand-off).
//
// Resident path (tensor fits the register file: C*S <= workgroups the device holds at once,
// slice <= 8 vectors per thread of a 512-thread workgroup, two workgroups per compute unit),
// one kernel and one trip through HBM per tensor:
//   forward : bn_fwd_resident_kernel  load x -> slice statistics -> publish as (value, epoch)
//             words, collect the words of the channel's other slices -> mean/invstd (+ running
//             stats, saved stats) -> write y
//   pullback: bn_bwd_resident_kernel  load delta, x -> slice sums -> publish, wait -> dgamma, dbeta
//             -> write dx
//   All workgroups of the grid are resident at once (the host asks the occupancy calculator how
//   many a compute unit holds), so the wait ends as
//   soon as the slowest peer has published.  The wait is bounded all the same: a workgroup that
//   gives up recomputes the peers' partials itself from global memory.
// Streaming path (any size):
//   forward, training : bn_stats_kernel (read x) -> partials; the workgroup of a channel that
//                       arrives last combines them -> mean, invstd, scale, shift, running stats
//                       bn_apply_kernel  (read x, write y)
//   forward, inference: bn_infer_prep_kernel (C threads) -> scale, shift;  bn_apply_kernel
//   pullback          : bn_bwd_reduce_kernel (read delta, x) -> partials; last arriver -> dgamma,
//                       dbeta, per-channel coefficients;  bn_bwd_apply_kernel (read delta, x, write dx)
#include <algorithm>
#include <mutex>
#include <unordered_map>

#include "common.h"

namespace luxhip {

constexpr int kBnThreads = 256;
constexpr int kBnUnroll = 4;  // 16-byte vectors per thread; all of a thread's loads are issued before the first use

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

// ------------------------------------------------------------------------------- statistics
struct BnFwdParams {
    const void *gamma, *beta, *rmean, *rvar;   // storage type T
    void *rmean_out, *rvar_out;                // NULL: running statistics are not updated
    float *save_mean, *save_invstd;            // may be NULL
    float count, momentum, eps;
};

// Wave-wide: combines S partial (count, mean, M2) triples read through `get(i, k)` in a fixed
// tree order; lane 0 holds the result.
template <typename Get>
__device__ __forceinline__ void merge_stat_partials(uint32_t S, Get get, float& n, float& mean, float& m2) {
    const uint32_t lane = threadIdx.x & 63;
    n = 0.0f; mean = 0.0f; m2 = 0.0f;
    for (uint32_t i = lane; i < S; i += kWave) chan_merge(n, mean, m2, get(i, 0), get(i, 1), get(i, 2));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float nb = __shfl_xor(n, off, kWave), mb = __shfl_xor(mean, off, kWave), qb = __shfl_xor(m2, off, kWave);
        chan_merge(n, mean, m2, nb, mb, qb);
    }
}

// One thread: every per-channel result of the forward pass from the channel's (mean, M2).
template <typename T>
__device__ __forceinline__ void bn_fwd_channel_results(const BnFwdParams& p, uint32_t c, float mean, float m2,
                                                       float* scale, float* shift, float& sc, float& sh) {
    const T* gamma = static_cast<const T*>(p.gamma);
    const T* beta = static_cast<const T*>(p.beta);
    const float var = m2 / p.count;
    const float invstd = 1.0f / sqrtf(var + p.eps);
    sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
    sh = fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
    if (scale) { scale[c] = sc; shift[c] = sh; }
    if (p.save_mean) p.save_mean[c] = mean;
    if (p.save_invstd) p.save_invstd[c] = invstd;
    if (p.rmean_out) {
        const float m1 = p.momentum, m3 = 1.0f - p.momentum;
        const float m2c = p.momentum * p.count / (p.count - 1.0f);
        st(static_cast<T*>(p.rmean_out) + c, m3 * ld(static_cast<const T*>(p.rmean) + c) + m1 * mean);
        st(static_cast<T*>(p.rvar_out) + c, m3 * ld(static_cast<const T*>(p.rvar) + c) + m2c * var);
    }
}

// Partial (count, mean, M2) of slice s of channel c -> partial[(c*S + s)*3 ..].  A workgroup
// keeps its slice (up to kStatVecs vectors per thread per trip) in registers and makes two
// passes over the registers: workgroup mean, then the sum of squared deviations from it (exact
// two-pass statistics per trip; trips and slices are combined with Chan's formula).
constexpr int kStatVecs = 4;
template <typename T, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_stats_kernel(const T* __restrict__ x, float* partial, uint32_t* counters,
                                                              uint32_t cstride, float* scale, float* shift,
                                                              BnFwdParams prm, ChanGeom g) {
    __shared__ float sm[kBnThreads / 64];
    __shared__ uint32_t last_flag;
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const uint32_t q0 = s * g.chunk, q1 = min(q0 + g.chunk, g.nq);
    float n = 0.0f, mean = 0.0f, m2 = 0.0f;   // running (count, mean, M2) over the trips of the outer loop
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
    float* mine = partial + ((size_t)c * S + s) * 3;
    if (threadIdx.x == 0) {
        publish(mine, n);
        publish(mine + 1, mean);
        publish(mine + 2, m2);
        publish_done();
    }
    if (!arrive_last(counters + (size_t)c * cstride, S, &last_flag)) return;
    if (threadIdx.x < kWave) {
        const float* p = partial + (size_t)c * S * 3;
        merge_stat_partials(S, [&](uint32_t i, int k) { return fetch(p + 3 * i + k); }, n, mean, m2);
        float sc, sh;
        if (threadIdx.x == 0) bn_fwd_channel_results<T>(prm, c, mean, m2, scale, shift, sc, sh);
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
            load_vec<T, VEC>(x, (size_t)min(idx[u], total_vec - 1) * VEC, v[u]);   // past the end: ignored below
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
// One thread: dgamma, dbeta and the coefficients of dx = A*dy + B*(x - mean) + D from the
// channel sums s1 = sum dy, s2 = sum dy * xhat.
template <typename T>
__device__ __forceinline__ void bn_bwd_channel_results(uint32_t c, float s1, float s2, const T* gamma, float invstd,
                                                       T* dgamma, T* dbeta, float inv_count, int stats_from_batch,
                                                       float& A, float& B, float& D) {
    const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
    if (dgamma) st(dgamma + c, s2);
    if (dbeta) st(dbeta + c, s1);
    A = sc;
    B = stats_from_batch ? -sc * invstd * s2 * inv_count : 0.0f;
    D = stats_from_batch ? -sc * s1 * inv_count : 0.0f;
}

// Partials of s1 = sum dy and s2 = sum dy * (x - mean) * invstd, dy = delta * act'(recomputed);
// the workgroup of a channel that arrives last adds them in slice order and writes dgamma, dbeta
// and coef[c], coef[C + c], coef[2C + c] = A, B, D.
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_reduce_kernel(
    const T* __restrict__ delta, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
    const float* __restrict__ save_mean, const float* __restrict__ save_invstd, float* partial, uint32_t* counters,
    uint32_t cstride, T* dgamma, T* dbeta, float* coef, float inv_count, int stats_from_batch, ChanGeom g) {
    __shared__ float sm[kBnThreads / 64];
    __shared__ uint32_t last_flag;
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
        publish(partial + ((size_t)c * S + s) * 2, s1);
        publish(partial + ((size_t)c * S + s) * 2 + 1, s2);
        publish_done();
    }
    if (!arrive_last(counters + (size_t)c * cstride, S, &last_flag)) return;
    if (threadIdx.x < kWave) {
        const float* p = partial + (size_t)c * S * 2;
        float t1 = 0.0f, t2 = 0.0f;
        for (uint32_t i = threadIdx.x; i < S; i += kWave) { t1 += fetch(p + 2 * i); t2 += fetch(p + 2 * i + 1); }
        t1 = wave_sum(t1);
        t2 = wave_sum(t2);
        if (threadIdx.x == 0) {
            float A, B, D;
            bn_bwd_channel_results<T>(c, t1, t2, gamma, invstd, dgamma, dbeta, inv_count, stats_from_batch, A, B, D);
            coef[c] = A;
            coef[g.C + c] = B;
            coef[2 * g.C + c] = D;
        }
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
            const size_t off = (size_t)min(idx[u], total_vec - 1) * VEC;   // past the end: ignored below
            load_vec<T, VEC>(delta, off, d[u]);
            load_vec<T, VEC>(x, off, v[u]);
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

// ------------------------------------------------------------------------------- resident path
constexpr int kResThreads = 512;    // two workgroups per compute unit
constexpr int kResVecs = 8;         // 16-byte vectors per thread held in registers
constexpr int kResMaxSlices = kResThreads / 3;   // one thread per exchange word, three words per slice
constexpr int kResPerCu = 1024 / kResThreads;   // resident workgroups per compute unit the kernels are compiled for

// Slice `slice` of channel c -> registers.  Vector u of a thread is vector q0 + u*1024 + tid of
// the slice; loads past the end of the slice are redirected to its last vector (every load is
// unconditional, so all of them are in flight together) and ignored by the users of v.
template <typename T>
__device__ __forceinline__ void res_load(const T* __restrict__ p, const ChanGeom& g, uint32_t c, uint32_t slice,
                                         raw16_t (&v)[kResVecs]) {
    constexpr int VEC = Vec<T>::N;
    const uint32_t q0 = slice * g.chunk, q1 = min(q0 + g.chunk, g.nq);
#pragma unroll
    for (int u = 0; u < kResVecs; ++u) {
        const uint32_t q = min(q0 + u * kResThreads + threadIdx.x, q1 - 1);
        v[u] = *reinterpret_cast<const raw16_t*>(p + g.offset(q, c, VEC));
    }
}

// Exact two-pass (count, mean, M2) of the slice held in v; every thread receives the result.
template <typename T>
__device__ __forceinline__ void res_slice_stats(const ChanGeom& g, uint32_t slice, const raw16_t (&v)[kResVecs],
                                                float* sm, float& n, float& mean, float& m2) {
    constexpr int VEC = Vec<T>::N;
    const uint32_t q0 = slice * g.chunk, q1 = min(q0 + g.chunk, g.nq);
    float sum = 0.0f;
#pragma unroll
    for (int u = 0; u < kResVecs; ++u)
        if (q0 + u * kResThreads + threadIdx.x < q1) {
            float f[VEC];
            Vec<T>::unpack(v[u], f);
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum += f[k];
        }
    n = (float)((q1 - q0) * VEC);
    mean = block_sum(sum, sm) / n;
    float dev = 0.0f;
#pragma unroll
    for (int u = 0; u < kResVecs; ++u)
        if (q0 + u * kResThreads + threadIdx.x < q1) {
            float f[VEC];
            Vec<T>::unpack(v[u], f);
#pragma unroll
            for (int k = 0; k < VEC; ++k) dev = fmaf(f[k] - mean, f[k] - mean, dev);
        }
    m2 = block_sum(dev, sm);
}

template <typename T, int ACT>
__global__ __launch_bounds__(kResThreads, kResPerCu) void bn_fwd_resident_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                      uint64_t* words, uint32_t epoch,
                                                                      uint32_t spin_limit, BnFwdParams prm, ChanGeom g) {
    constexpr int VEC = Vec<T>::N;
    __shared__ float sm[kResThreads / 64];
    __shared__ float parts[kResMaxSlices * 3];
    __shared__ float bc[2];
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    raw16_t v[kResVecs];
    res_load<T>(x, g, c, s, v);
    float n, mean, m2;
    res_slice_stats<T>(g, s, v, sm, n, mean, m2);
    uint64_t* chan_words = words + (size_t)c * S * 3;
    if (threadIdx.x == 0) {
        publish_tagged(chan_words + 3 * s, n, epoch);
        publish_tagged(chan_words + 3 * s + 1, mean, epoch);
        publish_tagged(chan_words + 3 * s + 2, m2, epoch);
    }
    if (!collect_tagged(chan_words, 3 * S, epoch, spin_limit, parts)) {
        // a peer did not show up in time: its share is recomputed here, the own slice last so
        // that v holds it again afterwards
        for (uint32_t i = 0; i <= S; ++i) {
            const uint32_t slice = i < S ? i : s;
            __syncthreads();
            res_load<T>(x, g, c, slice, v);
            res_slice_stats<T>(g, slice, v, sm, n, mean, m2);
            if (threadIdx.x == 0 && i < S) { parts[3 * i] = n; parts[3 * i + 1] = mean; parts[3 * i + 2] = m2; }
        }
    }
    __syncthreads();
    if (threadIdx.x < kWave) {
        merge_stat_partials(S, [&](uint32_t i, int k) { return parts[3 * i + k]; }, n, mean, m2);
        if (threadIdx.x == 0) {
            float sc, sh;
            BnFwdParams q = prm;
            if (s != 0) { q.save_mean = nullptr; q.save_invstd = nullptr; q.rmean_out = nullptr; }  // slice 0 writes
            bn_fwd_channel_results<T>(q, c, mean, m2, nullptr, nullptr, sc, sh);
            bc[0] = sc;
            bc[1] = sh;
        }
    }
    __syncthreads();
    const float sc = bc[0], sh = bc[1];
    const uint32_t q0 = s * g.chunk, q1 = min(q0 + g.chunk, g.nq);
#pragma unroll
    for (int u = 0; u < kResVecs; ++u) {
        const uint32_t q = q0 + u * kResThreads + threadIdx.x;
        if (q < q1) {
            float f[VEC];
            Vec<T>::unpack(v[u], f);
#pragma unroll
            for (int k = 0; k < VEC; ++k) f[k] = Act<ACT>::f(fmaf(f[k], sc, sh));
            *reinterpret_cast<raw16_t*>(y + g.offset(q, c, VEC)) = Vec<T>::pack(f);
        }
    }
}

// dy of the slice in place of delta (d), slice sums s1 = sum dy, s2 = sum dy * xhat.
template <typename T, int ACT>
__device__ __forceinline__ void res_bwd_slice_sums(const ChanGeom& g, uint32_t slice, raw16_t (&d)[kResVecs],
                                                   const raw16_t (&v)[kResVecs], float mean, float invstd, float sc,
                                                   float sh, float* sm, float& s1, float& s2) {
    constexpr int VEC = Vec<T>::N;
    const uint32_t q0 = slice * g.chunk, q1 = min(q0 + g.chunk, g.nq);
    s1 = 0.0f;
    s2 = 0.0f;
#pragma unroll
    for (int u = 0; u < kResVecs; ++u)
        if (q0 + u * kResThreads + threadIdx.x < q1) {
            float fd[VEC], fx[VEC];
            Vec<T>::unpack(d[u], fd);
            Vec<T>::unpack(v[u], fx);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float dy = fd[k];
                if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                    const float pre = fmaf(fx[k], sc, sh);
                    dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
                }
                s1 += dy;
                s2 = fmaf(dy, (fx[k] - mean) * invstd, s2);
            }
        }
    s1 = block_sum(s1, sm);
    s2 = block_sum(s2, sm);
}

template <typename T, int ACT>
__global__ __launch_bounds__(kResThreads, kResPerCu) void bn_bwd_resident_kernel(
    const T* __restrict__ delta, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
    const float* __restrict__ save_mean, const float* __restrict__ save_invstd, T* __restrict__ dx, T* dgamma, T* dbeta,
    uint64_t* words, uint32_t epoch, uint32_t spin_limit, float inv_count, int stats_from_batch, ChanGeom g) {
    constexpr int VEC = Vec<T>::N;
    __shared__ float sm[kResThreads / 64];
    __shared__ float parts[kResMaxSlices * 2];
    __shared__ float bc[3];
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const float mean = save_mean[c], invstd = save_invstd[c];
    const float sc = (gamma ? ld(gamma + c) : 1.0f) * invstd;
    const float sh = fmaf(-mean, sc, beta ? ld(beta + c) : 0.0f);
    raw16_t d[kResVecs], v[kResVecs];
    res_load<T>(delta, g, c, s, d);
    res_load<T>(x, g, c, s, v);
    float s1, s2;
    res_bwd_slice_sums<T, ACT>(g, s, d, v, mean, invstd, sc, sh, sm, s1, s2);
    uint64_t* chan_words = words + (size_t)c * S * 2;
    if (threadIdx.x == 0) {
        publish_tagged(chan_words + 2 * s, s1, epoch);
        publish_tagged(chan_words + 2 * s + 1, s2, epoch);
    }
    if (!collect_tagged(chan_words, 2 * S, epoch, spin_limit, parts)) {
        for (uint32_t i = 0; i <= S; ++i) {   // recompute the peers' sums; own slice last (d, v restored)
            const uint32_t slice = i < S ? i : s;
            __syncthreads();
            res_load<T>(delta, g, c, slice, d);
            res_load<T>(x, g, c, slice, v);
            res_bwd_slice_sums<T, ACT>(g, slice, d, v, mean, invstd, sc, sh, sm, s1, s2);
            if (threadIdx.x == 0 && i < S) { parts[2 * i] = s1; parts[2 * i + 1] = s2; }
        }
    }
    __syncthreads();
    if (threadIdx.x < kWave) {
        float t1 = 0.0f, t2 = 0.0f;
        for (uint32_t i = threadIdx.x; i < S; i += kWave) { t1 += parts[2 * i]; t2 += parts[2 * i + 1]; }
        t1 = wave_sum(t1);
        t2 = wave_sum(t2);
        if (threadIdx.x == 0) {
            float A, B, D;
            bn_bwd_channel_results<T>(c, t1, t2, gamma, invstd, s == 0 ? dgamma : nullptr, s == 0 ? dbeta : nullptr,
                                      inv_count, stats_from_batch, A, B, D);
            bc[0] = A; bc[1] = B; bc[2] = D;
        }
    }
    __syncthreads();
    const float A = bc[0], B = bc[1], D = bc[2];
    const uint32_t q0 = s * g.chunk, q1 = min(q0 + g.chunk, g.nq);
#pragma unroll
    for (int u = 0; u < kResVecs; ++u) {
        const uint32_t q = q0 + u * kResThreads + threadIdx.x;
        if (q < q1) {
            float fd[VEC], fx[VEC], o[VEC];
            Vec<T>::unpack(d[u], fd);
            Vec<T>::unpack(v[u], fx);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float dy = fd[k];
                if constexpr (ACT != LUXHIP_ACT_IDENTITY) {
                    const float pre = fmaf(fx[k], sc, sh);
                    dy *= Act<ACT>::d(Act<ACT>::f(pre), pre);
                }
                o[k] = fmaf(A, dy, fmaf(B, fx[k] - mean, D));
            }
            *reinterpret_cast<raw16_t*>(dx + g.offset(q, c, VEC)) = Vec<T>::pack(o);
        }
    }
}

// Workgroups of a resident kernel that one compute unit holds at once (register use decides; the
// exchange between the workgroups of a channel needs all of them on the device together).
static int resident_per_cu(const void* kernel) {
    static std::mutex mu;
    static std::unordered_map<const void*, int> cache;
    std::lock_guard<std::mutex> lk(mu);
    auto it = cache.find(kernel);
    if (it != cache.end()) return it->second;
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, kResThreads, 0) != hipSuccess) n = 0;
    cache[kernel] = n;
    return n;
}

// Slices per channel for the resident path, 0 if the tensor does not qualify.
static int64_t resident_slices(int64_t I, int64_t C, int64_t N, int vec, bool aligned, int per_cu) {
    if (!option_bn_resident() || !aligned || I % vec != 0 || per_cu < 1) return 0;
    const int64_t slots = (int64_t)per_cu * num_cus();
    if (C > slots) return 0;
    const int64_t nq = I * N / vec;
    const int64_t per_wg = (int64_t)kResThreads * kResVecs;
    const int64_t s_need = ceil_div(nq, per_wg);
    // slices: bounded by the resident workgroups, by one polling thread per exchange word and by
    // the exchange area (three 8-byte words per slice)
    const int64_t s_max = std::min<int64_t>({slots / C, (int64_t)kResMaxSlices, (int64_t)(kWorkspaceFlags / 6) / C});
    if (s_need > s_max) return 0;
    // as many slices as fit (more compute units busy) while a slice keeps at least one vector per thread
    int64_t S = std::min<int64_t>(s_max, std::max<int64_t>(s_need, nq / kResThreads));
    if (S < 1) S = 1;
    return S;
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
    const bool upd = training && rmean != nullptr;
    BnFwdParams prm;
    prm.gamma = gamma; prm.beta = beta; prm.rmean = rmean; prm.rvar = rvar;
    prm.rmean_out = upd ? rmean_out : nullptr;
    prm.rvar_out = upd ? rvar_out : nullptr;
    prm.save_mean = save_mean; prm.save_invstd = save_invstd;
    prm.count = (float)(I * N); prm.momentum = momentum; prm.eps = eps;

    const void* res_kernel = nullptr;
#define PICK_RES(A) res_kernel = reinterpret_cast<const void*>(&bn_fwd_resident_kernel<T, A>)
    LUX_DISPATCH_ACT(act, PICK_RES);
#undef PICK_RES
    const int64_t SR = batch_stats && !stream_capturing(s) ? resident_slices(I, C, N, V, vec, resident_per_cu(res_kernel)) : 0;
    if (SR > 0) {
        ChanGeom g;
        g.nq = (uint32_t)(I * N / V);
        g.vec_per_row = (uint32_t)(I / V);
        g.C = (uint32_t)C;
        g.rowdiv = FastDiv(g.vec_per_row);
        g.chunk = (uint32_t)ceil_div(g.nq, SR);
        const int64_t S = ceil_div(g.nq, g.chunk);
        // sized for the two-pass kernels as well, which the same call takes while a stream records a graph
        // (where the workspace cannot grow): an eager call then prepares the recorded one
        int64_t S2 = 1;
        (void)make_geom(I, C, N, vv, &S2);
        Workspace ws;
        int rc = get_workspace(s, (size_t)C * (2 + 3 * S2) * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        uint64_t* words = reinterpret_cast<uint64_t*>(ws.flags);
        const uint32_t spin = (uint32_t)option_bn_spin_limit();
        dim3 grid((unsigned)S, (unsigned)C);
#define LAUNCH_RES(A) launch_exact(ps, bn_fwd_resident_kernel<T, A>, dim3(grid), dim3(kResThreads), 0, s, x, y, words, ws.epoch, spin, prm, g)
        {
            ProfScope ps("bn_fwd_resident_kernel", s, true);
            LUX_DISPATCH_ACT(act, LAUNCH_RES);
        }
#undef LAUNCH_RES
        LUX_CHECK_LAUNCH();
        return LUXHIP_OK;
    }

    int64_t S = 1;
    ChanGeom g = make_geom(I, C, N, vv, &S);
    Workspace ws;
    int rc = get_workspace(s, (size_t)C * (2 + 3 * S) * sizeof(float), &ws);  // scale, shift, partials
    if (rc != LUXHIP_OK) return rc;
    float* scale = reinterpret_cast<float*>(ws.data);
    float* shift = scale + C;
    float* partial = shift + C;
    if (batch_stats) {
        dim3 grid((unsigned)S, (unsigned)C);
        ProfScope ps("bn_stats_kernel", s);
        if (vec) bn_stats_kernel<T, V><<<grid, kBnThreads, 0, s>>>(x, partial, ws.counters, counter_stride(C), scale, shift, prm, g);
        else bn_stats_kernel<T, 1><<<grid, kBnThreads, 0, s>>>(x, partial, ws.counters, counter_stride(C), scale, shift, prm, g);
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
    const float inv_count = 1.0f / (float)(I * N);

    const void* res_kernel = nullptr;
#define PICK_RES(A) res_kernel = reinterpret_cast<const void*>(&bn_bwd_resident_kernel<T, A>)
    LUX_DISPATCH_ACT(act, PICK_RES);
#undef PICK_RES
    const int64_t SR = stream_capturing(s) ? 0 : resident_slices(I, C, N, V, vec, resident_per_cu(res_kernel));
    if (SR > 0) {
        ChanGeom g;
        g.nq = (uint32_t)(I * N / V);
        g.vec_per_row = (uint32_t)(I / V);
        g.C = (uint32_t)C;
        g.rowdiv = FastDiv(g.vec_per_row);
        g.chunk = (uint32_t)ceil_div(g.nq, SR);
        const int64_t S = ceil_div(g.nq, g.chunk);
        int64_t S2 = 1;                      // the two-pass kernels' share, as in the forward pass
        (void)make_geom(I, C, N, vv, &S2);
        Workspace ws;
        int rc = get_workspace(s, (size_t)C * (3 + 2 * S2) * sizeof(float), &ws);
        if (rc != LUXHIP_OK) return rc;
        uint64_t* words = reinterpret_cast<uint64_t*>(ws.flags);
        const uint32_t spin = (uint32_t)option_bn_spin_limit();
        dim3 grid((unsigned)S, (unsigned)C);
#define LAUNCH_RES(A)                                                                                               \
    launch_exact(ps, bn_bwd_resident_kernel<T, A>, dim3(grid), dim3(kResThreads), 0, s, delta, x, gamma, beta, save_mean, save_invstd, dx, dgamma, dbeta, \
                                                              words, ws.epoch, spin, inv_count, stats_from_batch, g)
        {
            ProfScope ps("bn_bwd_resident_kernel", s, true);
            LUX_DISPATCH_ACT(act, LAUNCH_RES);
        }
#undef LAUNCH_RES
        LUX_CHECK_LAUNCH();
        return LUXHIP_OK;
    }

    int64_t S = 1;
    ChanGeom g = make_geom(I, C, N, vv, &S);
    Workspace ws;
    int rc = get_workspace(s, (size_t)C * (3 + 2 * S) * sizeof(float), &ws);
    if (rc != LUXHIP_OK) return rc;
    float* coef = reinterpret_cast<float*>(ws.data);
    float* partial = coef + 3 * C;
    dim3 grid((unsigned)S, (unsigned)C);
    const uint32_t tv = (uint32_t)(I * C * N / vv);
    const FastDiv rowdiv((uint32_t)(I / vv)), cdiv((uint32_t)C);
#define LAUNCH_REDUCE(A)                                                                                            \
    do {                                                                                                            \
        if (vec) bn_bwd_reduce_kernel<T, A, V><<<grid, kBnThreads, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, partial, ws.counters, counter_stride(C), dgamma, dbeta, coef, inv_count, stats_from_batch, g); \
        else bn_bwd_reduce_kernel<T, A, 1><<<grid, kBnThreads, 0, s>>>(delta, x, gamma, beta, save_mean, save_invstd, partial, ws.counters, counter_stride(C), dgamma, dbeta, coef, inv_count, stats_from_batch, g);     \
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
    if (I * C * N == 0) {   // nothing to read: the parameter gradients are empty sums
        const size_t bytes = (size_t)C * (dtype == LUXHIP_F32 ? 4 : 2);
        if (C > 0 && dgamma) { rc = luxhip_fill_zero(dgamma, bytes, s); if (rc) return rc; }
        if (C > 0 && dbeta) { rc = luxhip_fill_zero(dbeta, bytes, s); if (rc) return rc; }
        return LUXHIP_OK;
    }
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
