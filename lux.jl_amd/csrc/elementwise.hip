// bias_activation forward / pullback: HBM-bound streaming kernels.
//
// Tensor view: (I, C, N) column-major; element (i, c, n) lives at (n*C + c)*I + i.
// Two reduction layouts for dbias[c] = sum_{i,n} dx[i,c,n]:
//   "channel": workgroup (s, c) streams a slice of channel c's I*N elements (rows of I
//              contiguous elements) -- used when rows are long enough to coalesce;
//   "plane":   the I*C elements of one n are contiguous; a thread owns VEC consecutive plane
//              positions and walks over n -- used when I is small (dense layers: I == 1).
// Reductions are deterministic: per-workgroup partials are combined in a fixed order by a
// small finalize kernel.
#include <algorithm>

#include "common.h"
#include "act_vec.h"

namespace luxhip {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;  // 16-byte vectors per thread; all of a thread's loads are issued before the first use

// ------------------------------------------------------------------------------- forward
template <typename T, int ACT, int VEC, bool HAS_BIAS, bool WRITE_PRE>
__global__ __launch_bounds__(kThreads) void bias_act_fwd_kernel(const T* __restrict__ x, const T* __restrict__ bias,
                                                                T* y, T* pre, uint32_t total_vec, FastDiv rowdiv,
                                                                FastDiv cdiv, uint32_t C) {
    // rowdiv divides a vector index by the number of vectors per row (I / VEC)
    for (uint32_t base = blockIdx.x * (kThreads * kUnroll); base < total_vec; base += gridDim.x * (kThreads * kUnroll)) {
        float v[kUnroll][VEC];
        uint32_t idx[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            idx[u] = base + u * kThreads + threadIdx.x;
            const uint32_t li = min(idx[u], total_vec - 1);      // past the end: last vector again (ignored below)
            if constexpr (VEC == 1) v[u][0] = ld(x + li);
            else Vec<T>::load(x + (size_t)li * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (idx[u] < total_vec) {
                float b = 0.0f;
                if constexpr (HAS_BIAS) {
                    uint32_t row = rowdiv.div(idx[u]);
                    uint32_t c = row - cdiv.div(row) * C;
                    b = ld(bias + c);
                }
                float p[VEC], o[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    p[k] = v[u][k] + b;
                    o[k] = Act<ACT>::f(p[k]);
                }
                if constexpr (VEC == 1) {
                    if constexpr (WRITE_PRE) st(pre + idx[u], p[0]);
                    st(y + idx[u], o[0]);
                } else {
                    if constexpr (WRITE_PRE) Vec<T>::store(pre + (size_t)idx[u] * VEC, p);
                    Vec<T>::store(y + (size_t)idx[u] * VEC, o);
                }
            }
        }
    }
}

// Plane layout with the bias varying inside a vector (I < VEC, e.g. dense layers where
// I == 1): element e of the flat tensor belongs to channel (e / I) % C.
template <typename T, int ACT, int VEC, bool WRITE_PRE>
__global__ __launch_bounds__(kThreads) void bias_act_fwd_smallI_kernel(const T* __restrict__ x,
                                                                       const T* __restrict__ bias, T* y, T* pre,
                                                                       uint32_t total_vec, FastDiv idiv, FastDiv cdiv,
                                                                       uint32_t C) {
    for (uint32_t base = blockIdx.x * (kThreads * kUnroll); base < total_vec; base += gridDim.x * (kThreads * kUnroll)) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            uint32_t idx = base + u * kThreads + threadIdx.x;
            if (idx < total_vec) {
                float v[VEC], p[VEC], o[VEC];
                Vec<T>::load(x + (size_t)idx * VEC, v);
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    uint32_t row = idiv.div(idx * VEC + k);
                    uint32_t c = row - cdiv.div(row) * C;
                    p[k] = v[k] + ld(bias + c);
                    o[k] = Act<ACT>::f(p[k]);
                }
                if constexpr (WRITE_PRE) Vec<T>::store(pre + (size_t)idx * VEC, p);
                Vec<T>::store(y + (size_t)idx * VEC, o);
            }
        }
    }
}

// ------------------------------------------------------------------------------- pullback
// dx only (no bias gradient): flat streaming.
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kThreads) void act_bwd_kernel(const T* __restrict__ delta, const T* __restrict__ out,
                                                           const T* __restrict__ pre, T* dx, uint32_t total_vec) {
    for (uint32_t base = blockIdx.x * (kThreads * kUnroll); base < total_vec; base += gridDim.x * (kThreads * kUnroll)) {
        float r[kUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t li = min(base + u * kThreads + threadIdx.x, total_vec - 1);   // past the end: ignored below
            dx_vec<T, ACT, VEC>(delta, out, pre, (size_t)li * VEC, r[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t idx = base + u * kThreads + threadIdx.x;
            if (idx < total_vec) store_vec<T, VEC>(dx, (size_t)idx * VEC, r[u]);
        }
    }
}

constexpr int kChanVecs = 4;   // vectors per thread of the channel-layout pullback

// "channel" layout: grid (S, C).  Workgroup (s, c) handles vectors [s*chunk, (s+1)*chunk) of
// the nq = I*N/VEC vectors of channel c and publishes its partial sum; the workgroup of a
// channel that arrives last adds the S partials in index order (same result on every run).
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kThreads) void bias_act_bwd_channel_kernel(const T* __restrict__ delta,
                                                                        const T* __restrict__ out,
                                                                        const T* __restrict__ pre, T* dx, T* dbias,
                                                                        float* partial, uint32_t* counters,
                                                                        uint32_t cstride, uint32_t nq,
                                                                        uint32_t chunk, FastDiv rowdiv,
                                                                        uint32_t vec_per_row, uint32_t C) {
    __shared__ float smem[kThreads / 64];
    __shared__ uint32_t last_flag;
    const uint32_t c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const uint32_t q0 = s * chunk;
    const uint32_t q1 = min(q0 + chunk, nq);
    float acc = 0.0f;
    // Up to kChanVecs vectors per thread (the usual split): all loads in flight together, and the
    // partial sum is handed over before dx is stored, so the hand-off does not wait for the stores.
    const bool single = chunk <= kThreads * kChanVecs;
    float r0[kChanVecs][VEC];
    size_t off0[kChanVecs];
    bool have0[kChanVecs];
    if (single) {
        // all loads of the thread are issued before the first use
#pragma unroll
        for (int u = 0; u < kChanVecs; ++u) {
            const uint32_t q = q0 + u * kThreads + threadIdx.x;
            have0[u] = q < q1;
            const uint32_t qq = have0[u] ? q : q1 - 1;            // past the end: last vector again (ignored)
            const uint32_t n = rowdiv.div(qq);
            off0[u] = ((size_t)qq + (size_t)vec_per_row * ((size_t)n * (C - 1) + c)) * VEC;
        }
#pragma unroll
        for (int u = 0; u < kChanVecs; ++u) dx_vec<T, ACT, VEC>(delta, out, pre, off0[u], r0[u]);
#pragma unroll
        for (int u = 0; u < kChanVecs; ++u)
            if (have0[u]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc += r0[u][k];
            }
    } else {
        for (uint32_t q = q0 + threadIdx.x; q < q1; q += kThreads) {
            const uint32_t n = rowdiv.div(q);
            const size_t off = ((size_t)q + (size_t)vec_per_row * ((size_t)n * (C - 1) + c)) * VEC;
            float r[VEC];
            dx_vec<T, ACT, VEC>(delta, out, pre, off, r);
            if (dx) store_vec<T, VEC>(dx, off, r);
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc += r[k];
        }
    }
    acc = block_sum(acc, smem);
    if (threadIdx.x == 0) {
        publish(partial + (size_t)c * S + s, acc);
        publish_done();
    }
    const bool last = arrive_last(counters + (size_t)c * cstride, S, &last_flag);
    if (single && dx) {
#pragma unroll
        for (int u = 0; u < kChanVecs; ++u)
            if (have0[u]) store_vec<T, VEC>(dx, off0[u], r0[u]);
    }
    if (!last) return;
    if (threadIdx.x < 64) {
        float t = 0.0f;
        for (uint32_t i = threadIdx.x; i < S; i += 64) t += fetch(partial + (size_t)c * S + i);
        t = wave_sum(t);
        if (threadIdx.x == 0) st(dbias + c, t);
    }
}

// "plane" layout: P = I*C contiguous elements per n.  grid (ceil(P/(T*VEC)), S); a thread
// owns VEC consecutive plane positions and sums over the n of its slice.
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kThreads) void bias_act_bwd_plane_kernel(const T* __restrict__ delta,
                                                                      const T* __restrict__ out,
                                                                      const T* __restrict__ pre, T* dx, float* partial,
                                                                      uint32_t P, uint32_t N, uint32_t n_per_slice) {
    const uint32_t p = (blockIdx.x * kThreads + threadIdx.x) * VEC;
    if (p >= P) return;
    const uint32_t n0 = blockIdx.y * n_per_slice, n1 = min(n0 + n_per_slice, N);
    float acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
    // Four n at a time, their loads before the first store: a load behind a store waits for it (a wave's memory
    // operations complete in the order of their issue), so one n per trip pays a store and a load latency per n.
    constexpr uint32_t U = 4;
    uint32_t n = n0;
    for (; n + U <= n1; n += U) {
        float r[U][VEC];
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) dx_vec<T, ACT, VEC>(delta, out, pre, (size_t)(n + u) * P + p, r[u]);
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            if (dx) store_vec<T, VEC>(dx, (size_t)(n + u) * P + p, r[u]);
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] += r[u][k];
        }
    }
    for (; n < n1; ++n) {
        const size_t off = (size_t)n * P + p;
        float r[VEC];
        dx_vec<T, ACT, VEC>(delta, out, pre, off, r);
        if (dx) store_vec<T, VEC>(dx, off, r);
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] += r[k];
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) partial[(size_t)blockIdx.y * P + p + k] = acc[k];
}

// dbias[c] = sum_s sum_{i<I} partial[s][c*I + i]; one wave per channel.
template <typename T>
__global__ __launch_bounds__(64) void plane_finalize_kernel(const float* __restrict__ partial, T* dbias, uint32_t P,
                                                            uint32_t I, uint32_t S) {
    const uint32_t c = blockIdx.x;
    float acc = 0.0f;
    const uint32_t cnt = S * I;
    for (uint32_t t = threadIdx.x; t < cnt; t += 64) {
        const uint32_t s = t / I, i = t - s * I;
        acc += partial[(size_t)s * P + (size_t)c * I + i];
    }
    acc = wave_sum(acc);
    if (threadIdx.x == 0) st(dbias + c, acc);
}

// I == 1 (dense layout): dbias[c] = sum_s partial[s][c] with threads along c.  Workgroup of 64
// channels x 16 slice groups: group g adds slices g, g+16, ...; the group sums are added in order.
template <typename T>
__global__ __launch_bounds__(1024) void plane_finalize_dense_kernel(const float* __restrict__ partial, T* dbias, uint32_t C,
                                                                    uint32_t S) {
    __shared__ float sg[16][64];
    const uint32_t cx = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const uint32_t c = blockIdx.x * 64 + cx;
    float t = 0.0f;
    if (c < C)
        for (uint32_t s = grp; s < S; s += 16) t += partial[(size_t)s * C + c];
    sg[grp][cx] = t;
    __syncthreads();
    if (grp == 0 && c < C) {
        t = 0.0f;
#pragma unroll
        for (int g = 0; g < 16; ++g) t += sg[g][cx];
        st(dbias + c, t);
    }
}

// Dense pullback, bf16, large matrices: dz = delta .* act'(y, pre) (M x N, m contiguous), its transpose dzT (n
// contiguous: the layout in which the weight-gradient product reads it along its contraction index) and the bias
// gradient's partial sums over the 64 columns of a tile, in one pass over delta.  A 64 x 64 tile goes through LDS
// as fp32 (the sums add unrounded values): phase 1 reads 16-byte vectors along m, stores dz and fills the tile;
// phase 2 reads eight n of one m per thread (rows of 65 words: the 64 lanes of a wave hit 64 banks in both phases),
// stores 16 bytes of dzT and adds its eight values; the eight threads of an m add theirs in a fixed order.
// M and N multiples of 64, every pointer 16-byte aligned.  dz may be null (identity: dz is delta), partial may be null.
template <int ACT>
__global__ __launch_bounds__(256) void dense_dz_transposed_kernel(const bf16_t* __restrict__ delta, const bf16_t* __restrict__ out,
                                                                  const bf16_t* __restrict__ pre, bf16_t* dz, bf16_t* __restrict__ dzT,
                                                                  float* __restrict__ partial, uint32_t M, uint32_t N) {
    constexpr int PITCH = 65;
    __shared__ float tile[64 * PITCH];
    const uint32_t m0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
    float r[2][8];
#pragma unroll
    for (int it = 0; it < 2; ++it) {                 // loads first, then the stores
        const uint32_t idx = threadIdx.x + it * 256, nl = idx >> 3, mv = idx & 7;
        dx_vec<bf16_t, ACT, 8>(delta, out, pre, (size_t)(n0 + nl) * M + m0 + mv * 8, r[it]);
    }
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const uint32_t idx = threadIdx.x + it * 256, nl = idx >> 3, mv = idx & 7;
        if (dz != nullptr) store_vec<bf16_t, 8>(dz, (size_t)(n0 + nl) * M + m0 + mv * 8, r[it]);
#pragma unroll
        for (int k = 0; k < 8; ++k) tile[nl * PITCH + mv * 8 + k] = r[it][k];
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const uint32_t idx = threadIdx.x + it * 256, ml = idx >> 3, nv = idx & 7;
        float v[8], sum = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            v[k] = tile[(nv * 8 + k) * PITCH + ml];
            sum += v[k];
        }
        store_vec<bf16_t, 8>(dzT, (size_t)(m0 + ml) * N + n0 + nv * 8, v);
        if (partial != nullptr) {
            // the eight threads of this m are neighbouring lanes: (((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7)))
            sum += __shfl_xor(sum, 1);
            sum += __shfl_xor(sum, 2);
            sum += __shfl_xor(sum, 4);
            if (nv == 0) partial[(size_t)blockIdx.y * M + m0 + ml] = sum;
        }
    }
}

static inline unsigned grid_for(uint32_t total_vec) {
    return (unsigned)ceil_div(total_vec, kThreads * kUnroll);
}

template <typename T>
static int bias_act_fwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t N, const T* x, const T* bias, T* y,
                             T* pre) {
    constexpr int V = Vec<T>::N;
    const int64_t total = I * C * N;
    const bool ptr_ok = aligned16(x) && aligned16(y) && (pre == nullptr || aligned16(pre));
    const FastDiv cdiv((uint32_t)C);
#define LAUNCH_FWD(A)                                                                                              \
    do {                                                                                                           \
        if (ptr_ok && I % V == 0) {                                                                                \
            const uint32_t tv = (uint32_t)(total / V);                                                             \
            const FastDiv rowdiv((uint32_t)(I / V));                                                               \
            if (bias && pre)                                                                                       \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, true, true>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else if (bias)                                                                                         \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, true, false>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else if (pre)                                                                                          \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, false, true>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else                                                                                                   \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, false, false>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
        } else if (ptr_ok && bias && total % V == 0) {                                                             \
            const uint32_t tv = (uint32_t)(total / V);                                                             \
            const FastDiv idiv((uint32_t)I);                                                                       \
            if (pre)                                                                                               \
                bias_act_fwd_smallI_kernel<T, A, V, true><<<grid_for(tv), kThreads, 0, s>>>(x, bias, y, pre, tv, idiv, cdiv, (uint32_t)C); \
            else                                                                                                   \
                bias_act_fwd_smallI_kernel<T, A, V, false><<<grid_for(tv), kThreads, 0, s>>>(x, bias, y, pre, tv, idiv, cdiv, (uint32_t)C); \
        } else if (ptr_ok && !bias && total % V == 0) {                                                            \
            const uint32_t tv = (uint32_t)(total / V);                                                             \
            if (pre)                                                                                               \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, false, true>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, cdiv, cdiv, (uint32_t)C); \
            else                                                                                                   \
                launch_exact(ps, bias_act_fwd_kernel<T, A, V, false, false>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, cdiv, cdiv, (uint32_t)C); \
        } else {                                                                                                   \
            const uint32_t tv = (uint32_t)total;                                                                   \
            const FastDiv rowdiv((uint32_t)I);                                                                     \
            if (bias && pre)                                                                                       \
                launch_exact(ps, bias_act_fwd_kernel<T, A, 1, true, true>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else if (bias)                                                                                         \
                launch_exact(ps, bias_act_fwd_kernel<T, A, 1, true, false>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else if (pre)                                                                                          \
                launch_exact(ps, bias_act_fwd_kernel<T, A, 1, false, true>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
            else                                                                                                   \
                launch_exact(ps, bias_act_fwd_kernel<T, A, 1, false, false>, dim3(grid_for(tv)), dim3(kThreads), 0, s, x, bias, y, pre, tv, rowdiv, cdiv, (uint32_t)C); \
        }                                                                                                          \
    } while (0)
    {
        ProfScope ps("bias_act_fwd_kernel", s, true);
        LUX_DISPATCH_ACT(act, LAUNCH_FWD);
    }
#undef LAUNCH_FWD
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// Where the pullback's scratch memory (partial sums, arrival counters) comes from: the stream's
// workspace, which may allocate, or a fixed block handed in by the entry point that allocates nothing.
struct FixedScratch {
    float* partial;
    size_t partial_bytes;
    uint32_t* counters;      // kWorkspaceCounters words, zero
};
static int bwd_scratch(hipStream_t s, const FixedScratch* fixed, size_t bytes, float** partial, uint32_t** counters) {
    if (fixed != nullptr) {
        LUX_INVALID_IF(bytes > fixed->partial_bytes,
                       "bias_activation_bwd_noalloc: this shape needs %zu bytes of scratch memory, the fixed block has %zu", bytes,
                       fixed->partial_bytes);
        *partial = fixed->partial;
        *counters = fixed->counters;
        return LUXHIP_OK;
    }
    Workspace ws;
    int rc = get_workspace(s, bytes, &ws);
    if (rc != LUXHIP_OK) return rc;
    *partial = reinterpret_cast<float*>(ws.data);
    *counters = ws.counters;
    return LUXHIP_OK;
}

template <typename T>
static int bias_act_bwd_impl(hipStream_t s, int act, int64_t I, int64_t C, int64_t N, const T* delta, const T* out,
                             const T* pre, T* dx, T* dbias, const FixedScratch* fixed = nullptr) {
    constexpr int V = Vec<T>::N;
    const int64_t total = I * C * N;
    const bool ptr_ok = aligned16(delta) && aligned16(dx) && (out == nullptr || aligned16(out)) &&
                        (pre == nullptr || aligned16(pre));
    if (dbias == nullptr) {
#define LAUNCH_ACT_BWD(A)                                                                                   \
    do {                                                                                                    \
        if (ptr_ok && total % V == 0) {                                                                     \
            const uint32_t tv = (uint32_t)(total / V);                                                      \
            act_bwd_kernel<T, A, V><<<grid_for(tv), kThreads, 0, s>>>(delta, out, pre, dx, tv);             \
        } else {                                                                                            \
            act_bwd_kernel<T, A, 1><<<grid_for((uint32_t)total), kThreads, 0, s>>>(delta, out, pre, dx, (uint32_t)total); \
        }                                                                                                   \
    } while (0)
        {
            ProfScope ps("act_bwd_kernel", s);
            LUX_DISPATCH_ACT(act, LAUNCH_ACT_BWD);
        }
#undef LAUNCH_ACT_BWD
        LUX_CHECK_LAUNCH();
        return LUXHIP_OK;
    }

    const bool channel_layout = I >= 64 && C <= 65535;
    if (channel_layout) {
        const bool vec = ptr_ok && I % V == 0;
        const int vv = vec ? V : 1;
        const uint32_t nq = (uint32_t)(I * N / vv);
        int64_t S = ceil_div(nq, kThreads * kChanVecs);
        const int64_t smax = std::min<int64_t>(kThreads, std::max<int64_t>(1, 16384 / C));
        if (S > smax) S = smax;
        if (S < 1) S = 1;
        const uint32_t chunk = (uint32_t)ceil_div(nq, S);
        S = ceil_div(nq, chunk);
        float* partial = nullptr;
        uint32_t* counters = nullptr;
        int rc = bwd_scratch(s, fixed, (size_t)C * S * sizeof(float), &partial, &counters);
        if (rc != LUXHIP_OK) return rc;
        const FastDiv rowdiv((uint32_t)(I / vv));
        dim3 grid((unsigned)S, (unsigned)C);
#define LAUNCH_CH(A)                                                                                               \
    do {                                                                                                           \
        if (vec)                                                                                                   \
            launch_exact(ps, bias_act_bwd_channel_kernel<T, A, V>, dim3(grid), dim3(kThreads), 0, s, delta, out, pre, dx, dbias, partial, counters, counter_stride(C), nq, chunk, rowdiv, (uint32_t)(I / vv), (uint32_t)C); \
        else                                                                                                       \
            launch_exact(ps, bias_act_bwd_channel_kernel<T, A, 1>, dim3(grid), dim3(kThreads), 0, s, delta, out, pre, dx, dbias, partial, counters, counter_stride(C), nq, chunk, rowdiv, (uint32_t)(I / vv), (uint32_t)C); \
    } while (0)
        {
            ProfScope ps("bias_act_bwd_channel_kernel", s, true);
            LUX_DISPATCH_ACT(act, LAUNCH_CH);
        }
#undef LAUNCH_CH
        LUX_CHECK_LAUNCH();
        return LUXHIP_OK;
    }

    // plane layout
    const int64_t P = I * C;
    const bool vec = ptr_ok && P % V == 0;
    const int vv = vec ? V : 1;
    const int64_t gx = ceil_div(P, (int64_t)kThreads * vv);
    int64_t S = std::max<int64_t>(1, std::min<int64_t>(ceil_div(N, 8), ceil_div(2048, gx)));
    const uint32_t n_per_slice = (uint32_t)ceil_div(N, S);
    S = ceil_div(N, n_per_slice);
    LUX_UNSUPPORTED_IF(S > 65535, "bias_activation_bwd: batch split too large");
    float* partial = nullptr;
    uint32_t* counters_unused = nullptr;
    int rc = bwd_scratch(s, fixed, (size_t)P * S * sizeof(float), &partial, &counters_unused);
    if (rc != LUXHIP_OK) return rc;
    dim3 grid((unsigned)gx, (unsigned)S);
#define LAUNCH_PL(A)                                                                                               \
    do {                                                                                                           \
        if (vec)                                                                                                   \
            bias_act_bwd_plane_kernel<T, A, V><<<grid, kThreads, 0, s>>>(delta, out, pre, dx, partial, (uint32_t)P, (uint32_t)N, n_per_slice); \
        else                                                                                                       \
            bias_act_bwd_plane_kernel<T, A, 1><<<grid, kThreads, 0, s>>>(delta, out, pre, dx, partial, (uint32_t)P, (uint32_t)N, n_per_slice); \
    } while (0)
    {
        ProfScope ps("bias_act_bwd_plane_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_PL);
    }
#undef LAUNCH_PL
    LUX_CHECK_LAUNCH();
    ProfScope ps2("plane_finalize_kernel", s);
    if (I == 1) plane_finalize_dense_kernel<T><<<(unsigned)ceil_div(C, 64), 1024, 0, s>>>(partial, dbias, (uint32_t)C, (uint32_t)S);
    else plane_finalize_kernel<T><<<(unsigned)C, 64, 0, s>>>(partial, dbias, (uint32_t)P, (uint32_t)I, (uint32_t)S);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

static int check_common(int dtype, int act, int64_t I, int64_t C, int64_t N) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    LUX_INVALID_IF(I < 0 || C < 0 || N < 0, "negative dimension (%lld, %lld, %lld)", (long long)I, (long long)C, (long long)N);
    // 31-bit element indexing inside the kernels
    if (I > 0 && C > 0 && N > 0) {
        const long double tot = (long double)I * (long double)C * (long double)N;
        LUX_UNSUPPORTED_IF(tot >= 2147483648.0L, "tensors of 2^31 or more elements are not supported");
    }
    return LUXHIP_OK;
}

// The dense pullback's first pass when the weight-gradient product wants dz transposed (gemm.hip decides): dz (may be
// NULL for the identity), dzT and, if dbias != NULL, the bias gradient.  `partial`: N / 64 * M floats of scratch.
int dense_dz_transposed(hipStream_t s, int act, int64_t M, int64_t N, const bf16_t* delta, const bf16_t* out, const bf16_t* pre,
                        bf16_t* dz, bf16_t* dzT, float* partial, bf16_t* dbias) {
    LUX_INVALID_IF(M % 64 != 0 || N % 64 != 0 || N / 64 > 65535, "dense_dz_transposed: whole 64 x 64 tiles only");
    const dim3 grid((unsigned)(M / 64), (unsigned)(N / 64));
    float* const part = dbias != nullptr ? partial : nullptr;
#define LAUNCH_DZT(A) dense_dz_transposed_kernel<A><<<grid, 256, 0, s>>>(delta, out, pre, dz, dzT, part, (uint32_t)M, (uint32_t)N)
    {
        ProfScope ps("dense_dz_transposed_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_DZT);
    }
#undef LAUNCH_DZT
    LUX_CHECK_LAUNCH();
    if (dbias != nullptr) {
        ProfScope ps2("plane_finalize_kernel", s);
        plane_finalize_dense_kernel<bf16_t><<<(unsigned)ceil_div(M, 64), 1024, 0, s>>>(partial, dbias, (uint32_t)M, (uint32_t)(N / 64));
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

// Shared with the dense and convolution pullbacks: dx may be NULL (bias gradient only).
int bias_act_bwd_dispatch(hipStream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* delta,
                          const void* out, const void* pre, void* dx, void* dbias) {
    int rc = check_common(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    if (I * C * N == 0) {
        if (dbias != nullptr && C > 0) return luxhip_fill_zero(dbias, (size_t)C * (dtype == LUXHIP_F32 ? 4 : 2), s);
        return LUXHIP_OK;
    }
    if (dx == nullptr && dbias == nullptr) return LUXHIP_OK;
    if (dtype == LUXHIP_F32)
        return bias_act_bwd_impl<float>(s, act, I, C, N, (const float*)delta, (const float*)out, (const float*)pre,
                                        (float*)dx, (float*)dbias);
    return bias_act_bwd_impl<bf16_t>(s, act, I, C, N, (const bf16_t*)delta, (const bf16_t*)out, (const bf16_t*)pre,
                                     (bf16_t*)dx, (bf16_t*)dbias);
}


// Storage conversion fp32 <-> bf16 (round to nearest even), for operands of mixed storage types that
// are promoted before a fused operator and for taking their gradients back.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void convert_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) st(out + i, ld(in + i));
}
// Eight elements per thread with 16-byte accesses on both sides (n a multiple of 8, both pointers 16-byte aligned).
template <typename T, int K>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        Vec<bf16_t>::load(reinterpret_cast<const bf16_t*>(p), v);
    } else {
        float a[4], b[4];
        Vec<float>::load(reinterpret_cast<const float*>(p), a);
        Vec<float>::load(reinterpret_cast<const float*>(p) + 4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
    }
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        Vec<bf16_t>::store(reinterpret_cast<bf16_t*>(p), v);
    } else {
        const float a[4] = {v[0], v[1], v[2], v[3]}, b[4] = {v[4], v[5], v[6], v[7]};
        Vec<float>::store(reinterpret_cast<float*>(p), a);
        Vec<float>::store(reinterpret_cast<float*>(p) + 4, b);
    }
}
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void convert_vec_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t nvec) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (size_t)gridDim.x * 256) {
        float v[8];
        load8<TI, 8>(in + i * 8, v);
        store8<TO>(out + i * 8, v);
    }
}

// ------------------------------------------------------------------------------- scratch of the entry point that allocates nothing
// luxhip_bias_activation_bwd_noalloc keeps its partial sums and arrival counters in this array instead
// of the stream's workspace.  Every device the library runs on holds its own copy for the life of the
// process.  In host code the array's name is only a handle for hipGetSymbolAddress: the device
// address it returns (kept per device in g_noalloc_ptr) is what kernels and fills receive.
constexpr size_t kNoAllocCounterBytes = kWorkspaceCounters * sizeof(uint32_t);    // 256 KiB
constexpr size_t kNoAllocPartialBytes = size_t(2) << 20;                          // 2 MiB of partial sums
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kNoAllocCounterBytes + kNoAllocPartialBytes];
static unsigned char* g_noalloc_ptr[kNoAllocMaxDevices] = {};

// Called by luxhip_init with `device` current.
int noalloc_setup(int device) {
    LUX_INVALID_IF(device < 0 || device >= kNoAllocMaxDevices, "device %d beyond the %d the library keeps scratch blocks for", device,
                   kNoAllocMaxDevices);
    if (g_noalloc_ptr[device] != nullptr) return LUXHIP_OK;
    unsigned char* ptr = nullptr;
    LUX_CHECK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    LUX_INVALID_IF(ptr == nullptr, "hipGetSymbolAddress returned no address for the scratch block");
    g_noalloc_ptr[device] = ptr;
    return LUXHIP_OK;
}

__global__ void fill_zero_words_kernel(uint32_t* p, size_t nwords) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nwords) p[i] = 0u;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_bias_activation_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* x,
                               const void* bias, void* y, void* pre) {
    LUX_REQUIRE_INIT();
    int rc = check_common(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    if (I * C * N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || y == nullptr, "bias_activation_fwd: x and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return bias_act_fwd_impl<float>((hipStream_t)s, act, I, C, N, (const float*)x, (const float*)bias, (float*)y, (float*)pre);
    return bias_act_fwd_impl<bf16_t>((hipStream_t)s, act, I, C, N, (const bf16_t*)x, (const bf16_t*)bias, (bf16_t*)y, (bf16_t*)pre);
}

int luxhip_bias_activation_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                               const void* delta, const void* out, const void* pre, void* dx, void* dbias) {
    LUX_REQUIRE_INIT();
    int rc = check_common(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    if (I * C * N == 0) {
        if (dbias != nullptr && C > 0) return luxhip_fill_zero(dbias, (size_t)C * (dtype == LUXHIP_F32 ? 4 : 2), s);
        return LUXHIP_OK;
    }
    LUX_INVALID_IF(delta == nullptr || dx == nullptr, "bias_activation_bwd: delta and dx must not be NULL");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && !act_needs_pre(act) && out == nullptr,
                   "bias_activation_bwd: activation %d needs `out`", act);
    LUX_INVALID_IF(act_needs_pre(act) && pre == nullptr, "bias_activation_bwd: activation %d needs `pre`", act);
    if (dtype == LUXHIP_F32)
        return bias_act_bwd_impl<float>((hipStream_t)s, act, I, C, N, (const float*)delta, (const float*)out,
                                        (const float*)pre, (float*)dx, (float*)dbias);
    return bias_act_bwd_impl<bf16_t>((hipStream_t)s, act, I, C, N, (const bf16_t*)delta, (const bf16_t*)out,
                                     (const bf16_t*)pre, (bf16_t*)dx, (bf16_t*)dbias);
}

int luxhip_bias_activation_bwd_noalloc(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                                       const void* delta, const void* out, const void* pre, void* dx, void* dbias) {
    LUX_REQUIRE_INIT();
    int rc = check_common(dtype, act, I, C, N);
    if (rc != LUXHIP_OK) return rc;
    int device = -1;
    LUX_CHECK_HIP(hipGetDevice(&device));
    unsigned char* const block = (device >= 0 && device < kNoAllocMaxDevices) ? g_noalloc_ptr[device] : nullptr;
    LUX_INVALID_IF(block == nullptr, "bias_activation_bwd_noalloc: no scratch block on device %d (luxhip_init sets it up)", device);
    if (I * C * N == 0) {
        if (dbias != nullptr && C > 0) return luxhip_fill_zero(dbias, (size_t)C * (dtype == LUXHIP_F32 ? 4 : 2), s);
        return LUXHIP_OK;
    }
    LUX_INVALID_IF(delta == nullptr || dx == nullptr, "bias_activation_bwd_noalloc: delta and dx must not be NULL");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && !act_needs_pre(act) && out == nullptr,
                   "bias_activation_bwd_noalloc: activation %d needs `out`", act);
    LUX_INVALID_IF(act_needs_pre(act) && pre == nullptr, "bias_activation_bwd_noalloc: activation %d needs `pre`", act);
    FixedScratch fx;
    fx.counters = reinterpret_cast<uint32_t*>(block);
    fx.partial = reinterpret_cast<float*>(block + kNoAllocCounterBytes);
    fx.partial_bytes = kNoAllocPartialBytes;
    if (dbias != nullptr) {
        // the block keeps what the last call left: the arrival counters this call uses start at zero (a fill
        // kernel, which a recording stream can hold, unlike a memset node)
        const size_t words = std::min<size_t>((size_t)C * counter_stride(C), kWorkspaceCounters);
        fill_zero_words_kernel<<<dim3((unsigned)ceil_div((int64_t)words, 256)), dim3(256), 0, (hipStream_t)s>>>(fx.counters, words);
        LUX_CHECK_LAUNCH();
    }
    if (dtype == LUXHIP_F32)
        return bias_act_bwd_impl<float>((hipStream_t)s, act, I, C, N, (const float*)delta, (const float*)out, (const float*)pre,
                                        (float*)dx, (float*)dbias, &fx);
    return bias_act_bwd_impl<bf16_t>((hipStream_t)s, act, I, C, N, (const bf16_t*)delta, (const bf16_t*)out, (const bf16_t*)pre,
                                     (bf16_t*)dx, (bf16_t*)dbias, &fx);
}

int luxhip_convert(luxhip_stream_t s, int dtype_in, int dtype_out, int64_t n, const void* in, void* out) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF((dtype_in != LUXHIP_F32 && dtype_in != LUXHIP_BF16) || (dtype_out != LUXHIP_F32 && dtype_out != LUXHIP_BF16),
                       "convert: unsupported dtype %d -> %d", dtype_in, dtype_out);
    LUX_INVALID_IF(n < 0, "convert: negative length");
    if (n == 0) return LUXHIP_OK;
    LUX_INVALID_IF(in == nullptr || out == nullptr, "convert: in and out must not be NULL");
    const unsigned blocks = (unsigned)std::min<int64_t>((n + 255) / 256, 65535 * 8);
    const hipStream_t st_ = (hipStream_t)s;
    ProfScope ps("convert_kernel", st_);
    if (dtype_in == dtype_out)
        return luxhip_memcpy_d2d(out, in, (size_t)n * (dtype_in == LUXHIP_F32 ? 4 : 2), s);
    if (n % 8 == 0 && aligned16(in) && aligned16(out)) {
        const unsigned vblocks = (unsigned)std::min<int64_t>((n / 8 + 255) / 256, 65535 * 8);
        if (dtype_in == LUXHIP_BF16)
            convert_vec_kernel<bf16_t, float><<<vblocks, 256, 0, st_>>>((const bf16_t*)in, (float*)out, (size_t)(n / 8));
        else
            convert_vec_kernel<float, bf16_t><<<vblocks, 256, 0, st_>>>((const float*)in, (bf16_t*)out, (size_t)(n / 8));
    } else if (dtype_in == LUXHIP_BF16)
        convert_kernel<bf16_t, float><<<blocks, 256, 0, st_>>>((const bf16_t*)in, (float*)out, (size_t)n);
    else
        convert_kernel<float, bf16_t><<<blocks, 256, 0, st_>>>((const float*)in, (bf16_t*)out, (size_t)n);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

}  // extern "C"
