// dropout / alpha_dropout: HBM-bound streaming kernels plus the counter-based generator that
// stands in for `rand!(rng, y)`.
//
// Random numbers: Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
// SC'11).  Element e of a tensor takes lane e % 4 of the block with counter
// (offset + e / 4, 0) under the 64-bit key `seed`, so the stream depends only on (seed, offset, e):
// not on the launch shape, the vector width or whether the noise is stored or consumed in
// registers.  A 32-bit word u becomes a uniform value in [0, 1): (u >> 8) 2^-24 for fp32 storage,
// (u >> 24) 2^-8 for bf16 storage (every such value is a bf16 number, so nothing rounds up to 1).
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "common.h"

namespace luxhip {

constexpr int kDropThreads = 256;

struct Philox {
    uint32_t k0, k1;
    uint64_t offset;
    __device__ __forceinline__ void block(uint64_t index, uint32_t (&r)[4]) const {
        const uint64_t ctr = offset + index;
        uint32_t c0 = (uint32_t)ctr, c1 = (uint32_t)(ctr >> 32), c2 = 0, c3 = 0;
        uint32_t a = k0, b = k1;
#pragma unroll
        for (int round = 0; round < 10; ++round) {
            const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
            const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
            const uint32_t n0 = hi1 ^ c1 ^ a, n2 = hi0 ^ c3 ^ b;
            c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
            a += 0x9E3779B9u;
            b += 0xBB67AE85u;
        }
        r[0] = c0; r[1] = c1; r[2] = c2; r[3] = c3;
    }
};

template <typename T>
__device__ __forceinline__ float uniform01(uint32_t u) {
    if constexpr (sizeof(T) == 4) return (float)(u >> 8) * 5.9604644775390625e-8f;       // 2^-24
    else return (float)(u >> 24) * 0.00390625f;                                          // 2^-8
}

// the VEC uniform values of the elements e .. e + VEC - 1 (e a multiple of VEC, VEC 1, 4 or 8)
template <typename T, int VEC>
__device__ __forceinline__ void uniform_vec(const Philox& g, uint64_t e, float (&u)[VEC]) {
    uint32_t r[4];
    if constexpr (VEC == 1) {
        g.block(e >> 2, r);
        u[0] = uniform01<T>(r[e & 3]);
    } else {
#pragma unroll
        for (int q = 0; q < VEC / 4; ++q) {
            g.block((e >> 2) + q, r);
#pragma unroll
            for (int k = 0; k < 4; ++k) u[4 * q + k] = uniform01<T>(r[k]);
        }
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void load_n(const T* p, size_t off, float (&v)[VEC]) {
    if constexpr (VEC == 1) v[0] = ld(p + off);
    else Vec<T>::load(p + off, v);
}
template <typename T, int VEC>
__device__ __forceinline__ void store_n(T* p, size_t off, const float (&v)[VEC]) {
    if constexpr (VEC == 1) st(p + off, v[0]);
    else Vec<T>::store(p + off, v);
}

// MODE 0: out = noise.  MODE 1: mask = (noise > p) invp.  MODE 2: mask as in 1 and y = x mask.
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kDropThreads) void dropout_rng_kernel(Philox g, uint64_t first, uint64_t nvec, float p,
                                                                   float invp, const T* __restrict__ x, T* __restrict__ y,
                                                                   T* __restrict__ out) {
    for (uint64_t i = (uint64_t)blockIdx.x * kDropThreads + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kDropThreads) {
        const uint64_t e = first + i * VEC;
        float xv[VEC], u[VEC], m[VEC];
        if constexpr (MODE == 2) load_n<T, VEC>(x, e, xv);
        uniform_vec<T, VEC>(g, e, u);
#pragma unroll
        for (int k = 0; k < VEC; ++k) m[k] = MODE == 0 ? u[k] : (u[k] > p ? invp : 0.f);
        if (out != nullptr) store_n<T, VEC>(out, e, m);
        if constexpr (MODE == 2) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) xv[k] *= m[k];
            store_n<T, VEC>(y, e, xv);
        }
    }
}

// generate_dropout_mask! on stored noise: y = (y > p) invp
template <typename T, int VEC>
__global__ __launch_bounds__(kDropThreads) void dropout_mask_kernel(uint64_t first, uint64_t nvec, float p, float invp, T* y) {
    for (uint64_t i = (uint64_t)blockIdx.x * kDropThreads + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kDropThreads) {
        float v[VEC];
        load_n<T, VEC>(y, first + i * VEC, v);
#pragma unroll
        for (int k = 0; k < VEC; ++k) v[k] = v[k] > p ? invp : 0.f;
        store_n<T, VEC>(y, first + i * VEC, v);
    }
}

// y = x .* mask with the mask broadcast along the dims where its extent is 1.  The dims are
// collapsed on the host into at most kMaxGroups runs of "kept" / "broadcast" dims.
constexpr int kMaxGroups = 8;
struct BroadcastGeom {
    int groups;
    uint32_t size[kMaxGroups];      // extent of the run in x
    uint32_t mstride[kMaxGroups];   // element stride of the run in the mask (0: broadcast)
};

template <typename T, int VEC>
__global__ __launch_bounds__(kDropThreads) void dropout_mul_kernel(BroadcastGeom g, uint64_t nvec, const T* __restrict__ x,
                                                                   const T* __restrict__ mask, T* __restrict__ y) {
    for (uint64_t i = (uint64_t)blockIdx.x * kDropThreads + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kDropThreads) {
        const uint64_t e = i * VEC;
        uint64_t rest = e, moff = 0;
        for (int k = 0; k < g.groups; ++k) {
            const uint64_t q = rest / g.size[k];
            moff += (rest - q * g.size[k]) * g.mstride[k];
            rest = q;
        }
        float xv[VEC], m[VEC];
        load_n<T, VEC>(x, e, xv);
        if (g.mstride[0] != 0) {
            load_n<T, VEC>(mask, moff, m);           // run 0 is kept: VEC consecutive mask values
        } else {
            const float mv = ld(mask + moff);        // run 0 is broadcast: one value for the vector
#pragma unroll
            for (int k = 0; k < VEC; ++k) m[k] = mv;
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) xv[k] *= m[k];
        store_n<T, VEC>(y, e, xv);
    }
}

// alpha_dropout: y = ifelse(noise > p, x, alpha) A + B; pullback dx = delta (noise > p) A
template <typename T, int VEC, bool BWD>
__global__ __launch_bounds__(kDropThreads) void alpha_dropout_kernel(uint64_t first, uint64_t nvec, const T* __restrict__ noise,
                                                                     float p, const T* __restrict__ x, float alpha, float A,
                                                                     float B, T* __restrict__ y) {
    for (uint64_t i = (uint64_t)blockIdx.x * kDropThreads + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kDropThreads) {
        const uint64_t e = first + i * VEC;
        float nv[VEC], xv[VEC];
        load_n<T, VEC>(noise, e, nv);
        load_n<T, VEC>(x, e, xv);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            if constexpr (BWD) xv[k] = nv[k] > p ? xv[k] * A : 0.f;
            else xv[k] = fmaf(nv[k] > p ? xv[k] : alpha, A, B);
        }
        store_n<T, VEC>(y, e, xv);
    }
}

static inline unsigned drop_grid(uint64_t nvec) {
    return (unsigned)std::min<uint64_t>(ceil_div((int64_t)nvec, kDropThreads), (uint64_t)num_cus() * 32);
}

// Flat launch over n elements: whole 16-byte vectors when every pointer allows it, then a scalar
// launch for the last n % VEC elements (or for everything).
template <typename T, typename Launch>
static int flat_launch(int64_t n, bool aligned, Launch&& launch) {
    constexpr int V = Vec<T>::N;
    const uint64_t nvec = aligned ? (uint64_t)n / V : 0;
    if (nvec > 0) {
        launch(std::integral_constant<int, V>{}, (uint64_t)0, nvec);
        LUX_CHECK_LAUNCH();
    }
    const uint64_t done = nvec * V;
    if (done < (uint64_t)n) {
        launch(std::integral_constant<int, 1>{}, done, (uint64_t)n - done);
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

// round to nearest even to a bf16 value (host side; finite arguments)
static inline float bf16_round_host(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    std::memcpy(&f, &u, 4);
    return f;
}

static inline Philox philox_of(uint64_t seed, uint64_t offset) {
    return Philox{(uint32_t)seed, (uint32_t)(seed >> 32), offset};
}

template <typename T>
static int dropout_rng_impl(hipStream_t s, int mode, int64_t n, uint64_t seed, uint64_t offset, float p, float invp,
                            const T* x, T* y, T* out) {
    const Philox g = philox_of(seed, offset);
    const bool aligned = (out == nullptr || aligned16(out)) && (x == nullptr || aligned16(x)) && (y == nullptr || aligned16(y));
    ProfScope ps(mode == 0 ? "rand_uniform_kernel" : (mode == 1 ? "dropout_make_mask_kernel" : "dropout_fwd_kernel"), s);
    return flat_launch<T>(n, aligned, [&](auto vec, uint64_t first, uint64_t nvec) {
        constexpr int V = decltype(vec)::value;
        if (mode == 0) dropout_rng_kernel<T, V, 0><<<drop_grid(nvec), kDropThreads, 0, s>>>(g, first, nvec, p, invp, x, y, out);
        else if (mode == 1) dropout_rng_kernel<T, V, 1><<<drop_grid(nvec), kDropThreads, 0, s>>>(g, first, nvec, p, invp, x, y, out);
        else dropout_rng_kernel<T, V, 2><<<drop_grid(nvec), kDropThreads, 0, s>>>(g, first, nvec, p, invp, x, y, out);
    });
}

template <typename T>
static int dropout_mul_impl(hipStream_t s, const BroadcastGeom& g, int64_t n, const T* x, const T* mask, T* y) {
    constexpr int V = Vec<T>::N;
    const bool vec_ok = aligned16(x) && aligned16(y) && aligned16(mask) && g.size[0] % V == 0;
    ProfScope ps("dropout_mul_kernel", s);
    if (vec_ok) dropout_mul_kernel<T, V><<<drop_grid((uint64_t)n / V), kDropThreads, 0, s>>>(g, (uint64_t)n / V, x, mask, y);
    else dropout_mul_kernel<T, 1><<<drop_grid((uint64_t)n), kDropThreads, 0, s>>>(g, (uint64_t)n, x, mask, y);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
static int alpha_dropout_impl(hipStream_t s, bool bwd, int64_t n, const T* noise, float p, const T* x, float alpha, float A,
                              float B, T* y) {
    const bool aligned = aligned16(noise) && aligned16(x) && aligned16(y);
    ProfScope ps(bwd ? "alpha_dropout_bwd_kernel" : "alpha_dropout_fwd_kernel", s);
    return flat_launch<T>(n, aligned, [&](auto vec, uint64_t first, uint64_t nvec) {
        constexpr int V = decltype(vec)::value;
        if (bwd) alpha_dropout_kernel<T, V, true><<<drop_grid(nvec), kDropThreads, 0, s>>>(first, nvec, noise, p, x, alpha, A, B, y);
        else alpha_dropout_kernel<T, V, false><<<drop_grid(nvec), kDropThreads, 0, s>>>(first, nvec, noise, p, x, alpha, A, B, y);
    });
}

static int drop_check(int dtype, int64_t n) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(n < 0, "invalid element count");
    return LUXHIP_OK;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_rand_uniform(luxhip_stream_t s, int dtype, int64_t n, uint64_t seed, uint64_t offset, void* out) {
    LUX_REQUIRE_INIT();
    int rc = drop_check(dtype, n);
    if (rc != LUXHIP_OK || n == 0) return rc;
    LUX_INVALID_IF(out == nullptr, "rand_uniform: out must not be NULL");
    if (dtype == LUXHIP_F32)
        return dropout_rng_impl<float>((hipStream_t)s, 0, n, seed, offset, 0.f, 0.f, nullptr, nullptr, (float*)out);
    return dropout_rng_impl<bf16_t>((hipStream_t)s, 0, n, seed, offset, 0.f, 0.f, nullptr, nullptr, (bf16_t*)out);
}

int luxhip_dropout_fwd(luxhip_stream_t s, int dtype, int64_t n, uint64_t seed, uint64_t offset, double p, double invp,
                       const void* x, void* y, void* mask) {
    LUX_REQUIRE_INIT();
    int rc = drop_check(dtype, n);
    if (rc != LUXHIP_OK || n == 0) return rc;
    LUX_INVALID_IF((x == nullptr) != (y == nullptr), "dropout_fwd: x and y must be given together");
    LUX_INVALID_IF(x == nullptr && mask == nullptr, "dropout_fwd: nothing to compute");
    const int mode = x == nullptr ? 1 : 2;
    if (dtype == LUXHIP_F32)
        return dropout_rng_impl<float>((hipStream_t)s, mode, n, seed, offset, (float)p, (float)invp, (const float*)x, (float*)y,
                                       (float*)mask);
    // p and invp act in the storage type, as T(p), T(invp) do in generate_dropout_mask!
    return dropout_rng_impl<bf16_t>((hipStream_t)s, mode, n, seed, offset, bf16_round_host((float)p), bf16_round_host((float)invp),
                                    (const bf16_t*)x, (bf16_t*)y, (bf16_t*)mask);
}

int luxhip_dropout_mask(luxhip_stream_t s, int dtype, int64_t n, double p, double invp, void* noise_to_mask) {
    LUX_REQUIRE_INIT();
    int rc = drop_check(dtype, n);
    if (rc != LUXHIP_OK || n == 0) return rc;
    LUX_INVALID_IF(noise_to_mask == nullptr, "dropout_mask: the array must not be NULL");
    hipStream_t st = (hipStream_t)s;
    ProfScope ps("dropout_mask_kernel", st);
    if (dtype == LUXHIP_F32) {
        float* y = (float*)noise_to_mask;
        const float pf = (float)p, ip = (float)invp;
        return flat_launch<float>(n, aligned16(y), [&](auto vec, uint64_t first, uint64_t nvec) {
            dropout_mask_kernel<float, decltype(vec)::value><<<drop_grid(nvec), kDropThreads, 0, st>>>(first, nvec, pf, ip, y);
        });
    }
    bf16_t* y = (bf16_t*)noise_to_mask;
    const float pf = bf16_round_host((float)p), ip = bf16_round_host((float)invp);
    return flat_launch<bf16_t>(n, aligned16(y), [&](auto vec, uint64_t first, uint64_t nvec) {
        dropout_mask_kernel<bf16_t, decltype(vec)::value><<<drop_grid(nvec), kDropThreads, 0, st>>>(first, nvec, pf, ip, y);
    });
}

int luxhip_dropout_mul(luxhip_stream_t s, int dtype, int ndim, const int64_t* x_shape, const int64_t* mask_shape, const void* x,
                       const void* mask, void* y) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(ndim < 0 || (ndim > 0 && (x_shape == nullptr || mask_shape == nullptr)), "dropout_mul: invalid shapes");
    // collapse neighbouring dims of the same kind (kept / broadcast); dims of extent 1 in x vanish
    BroadcastGeom g{};
    int64_t n = 1, mstride = 1;
    int last_kind = -1;
    for (int d = 0; d < ndim; ++d) {
        const int64_t xs = x_shape[d], ms = mask_shape[d];
        LUX_INVALID_IF(xs < 0 || (ms != xs && ms != 1),
                       "dropout_mul: mask extent %lld does not match x extent %lld in dim %d", (long long)ms, (long long)xs, d + 1);
        n *= xs;
        if (xs == 1) continue;
        const int kind = ms == xs ? 1 : 0;
        if (kind == last_kind) {
            g.size[g.groups - 1] *= (uint32_t)xs;
        } else {
            LUX_UNSUPPORTED_IF(g.groups == kMaxGroups, "dropout_mul: too many broadcast runs");
            g.size[g.groups] = (uint32_t)xs;
            g.mstride[g.groups] = kind ? (uint32_t)mstride : 0u;
            ++g.groups;
            last_kind = kind;
        }
        if (kind) mstride *= xs;
    }
    if (n == 0) return LUXHIP_OK;
    LUX_UNSUPPORTED_IF(n >= 2147483648LL, "tensors of 2^31 or more elements are not supported");
    LUX_INVALID_IF(x == nullptr || mask == nullptr || y == nullptr, "dropout_mul: x, mask and y must not be NULL");
    if (g.groups == 0) {            // a single element
        g.groups = 1;
        g.size[0] = 1;
        g.mstride[0] = 1;
    }
    if (dtype == LUXHIP_F32) return dropout_mul_impl<float>((hipStream_t)s, g, n, (const float*)x, (const float*)mask, (float*)y);
    return dropout_mul_impl<bf16_t>((hipStream_t)s, g, n, (const bf16_t*)x, (const bf16_t*)mask, (bf16_t*)y);
}

int luxhip_alpha_dropout_fwd(luxhip_stream_t s, int dtype, int64_t n, const void* noise, double p, const void* x, double alpha,
                             double A, double B, void* y) {
    LUX_REQUIRE_INIT();
    int rc = drop_check(dtype, n);
    if (rc != LUXHIP_OK || n == 0) return rc;
    LUX_INVALID_IF(noise == nullptr || x == nullptr || y == nullptr, "alpha_dropout_fwd: noise, x and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return alpha_dropout_impl<float>((hipStream_t)s, false, n, (const float*)noise, (float)p, (const float*)x, (float)alpha,
                                         (float)A, (float)B, (float*)y);
    // alpha, A and B act in the storage type (T(A), T(B), T(alpha)); p is compared as given
    return alpha_dropout_impl<bf16_t>((hipStream_t)s, false, n, (const bf16_t*)noise, (float)p, (const bf16_t*)x,
                                      bf16_round_host((float)alpha), bf16_round_host((float)A), bf16_round_host((float)B),
                                      (bf16_t*)y);
}

int luxhip_alpha_dropout_bwd(luxhip_stream_t s, int dtype, int64_t n, const void* noise, double p, const void* delta, double A,
                             void* dx) {
    LUX_REQUIRE_INIT();
    int rc = drop_check(dtype, n);
    if (rc != LUXHIP_OK || n == 0) return rc;
    LUX_INVALID_IF(noise == nullptr || delta == nullptr || dx == nullptr, "alpha_dropout_bwd: noise, delta and dx must not be NULL");
    if (dtype == LUXHIP_F32)
        return alpha_dropout_impl<float>((hipStream_t)s, true, n, (const float*)noise, (float)p, (const float*)delta, 0.f, (float)A,
                                         0.f, (float*)dx);
    return alpha_dropout_impl<bf16_t>((hipStream_t)s, true, n, (const bf16_t*)noise, (float)p, (const bf16_t*)delta, 0.f,
                                      bf16_round_host((float)A), 0.f, (bf16_t*)dx);
}

}  // extern "C"
