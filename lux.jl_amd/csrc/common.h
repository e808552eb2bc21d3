// Shared host + device helpers of libluxhip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "../../include/luxhip.h"

namespace luxhip {

// ----------------------------------------------------------------------------- host side
int set_error(int status, const char* fmt, ...);
bool initialized();
int num_cus();
// Tuning switches set through luxhip_set_option (defaults in runtime.hip).
int64_t option_bn_resident();     // 1: single-pass batchnorm kernels for tensors that fit the register file
int64_t option_bn_spin_limit();   // polls before a resident workgroup stops waiting for its peers
int64_t option_gemm_tile();       // 0 automatic, else 82 | 42 | 22 | 11
int64_t option_gemm_pretranspose();   // 1: large M/N-major bf16 operands are copied into the K-major layout first
int64_t option_conv_tile();       // 0 automatic, else a tile code of the bf16 whole-tap convolution kernels

// Per-stream scratch owned by the library (partial results of the reduction kernels,
// per-channel coefficients).  get_workspace grows it on demand; kernels on one stream are
// ordered, so consecutive operators may share it.
// `counters`: kWorkspaceCounters arrival counters, all zero whenever no kernel of the stream is
// running (the workgroup that arrives last puts its counter back to zero).
// `flags`: kWorkspaceFlags words reserved for the resident kernels' (value, epoch) exchange words;
// `epoch` is a value no earlier call on the stream has used, so the words never need clearing and
// no other kernel writes this memory.
constexpr size_t kWorkspaceCounters = 65536;
constexpr size_t kWorkspaceFlags = 16384;
// Counters of different channels are spread over different cache lines where the channel count
// allows it: arrivals of all channels in one line would queue up behind each other.
inline uint32_t counter_stride(int64_t channels) {
    uint32_t st = 64;
    while (st > 1 && (int64_t)st * channels > (int64_t)kWorkspaceCounters) st >>= 1;
    return st;
}
struct Workspace {
    char* data;  // >= the requested number of bytes, 256-byte aligned
    uint32_t* counters;
    uint32_t* flags;
    uint32_t epoch;
    const void* zeros;   // kWorkspaceZeroBytes bytes that are never written
};
constexpr size_t kWorkspaceZeroBytes = 256;
int get_workspace(hipStream_t s, size_t bytes, Workspace* out);
// True while `s` records into a HIP graph.  Kernels whose arguments carry the workspace epoch (the
// resident batchnorm kernels, the split groupnorm pullback) would find their own tagged words again
// on every replay of the graph, so the operators take their other code paths while a stream captures.
bool stream_capturing(hipStream_t s);

// What a persistent kernel needs to know once per process: its dynamic LDS limit raised and the
// number of its workgroups that the device holds at once.  Host threads may race to the first
// launch of a kernel: std::call_once lets one of them do the set-up while the others wait.
struct ResidentOnce {
    std::once_flag once;
    int resident = 0;        // 0: the set-up failed (`error` says why)
    hipError_t error = hipSuccess;
    template <typename F>
    int get(F&& setup) {     // setup(hipError_t&) -> workgroups resident at once
        std::call_once(once, [&] { resident = setup(error); });
        return resident;
    }
};

// Optional per-kernel timing with HIP events on the launch stream (luxhip_profile_enable).
struct ProfScope {
    const char* name;
    hipStream_t stream;
    bool active;
    // exact scopes (one launch through launch_exact): two events that the dispatch itself signals at its begin
    // and at its end, so the time is the kernel's alone, without the gap between dependent launches; null while
    // the profile is off
    hipEvent_t start = nullptr, stop = nullptr;
    ProfScope(const char* n, hipStream_t s, bool exact = false);
    ~ProfScope();
};

// kernel<<<grid, block, lds, s>>>(args...) of an exact scope
template <typename... KArgs, typename... Args>
inline void launch_exact(const ProfScope& ps, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s, Args&&... args) {
    if (ps.start != nullptr)
        hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, s, ps.start, ps.stop, 0, static_cast<KArgs>(args)...);
    else
        kernel<<<grid, block, lds, s>>>(static_cast<KArgs>(args)...);
}

#define LUX_CHECK_HIP(expr)                                                                     \
    do {                                                                                        \
        hipError_t _e = (expr);                                                                 \
        if (_e != hipSuccess)                                                                   \
            return ::luxhip::set_error(LUXHIP_HIP_ERROR, "%s failed: %s (%s:%d)", #expr,        \
                                       hipGetErrorString(_e), __FILE__, __LINE__);              \
    } while (0)

#define LUX_CHECK_LAUNCH()                                                                      \
    do {                                                                                        \
        hipError_t _e = hipGetLastError();                                                      \
        if (_e != hipSuccess)                                                                   \
            return ::luxhip::set_error(LUXHIP_HIP_ERROR, "kernel launch failed: %s (%s:%d)",    \
                                       hipGetErrorString(_e), __FILE__, __LINE__);              \
    } while (0)

#define LUX_REQUIRE_INIT()                                                                      \
    do {                                                                                        \
        if (!::luxhip::initialized())                                                           \
            return ::luxhip::set_error(LUXHIP_NOT_INITIALIZED, "luxhip_init has not been called"); \
    } while (0)

#define LUX_INVALID_IF(cond, ...)                                                               \
    do {                                                                                        \
        if (cond) return ::luxhip::set_error(LUXHIP_INVALID, __VA_ARGS__);                      \
    } while (0)

#define LUX_UNSUPPORTED_IF(cond, ...)                                                           \
    do {                                                                                        \
        if (cond) return ::luxhip::set_error(LUXHIP_UNSUPPORTED, __VA_ARGS__);                  \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Division of a 31-bit numerator by a fixed divisor with one multiply-high and a shift
// (round-up method of Granlund & Montgomery).  Valid for 0 <= n < 2^31, 1 <= d < 2^31.
struct FastDiv {
    uint32_t d, m, l;
    FastDiv() : d(1), m(0), l(0) {}
    explicit FastDiv(uint32_t div) : d(div) {
        l = 0;
        while ((1ull << l) < div) ++l;
        m = (uint32_t)(((1ull << 32) * ((1ull << l) - div)) / div + 1);
    }
    __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        uint32_t t = __umulhi(n, m);
#else
        uint32_t t = (uint32_t)(((uint64_t)n * m) >> 32);
#endif
        return (t + n) >> l;
    }
};

// ----------------------------------------------------------------------------- storage types
typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
// round to nearest even, NaN stays NaN: v_cvt_pk_bf16_f32 of gfx950
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {   // lo in bits 15:0
    const f32x2_hw v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_hw));
}

typedef uint32_t raw16_t __attribute__((ext_vector_type(4)));   // 16 bytes as they lie in memory

template <typename T>
struct Vec;  // 16-byte vector access
template <>
struct Vec<float> {
    static constexpr int N = 4;
    __device__ __forceinline__ static void unpack(raw16_t r, float (&v)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(r[i]);
    }
    __device__ __forceinline__ static raw16_t pack(const float (&v)[4]) {
        raw16_t r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = __float_as_uint(v[i]);
        return r;
    }
    __device__ __forceinline__ static void load(const float* p, float (&v)[4]) {
        float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    __device__ __forceinline__ static void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct Vec<bf16_t> {
    static constexpr int N = 8;
    __device__ __forceinline__ static void unpack(raw16_t r, float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(r[i] << 16);
            v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ static raw16_t pack(const float (&v)[8]) {
        raw16_t r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = f32x2_to_bf16x2(v[2 * i], v[2 * i + 1]);
        return r;
    }
    __device__ __forceinline__ static void load(const bf16_t* p, float (&v)[8]) {
        uint4 t = *reinterpret_cast<const uint4*>(p);
        uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ static void store(bf16_t* p, const float (&v)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = f32x2_to_bf16x2(v[2 * i], v[2 * i + 1]);
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

template <typename T>
__device__ __forceinline__ float ld(const T* p);

template <>
__device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }
template <typename T>
__device__ __forceinline__ void st(T* p, float v);
template <>
__device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void st<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// A vector kept in registers between the passes: the 16 bytes as they lie in memory (bf16 stays
// packed, which halves the register footprint), or one float for the scalar kernels.
template <typename T, int VEC>
struct Kept {
    using type = raw16_t;
    __device__ __forceinline__ static type load(const T* p, size_t off) { return *reinterpret_cast<const raw16_t*>(p + off); }
    __device__ __forceinline__ static void get(const type& k, float (&v)[VEC]) { Vec<T>::unpack(k, v); }
};
template <typename T>
struct Kept<T, 1> {
    using type = float;
    __device__ __forceinline__ static type load(const T* p, size_t off) { return ld(p + off); }
    __device__ __forceinline__ static void get(const type& k, float (&v)[1]) { v[0] = k; }
};
template <typename T, int VEC>
__device__ __forceinline__ typename Kept<T, VEC>::type keep(const float (&v)[VEC]) {   // the reverse of get()
    if constexpr (VEC == 1) return v[0];
    else return Vec<T>::pack(v);
}

// ----------------------------------------------------------------------------- activations
// value f(x) and the derivative LuxLib multiplies the cotangent by, given the output `o`
// and the pre-activation `x`.
template <int ACT>
struct Act;
// 1 / (1 + e^-x) with the hardware exponential and reciprocal (about 2 ulp each); the argument
// is clamped so that e^-x stays finite
__device__ __forceinline__ float sigmoidf_(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-fmaxf(x, -80.0f)));
}
template <>
struct Act<LUXHIP_ACT_IDENTITY> {
    static constexpr bool needs_pre = false;
    __device__ __forceinline__ static float f(float x) { return x; }
    __device__ __forceinline__ static float d(float, float) { return 1.0f; }
};
template <>
struct Act<LUXHIP_ACT_RELU> {
    static constexpr bool needs_pre = false;
    __device__ __forceinline__ static float f(float x) { return fmaxf(x, 0.0f); }
    __device__ __forceinline__ static float d(float o, float) { return o > 0.0f ? 1.0f : 0.0f; }
};
template <>
struct Act<LUXHIP_ACT_TANH> {
    static constexpr bool needs_pre = false;
    __device__ __forceinline__ static float f(float x) { return tanhf(x); }
    __device__ __forceinline__ static float d(float o, float) { return 1.0f - o * o; }
};
template <>
struct Act<LUXHIP_ACT_SIGMOID> {
    static constexpr bool needs_pre = false;
    __device__ __forceinline__ static float f(float x) { return sigmoidf_(x); }
    __device__ __forceinline__ static float d(float o, float) { return o * (1.0f - o); }
};
template <>
struct Act<LUXHIP_ACT_SWISH> {
    static constexpr bool needs_pre = true;
    __device__ __forceinline__ static float f(float x) { return x * sigmoidf_(x); }
    __device__ __forceinline__ static float d(float o, float x) { return o + sigmoidf_(x) * (1.0f - o); }
};
template <>
struct Act<LUXHIP_ACT_GELU> {
    // 0.5 x (1 + tanh u) with u = sqrt(2/pi) (x + 0.044715 x^3) is x * sigmoid(2u) exactly
    // (1 + tanh u = 2 sigmoid(2u)): no cancellation for negative x, and one exponential plus one
    // reciprocal instead of a tanh.
    static constexpr bool needs_pre = true;
    __device__ __forceinline__ static float f(float x) {
        const float u2 = 1.5957691216057308f * (x + 0.044715f * x * x * x);
        return x * sigmoidf_(u2);
    }
    __device__ __forceinline__ static float d(float, float x) {
        const float x2 = x * x;
        const float u2 = 1.5957691216057308f * (x + 0.044715f * x2 * x);
        const float s = sigmoidf_(u2);
        const float du2 = 1.5957691216057308f * (1.0f + 3.0f * 0.044715f * x2);
        return s + x * s * (1.0f - s) * du2;
    }
};
template <>
struct Act<LUXHIP_ACT_SOFTPLUS> {
    static constexpr bool needs_pre = true;
    __device__ __forceinline__ static float f(float x) { return log1pf(expf(-fabsf(x))) + fmaxf(x, 0.0f); }
    __device__ __forceinline__ static float d(float, float x) { return sigmoidf_(x); }
};
template <>
struct Act<LUXHIP_ACT_LOGSIGMOID> {
    static constexpr bool needs_pre = true;
    __device__ __forceinline__ static float f(float x) { return -(log1pf(expf(-fabsf(x))) + fmaxf(-x, 0.0f)); }
    __device__ __forceinline__ static float d(float, float x) { return sigmoidf_(-x); }
};
template <>
struct Act<LUXHIP_ACT_LISHT> {
    static constexpr bool needs_pre = true;
    __device__ __forceinline__ static float f(float x) { return x * tanhf(x); }
    __device__ __forceinline__ static float d(float, float x) {
        float t = tanhf(x);
        return t + x * (1.0f - t * t);
    }
};

inline bool act_needs_pre(int act) {
    return act == LUXHIP_ACT_SWISH || act == LUXHIP_ACT_GELU || act == LUXHIP_ACT_SOFTPLUS ||
           act == LUXHIP_ACT_LOGSIGMOID || act == LUXHIP_ACT_LISHT;
}

// Expands `CALL(ActId)` for the runtime activation id.
#define LUX_DISPATCH_ACT(act, CALL)                                      \
    switch (act) {                                                       \
        case LUXHIP_ACT_IDENTITY: CALL(LUXHIP_ACT_IDENTITY); break;      \
        case LUXHIP_ACT_RELU: CALL(LUXHIP_ACT_RELU); break;              \
        case LUXHIP_ACT_TANH: CALL(LUXHIP_ACT_TANH); break;              \
        case LUXHIP_ACT_SIGMOID: CALL(LUXHIP_ACT_SIGMOID); break;        \
        case LUXHIP_ACT_SWISH: CALL(LUXHIP_ACT_SWISH); break;            \
        case LUXHIP_ACT_GELU: CALL(LUXHIP_ACT_GELU); break;              \
        case LUXHIP_ACT_SOFTPLUS: CALL(LUXHIP_ACT_SOFTPLUS); break;      \
        case LUXHIP_ACT_LOGSIGMOID: CALL(LUXHIP_ACT_LOGSIGMOID); break;  \
        case LUXHIP_ACT_LISHT: CALL(LUXHIP_ACT_LISHT); break;            \
        default: break;                                                  \
    }

// ----------------------------------------------------------------------------- reductions
constexpr int kWave = 64;

// Sum over the 64 lanes of a wave, every lane receives the total.  Data-parallel-primitive
// moves inside the VALU (no trip through the LDS crossbar): butterfly inside each row of 16
// lanes, then the row totals are passed along (row_bcast15, row_bcast31) so that lane 63 holds
// the wave total, which a scalar read broadcasts.  Fixed order: same result on every run.
__device__ __forceinline__ float wave_sum(float v) {
    auto dpp_add = [](float x, auto ctrl, auto row_mask, auto bound) {
        const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value, decltype(row_mask)::value,
                                                  0xF, decltype(bound)::value);
        return x + __int_as_float(t);
    };
    using std::integral_constant;
    v = dpp_add(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}, integral_constant<bool, true>{});    // quad_perm [1,0,3,2]
    v = dpp_add(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}, integral_constant<bool, true>{});    // quad_perm [2,3,0,1]
    v = dpp_add(v, integral_constant<int, 0x141>{}, integral_constant<int, 0xF>{}, integral_constant<bool, true>{});   // row_half_mirror
    v = dpp_add(v, integral_constant<int, 0x140>{}, integral_constant<int, 0xF>{}, integral_constant<bool, true>{});   // row_mirror
    v = dpp_add(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{}, integral_constant<bool, false>{});  // row_bcast15 -> rows 1, 3
    v = dpp_add(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{}, integral_constant<bool, false>{});  // row_bcast31 -> rows 2, 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Sum over the workgroup; every thread receives the total.  `smem` needs blockDim.x/64
// floats; contains a trailing barrier so it can be reused immediately.
__device__ __forceinline__ float block_sum(float v, float* smem) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    if (nw == 1) return v;
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float t = 0.0f;
    for (int i = 0; i < nw; ++i) t += smem[i];
    __syncthreads();
    return t;
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

// ----------------------------------------------------------------------------- cross-workgroup hand-off
// Partial results travel between workgroups through agent-scope atomic stores and loads, which
// go past the per-XCD L2 caches, so no cache-wide release fence (an L2 write-back of everything
// the kernel has stored so far) is needed.  Protocol: every thread that published waits for its
// stores (publish_done), the workgroup synchronises and one thread bumps the arrival counter
// (arrive_last); the workgroup that arrives last reads everybody's values with fetch().
__device__ __forceinline__ void publish(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t fetch(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A float together with the epoch of the call that wrote it, as one 8-byte word: the reader sees
// either an older epoch or the complete pair, so the value needs no separate flag and the writer
// no wait between the two.
__device__ __forceinline__ void publish_tagged(uint64_t* p, float v, uint32_t epoch) {
    __hip_atomic_store(p, ((uint64_t)epoch << 32) | __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t fetch_tagged(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// words[0..nw) -> parts[0..nw) in LDS: thread i polls word i until it carries `epoch`.  False for
// the whole workgroup if any poll ran out of tries (then parts is incomplete).  Needs nw <=
// blockDim.x; contains workgroup barriers.
__device__ __forceinline__ bool collect_tagged(const uint64_t* words, uint32_t nw, uint32_t epoch, uint32_t spin_limit,
                                               float* parts) {
    int failed = 0;
    if (threadIdx.x < nw) {
        uint32_t tries = 0;
        for (;;) {
            const uint64_t wv = fetch_tagged(words + threadIdx.x);
            if ((uint32_t)(wv >> 32) == epoch) { parts[threadIdx.x] = __uint_as_float((uint32_t)wv); break; }
            if (tries++ >= spin_limit) { failed = 1; break; }
            __builtin_amdgcn_s_sleep(2);
        }
    }
    return __syncthreads_or(failed) == 0;
}
__device__ __forceinline__ void publish(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float fetch(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Call after the last publish of a thread and before the workgroup barrier that precedes arrive().
__device__ __forceinline__ void publish_done() {
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}
// True in every thread of the workgroup that arrives last out of `expected`; that workgroup also
// puts the counter back to zero for the next kernel.  `flag` is one word of LDS.  Contains
// workgroup barriers: all threads must call it.
__device__ __forceinline__ bool arrive_last(uint32_t* counter, uint32_t expected, uint32_t* flag) {
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev + 1 == expected;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last ? 1u : 0u;
    }
    __syncthreads();
    return *flag != 0u;
}

}  // namespace luxhip
