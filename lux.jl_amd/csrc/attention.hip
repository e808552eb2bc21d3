// The softmax of scaled_dot_product_attention: scale, additive bias, boolean / causal mask and the
// softmax over the key positions in one pass over the logits, and its pullback.  The two batched
// products around it run on the batched MFMA GEMM.
//
// logits, probs: (S, L, H, B) column-major, S = key positions (softmax axis), L = query positions.
// One wavefront owns one column of S values and keeps it in registers between the passes (16-byte
// accesses when S is a multiple of the vector width, up to 64 * 8 vectors; otherwise scalar accesses,
// up to 64 * 16 values); longer columns are read again per pass (they sit in the cache by then).
#include <algorithm>

#include "common.h"

namespace luxhip {

constexpr int kAttnWaves = 4;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_add(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// TL: type of the logits (T, or float under LUXHIP_BF16_WIDE)
template <typename T, typename TL>
struct SoftmaxCol {
    const TL* x;
    const T* bias;
    const uint8_t* mask;
    float scale;
    int limit;      // positions s > limit are masked (causal); S - 1 otherwise
    __device__ __forceinline__ float logit(int s) const {
        float z = ld(x + s) * scale;
        if (bias) z += ld(bias + s);
        const bool keep = s <= limit && (mask == nullptr || mask[s] != 0);
        return keep ? z : -INFINITY;
    }
};

// NV > 0: the column (S <= 64 NV) is held in registers; NV == 0: any S, re-read per pass
template <typename T, typename TL, int NV>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_softmax_fwd_kernel(const TL* __restrict__ logits, T* __restrict__ probs,
                                                                           int S, int L, int H, int64_t cols, float scale,
                                                                           int causal, const uint8_t* __restrict__ mask,
                                                                           int64_t mask_sh, int64_t mask_sb,
                                                                           const T* __restrict__ bias, int64_t bias_sh,
                                                                           int64_t bias_sb) {
    const int lane = threadIdx.x & 63;
    const int64_t col = (int64_t)blockIdx.x * kAttnWaves + (threadIdx.x >> 6);
    if (col >= cols) return;            // whole wavefronts leave; nothing below synchronises across waves
    const int l = (int)(col % L);
    const int64_t hb = col / L;
    const int h = (int)(hb % H);
    const int64_t b = hb / H;
    SoftmaxCol<T, TL> c;
    c.x = logits + col * S;
    c.bias = bias ? bias + (int64_t)l * S + h * bias_sh + b * bias_sb : nullptr;
    c.mask = mask ? mask + (int64_t)l * S + h * mask_sh + b * mask_sb : nullptr;
    c.scale = scale;
    c.limit = causal ? l : S - 1;       // make_causal_mask: keep key s for query l where s <= l
    T* y = probs + col * S;
    if constexpr (NV > 0) {
        float z[NV];
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int s = lane + 64 * i;
            z[i] = s < S ? c.logit(s) : -INFINITY;
            m = fmaxf(m, z[i]);
        }
        m = wave_max(m);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            z[i] = __expf(z[i] - m);
            sum += z[i];
        }
        const float inv = 1.f / wave_add(sum);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int s = lane + 64 * i;
            if (s < S) st(y + s, z[i] * inv);
        }
    } else {
        float m = -INFINITY;
        for (int s = lane; s < S; s += 64) m = fmaxf(m, c.logit(s));
        m = wave_max(m);
        float sum = 0.f;
        for (int s = lane; s < S; s += 64) sum += __expf(c.logit(s) - m);
        const float inv = 1.f / wave_add(sum);
        for (int s = lane; s < S; s += 64) st(y + s, __expf(c.logit(s) - m) * inv);
    }
}

// dlogits = scale * probs .* (dprobs - sum_s dprobs .* probs)
template <typename T, typename TL, int NV>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_softmax_bwd_kernel(const TL* __restrict__ dprobs,
                                                                           const T* __restrict__ probs, T* __restrict__ dlogits,
                                                                           int S, int L, int causal, int64_t cols, float scale) {
    const int lane = threadIdx.x & 63;
    const int64_t col = (int64_t)blockIdx.x * kAttnWaves + (threadIdx.x >> 6);
    if (col >= cols) return;
    const TL* dy = dprobs + col * S;
    const T* y = probs + col * S;
    T* dx = dlogits + col * S;
    const int limit = causal ? (int)(col % L) : S - 1;      // positions past it: weight 0, cotangent not read
    // causal: zeros are stored up to the end of the 128-block of s that holds the limit (what the
    // products with a triangular structure read); the rest of the column is left untouched
    const int wend = causal ? min(S, ((limit >> 7) + 1) << 7) : S;
    if constexpr (NV > 0) {
        float yv[NV], dv[NV];
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int s = lane + 64 * i;
            const bool in = s < S && s <= limit;
            yv[i] = in ? ld(y + s) : 0.f;
            dv[i] = in ? ld(dy + s) : 0.f;
            dot += yv[i] * dv[i];
        }
        dot = wave_add(dot);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int s = lane + 64 * i;
            if (s < wend) st(dx + s, scale * yv[i] * (dv[i] - dot));
        }
    } else {
        float dot = 0.f;
        for (int s = lane; s < S && s <= limit; s += 64) dot += ld(y + s) * ld(dy + s);
        dot = wave_add(dot);
        for (int s = lane; s < wend; s += 64) st(dx + s, s <= limit ? scale * ld(y + s) * (ld(dy + s) - dot) : 0.f);
    }
}

// The same with 16-byte accesses: lane j owns the vectors j, j + 64, ... of the column
// (S a multiple of the vector width, S <= 64 VEC NVV, every pointer 16-byte aligned).
// A wide tensor is read as VEC values of TL per lane and vector (two 16-byte loads for fp32 beside bf16).
template <typename T, typename TL>
__device__ __forceinline__ void load_wide(const TL* p, float (&v)[Vec<T>::N]) {
    if constexpr (sizeof(TL) == sizeof(T)) {
        Vec<T>::load(reinterpret_cast<const T*>(p), v);
    } else {
        static_assert(Vec<T>::N == 8 && sizeof(TL) == 4, "bf16 storage beside fp32");
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
}

template <typename T, typename TL, int NVV>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_softmax_fwd_vec_kernel(
    const TL* __restrict__ logits, T* __restrict__ probs, int S, int L, int H, int64_t cols, float scale, int causal,
    const uint8_t* __restrict__ mask, int64_t mask_sh, int64_t mask_sb, const T* __restrict__ bias, int64_t bias_sh,
    int64_t bias_sb) {
    constexpr int VEC = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t col = (int64_t)blockIdx.x * kAttnWaves + (threadIdx.x >> 6);
    if (col >= cols) return;
    const int l = (int)(col % L);
    const int64_t hb = col / L;
    const int h = (int)(hb % H);
    const int64_t b = hb / H;
    const TL* x = logits + col * S;
    const T* bp = bias ? bias + (int64_t)l * S + h * bias_sh + b * bias_sb : nullptr;
    const uint8_t* mp = mask ? mask + (int64_t)l * S + h * mask_sh + b * mask_sb : nullptr;
    const int limit = causal ? l : S - 1;
    float z[NVV][VEC];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NVV; ++i) {
        const int s0 = (lane + 64 * i) * VEC;
        if (s0 < S && s0 <= limit) {            // vectors past the causal limit are never read
            load_wide<T, TL>(x + s0, z[i]);
            float bv[VEC];
            if (bp) Vec<T>::load(bp + s0, bv);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float v = z[i][k] * scale;
                if (bp) v += bv[k];
                const bool keep = s0 + k <= limit && (mp == nullptr || mp[s0 + k] != 0);
                z[i][k] = keep ? v : -INFINITY;
                m = fmaxf(m, z[i][k]);
            }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) z[i][k] = -INFINITY;
        }
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NVV; ++i)
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            z[i][k] = __expf(z[i][k] - m);
            sum += z[i][k];
        }
    const float inv = 1.f / wave_add(sum);
    T* y = probs + col * S;
#pragma unroll
    for (int i = 0; i < NVV; ++i) {
        const int s0 = (lane + 64 * i) * VEC;
        if (s0 < S) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) z[i][k] *= inv;
            Vec<T>::store(y + s0, z[i]);
        }
    }
}

template <typename T, typename TL, int NVV>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_softmax_bwd_vec_kernel(const TL* __restrict__ dprobs,
                                                                               const T* __restrict__ probs,
                                                                               T* __restrict__ dlogits, int S, int L, int causal,
                                                                               int64_t cols, float scale) {
    constexpr int VEC = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t col = (int64_t)blockIdx.x * kAttnWaves + (threadIdx.x >> 6);
    if (col >= cols) return;
    const TL* dy = dprobs + col * S;
    const T* y = probs + col * S;
    const int limit = causal ? (int)(col % L) : S - 1;
    const int wend = causal ? min(S, ((limit >> 7) + 1) << 7) : S;       // see attn_softmax_bwd_kernel
    float yv[NVV][VEC], dv[NVV][VEC];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < NVV; ++i) {
        const int s0 = (lane + 64 * i) * VEC;
        if (s0 < S && s0 <= limit) {            // vectors wholly past the limit: weights are 0, nothing is read
            Vec<T>::load(y + s0, yv[i]);
            load_wide<T, TL>(dy + s0, dv[i]);
#pragma unroll
            for (int k = 0; k < VEC; ++k) dot += yv[i][k] * dv[i][k];
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) { yv[i][k] = 0.f; dv[i][k] = 0.f; }
        }
    }
    dot = wave_add(dot);
    T* dx = dlogits + col * S;
#pragma unroll
    for (int i = 0; i < NVV; ++i) {
        const int s0 = (lane + 64 * i) * VEC;
        if (s0 < wend) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) yv[i][k] = scale * yv[i][k] * (dv[i][k] - dot);
            Vec<T>::store(dx + s0, yv[i]);
        }
    }
}

// 16-byte vectors per lane for a column of S values, 0 when the vector kernels do not apply
template <typename T>
static inline int lane_vectors(int64_t S, bool aligned) {
    constexpr int V = Vec<T>::N;
    if (!aligned || S % V != 0) return 0;
    for (int nvv : {1, 2, 4, 8})
        if (S <= (int64_t)64 * V * nvv) return nvv;
    return 0;
}

static inline int cached_vectors(int64_t S) {
    for (int nv : {1, 2, 4, 8, 16})
        if (S <= 64 * nv) return nv;
    return 0;
}

template <typename T, typename TL>
static int softmax_fwd_impl(hipStream_t s, int64_t S, int64_t L, int64_t H, int64_t B, const TL* logits, float scale, int causal,
                            const uint8_t* mask, int64_t mask_sh, int64_t mask_sb, const T* bias, int64_t bias_sh,
                            int64_t bias_sb, T* probs) {
    const int64_t cols = L * H * B;
    const unsigned grid = (unsigned)ceil_div(cols, kAttnWaves);
    ProfScope ps("attn_softmax_fwd_kernel", s);
    const bool aligned = aligned16(logits) && aligned16(probs) && (bias == nullptr || aligned16(bias)) &&
                         (mask == nullptr || (reinterpret_cast<uintptr_t>(mask) & 7u) == 0);
#define LUX_SOFTMAX_FWD_VEC(NVV)                                                                                                \
    attn_softmax_fwd_vec_kernel<T, TL, NVV><<<grid, kAttnWaves * 64, 0, s>>>(logits, probs, (int)S, (int)L, (int)H, cols, scale, causal, \
                                                                         mask, mask_sh, mask_sb, bias, bias_sh, bias_sb)
    switch (lane_vectors<T>(S, aligned)) {
        case 1: LUX_SOFTMAX_FWD_VEC(1); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 2: LUX_SOFTMAX_FWD_VEC(2); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 4: LUX_SOFTMAX_FWD_VEC(4); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 8: LUX_SOFTMAX_FWD_VEC(8); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        default: break;
    }
#undef LUX_SOFTMAX_FWD_VEC
#define LUX_SOFTMAX_FWD(NV)                                                                                                   \
    attn_softmax_fwd_kernel<T, TL, NV><<<grid, kAttnWaves * 64, 0, s>>>(logits, probs, (int)S, (int)L, (int)H, cols, scale, causal, \
                                                                    mask, mask_sh, mask_sb, bias, bias_sh, bias_sb)
    switch (cached_vectors(S)) {
        case 1: LUX_SOFTMAX_FWD(1); break;
        case 2: LUX_SOFTMAX_FWD(2); break;
        case 4: LUX_SOFTMAX_FWD(4); break;
        case 8: LUX_SOFTMAX_FWD(8); break;
        case 16: LUX_SOFTMAX_FWD(16); break;
        default: LUX_SOFTMAX_FWD(0); break;
    }
#undef LUX_SOFTMAX_FWD
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T, typename TL>
static int softmax_bwd_impl(hipStream_t s, int64_t S, int64_t L, int causal, int64_t cols, const TL* dprobs, const T* probs,
                            float scale, T* dlogits) {
    const unsigned grid = (unsigned)ceil_div(cols, kAttnWaves);
    ProfScope ps("attn_softmax_bwd_kernel", s);
#define LUX_SOFTMAX_BWD_VEC(NVV) \
    attn_softmax_bwd_vec_kernel<T, TL, NVV><<<grid, kAttnWaves * 64, 0, s>>>(dprobs, probs, dlogits, (int)S, (int)L, causal, cols, scale)
    switch (lane_vectors<T>(S, aligned16(dprobs) && aligned16(probs) && aligned16(dlogits))) {
        case 1: LUX_SOFTMAX_BWD_VEC(1); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 2: LUX_SOFTMAX_BWD_VEC(2); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 4: LUX_SOFTMAX_BWD_VEC(4); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        case 8: LUX_SOFTMAX_BWD_VEC(8); LUX_CHECK_LAUNCH(); return LUXHIP_OK;
        default: break;
    }
#undef LUX_SOFTMAX_BWD_VEC
#define LUX_SOFTMAX_BWD(NV) attn_softmax_bwd_kernel<T, TL, NV><<<grid, kAttnWaves * 64, 0, s>>>(dprobs, probs, dlogits, (int)S, (int)L, causal, cols, scale)
    switch (cached_vectors(S)) {
        case 1: LUX_SOFTMAX_BWD(1); break;
        case 2: LUX_SOFTMAX_BWD(2); break;
        case 4: LUX_SOFTMAX_BWD(4); break;
        case 8: LUX_SOFTMAX_BWD(8); break;
        case 16: LUX_SOFTMAX_BWD(16); break;
        default: LUX_SOFTMAX_BWD(0); break;
    }
#undef LUX_SOFTMAX_BWD
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

static int softmax_check(int dtype, int64_t S, int64_t cols) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16 && dtype != LUXHIP_BF16_WIDE, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(S < 0 || cols < 0, "invalid dimension");
    LUX_UNSUPPORTED_IF(S >= (1ll << 31) || cols >= (1ll << 33), "attention softmax: dimension too large");
    return LUXHIP_OK;
}

// permutedims of the first three dims (operands whose embedding dim is not the first are brought
// to the (E, H, L, B...) layout and their gradients taken back): one element per thread, lanes
// along the output's first dim.
template <typename U>
__global__ __launch_bounds__(256) void permute3_kernel(const U* __restrict__ in, U* __restrict__ out, uint32_t o1, uint32_t o2,
                                                       uint32_t o3, uint32_t s1, uint32_t s2, uint32_t s3, uint32_t total) {
    const uint32_t block = o1 * o2 * o3;
    for (uint32_t idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += gridDim.x * 256u) {
        const uint32_t o = idx / block, r = idx - o * block;
        const uint32_t i3 = r / (o1 * o2), r2 = r - i3 * (o1 * o2);
        const uint32_t i2 = r2 / o1, i1 = r2 - i2 * o1;
        out[idx] = in[(size_t)o * block + (size_t)i1 * s1 + (size_t)i2 * s2 + (size_t)i3 * s3];
    }
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_attention_softmax_fwd(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t H, int64_t B, const void* logits,
                                 double scale, int causal, const uint8_t* mask, int64_t mask_stride_h, int64_t mask_stride_b,
                                 const void* bias, int64_t bias_stride_h, int64_t bias_stride_b, void* probs) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(L < 0 || H < 0 || B < 0, "invalid dimension");
    int rc = softmax_check(dtype, S, L * H * B);
    if (rc != LUXHIP_OK) return rc;
    if (S * L * H * B == 0) return LUXHIP_OK;
    LUX_INVALID_IF(logits == nullptr || probs == nullptr, "attention_softmax_fwd: logits and probs must not be NULL");
    LUX_INVALID_IF(mask_stride_h < 0 || mask_stride_b < 0 || bias_stride_h < 0 || bias_stride_b < 0, "negative stride");
    LUX_INVALID_IF(causal != 0 && mask != nullptr, "`mask` and `is_causal` cannot both be specified");
    if (dtype == LUXHIP_F32)
        return softmax_fwd_impl<float, float>((hipStream_t)s, S, L, H, B, (const float*)logits, (float)scale, causal, mask, mask_stride_h,
                                              mask_stride_b, (const float*)bias, bias_stride_h, bias_stride_b, (float*)probs);
    if (dtype == LUXHIP_BF16_WIDE)
        return softmax_fwd_impl<bf16_t, float>((hipStream_t)s, S, L, H, B, (const float*)logits, (float)scale, causal, mask,
                                               mask_stride_h, mask_stride_b, (const bf16_t*)bias, bias_stride_h, bias_stride_b,
                                               (bf16_t*)probs);
    return softmax_fwd_impl<bf16_t, bf16_t>((hipStream_t)s, S, L, H, B, (const bf16_t*)logits, (float)scale, causal, mask, mask_stride_h,
                                    mask_stride_b, (const bf16_t*)bias, bias_stride_h, bias_stride_b, (bf16_t*)probs);
}

int luxhip_attention_softmax_bwd(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t cols, int causal, const void* dprobs,
                                 const void* probs, double scale, void* dlogits) {
    LUX_REQUIRE_INIT();
    int rc = softmax_check(dtype, S, cols);
    if (rc != LUXHIP_OK) return rc;
    LUX_INVALID_IF(L <= 0 && cols > 0, "attention_softmax_bwd: L must be positive");
    if (S * cols == 0) return LUXHIP_OK;
    LUX_INVALID_IF(dprobs == nullptr || probs == nullptr || dlogits == nullptr,
                   "attention_softmax_bwd: dprobs, probs and dlogits must not be NULL");
    if (dtype == LUXHIP_F32)
        return softmax_bwd_impl<float, float>((hipStream_t)s, S, L, causal, cols, (const float*)dprobs, (const float*)probs,
                                              (float)scale, (float*)dlogits);
    if (dtype == LUXHIP_BF16_WIDE)
        return softmax_bwd_impl<bf16_t, float>((hipStream_t)s, S, L, causal, cols, (const float*)dprobs, (const bf16_t*)probs,
                                               (float)scale, (bf16_t*)dlogits);
    return softmax_bwd_impl<bf16_t, bf16_t>((hipStream_t)s, S, L, causal, cols, (const bf16_t*)dprobs, (const bf16_t*)probs, (float)scale,
                                    (bf16_t*)dlogits);
}

int luxhip_permute_leading3(luxhip_stream_t s, int dtype, int64_t d1, int64_t d2, int64_t d3, int64_t outer, int p1, int p2,
                            int p3, const void* in, void* out) {
    LUX_REQUIRE_INIT();
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_INVALID_IF(d1 < 0 || d2 < 0 || d3 < 0 || outer < 0, "permute_leading3: negative dimension");
    LUX_INVALID_IF(p1 < 1 || p1 > 3 || p2 < 1 || p2 > 3 || p3 < 1 || p3 > 3 || p1 == p2 || p1 == p3 || p2 == p3,
                   "permute_leading3: (%d, %d, %d) is not a permutation of 1:3", p1, p2, p3);
    LUX_UNSUPPORTED_IF((long double)d1 * d2 * d3 * std::max<int64_t>(outer, 1) >= 2147483648.0L,
                       "permute_leading3: tensors of 2^31 or more elements are not supported");
    const int64_t total = d1 * d2 * d3 * outer;
    if (total == 0) return LUXHIP_OK;
    LUX_INVALID_IF(in == nullptr || out == nullptr || in == out, "permute_leading3: in and out must be distinct buffers");
    const int64_t d[3] = {d1, d2, d3}, st[3] = {1, d1, d1 * d2};
    const uint32_t o1 = (uint32_t)d[p1 - 1], o2 = (uint32_t)d[p2 - 1], o3 = (uint32_t)d[p3 - 1];
    const uint32_t s1 = (uint32_t)st[p1 - 1], s2 = (uint32_t)st[p2 - 1], s3 = (uint32_t)st[p3 - 1];
    const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 65535 * 16);
    ProfScope ps("permute3_kernel", (hipStream_t)s);
    if (dtype == LUXHIP_F32)
        permute3_kernel<uint32_t><<<blocks, 256, 0, (hipStream_t)s>>>((const uint32_t*)in, (uint32_t*)out, o1, o2, o3, s1, s2, s3, (uint32_t)total);
    else
        permute3_kernel<uint16_t><<<blocks, 256, 0, (hipStream_t)s>>>((const uint16_t*)in, (uint16_t*)out, o1, o2, o3, s1, s2, s3, (uint32_t)total);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

}  // extern "C"
