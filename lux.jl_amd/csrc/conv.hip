// Convolution entry points: layout transforms, filter repacking, launch logic of the
// implicit-GEMM kernels (conv_kernels.h) and the split-K reduction of the filter gradient.
#include <algorithm>

#include "common.h"
#include "act_vec.h"
#include "conv_kernels.h"
#include "conv_patch.h"
#include "conv_wgrad_patch.h"

namespace luxhip {

int bias_act_bwd_dispatch(hipStream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* delta,
                          const void* out, const void* pre, void* dx, void* dbias);   // elementwise.hip

// ----------------------------------------------------------------------------- layout transforms
// in (P, C, N) with p contiguous  ->  out (C, P, N) with c contiguous
template <typename T>
__global__ __launch_bounds__(256) void whcn_to_cwhn_kernel(const T* __restrict__ in, T* __restrict__ out, int P, int C) {
    __shared__ T tile[32][33];
    const int n = blockIdx.z;
    const int p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;       // 32 x 8
    const T* src = in + (size_t)n * C * P;
    T* dst = out + (size_t)n * C * P;
#pragma unroll
    for (int j = 0; j < 32; j += 8) {
        const int c = c0 + ty + j, p = p0 + tx;
        if (c < C && p < P) tile[ty + j][tx] = src[(size_t)c * P + p];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 32; j += 8) {
        const int p = p0 + ty + j, c = c0 + tx;
        if (c < C && p < P) dst[(size_t)p * C + c] = tile[tx][ty + j];
    }
}

// Same transform with 16-byte global accesses on both sides (P and C multiples of the vector
// length, aligned pointers): a 64(p) x 64(c) tile goes through LDS as tile[c][p]; the row pitch
// (66 two-byte or 65 four-byte elements) spreads the strided reads of the second phase over
// the banks.
template <typename T>
__device__ __forceinline__ void whcn_to_cwhn_vec_tile(const T* __restrict__ in, T* __restrict__ out, int P, int C) {
    constexpr int V = 16 / sizeof(T), TP = 64, TC = 64;
    constexpr int PITCH = TP + 4 / sizeof(T);   // 66 (bf16) / 65 (fp32) elements: rows stay 4-byte aligned
    __shared__ __align__(16) T tile[TC * PITCH];
    const int n = blockIdx.z;
    const int p0 = blockIdx.x * TP, c0 = blockIdx.y * TC;
    const T* src = in + (size_t)n * C * P;
    T* dst = out + (size_t)n * C * P;
    // phase 1: vectors along p
    constexpr int VP = TP / V;                       // vectors per tile row
#pragma unroll
    for (int it = 0; it < TC * VP / 256; ++it) {
        const int idx = threadIdx.x + it * 256;
        const int c = idx / VP, pv = idx % VP;
        if (c0 + c < C && p0 + pv * V < P) {
            const raw16_t v = *reinterpret_cast<const raw16_t*>(src + (size_t)(c0 + c) * P + p0 + pv * V);
            uint32_t* row = reinterpret_cast<uint32_t*>(tile + c * PITCH + pv * V);
#pragma unroll
            for (int k = 0; k < 4; ++k) row[k] = v[k];
        }
    }
    __syncthreads();
    // phase 2: vectors along c
    constexpr int VC = TC / V;
#pragma unroll
    for (int it = 0; it < TP * VC / 256; ++it) {
        const int idx = threadIdx.x + it * 256;
        const int pp = idx / VC, cv = idx % VC;
        if (p0 + pp < P && c0 + cv * V < C) {
            raw16_t r;
            T* e = reinterpret_cast<T*>(&r);
#pragma unroll
            for (int k = 0; k < V; ++k) e[k] = tile[(cv * V + k) * PITCH + pp];
            *reinterpret_cast<raw16_t*>(dst + (size_t)(p0 + pp) * C + c0 + cv * V) = r;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void whcn_to_cwhn_vec_kernel(const T* __restrict__ in, T* __restrict__ out, int P, int C) {
    whcn_to_cwhn_vec_tile<T>(in, out, P, C);
}

// wF[(co*T + t)*Cin_g + ci] (fprop, K = T*Cin_g) or wD[((g*Cin_g + ci)*T + t)*Cout_g + col]
// (dgrad, K = T*Cout_g) from w[a + kW*(b + kH*(ci + Cin_g*co))]; tap t = ka + kW*kb with
// a = flip ? ka : kW-1-ka (same for b).
template <typename T>
__device__ __forceinline__ void pack_filter_element(const T* __restrict__ w, T* __restrict__ out, const ConvGeom& g, int for_dgrad, int idx) {
    const int total = g.kW * g.kH * g.Cin_g * g.Cout;
    if (idx >= total) return;
    const int Tt = g.kW * g.kH;
    int co, t, ci;
    if (!for_dgrad) {
        ci = idx % g.Cin_g;
        t = (idx / g.Cin_g) % Tt;
        co = idx / (g.Cin_g * Tt);
    } else {
        const int col = idx % g.Cout_g;
        t = (idx / g.Cout_g) % Tt;
        const int cig = idx / (g.Cout_g * Tt);       // g*Cin_g + ci
        const int grp = cig / g.Cin_g;
        ci = cig - grp * g.Cin_g;
        co = grp * g.Cout_g + col;
    }
    const int ka = t % g.kW, kb = t / g.kW;
    const int a = g.flip ? ka : g.kW - 1 - ka, b = g.flip ? kb : g.kH - 1 - kb;
    out[idx] = w[a + g.kW * (b + g.kH * (ci + g.Cin_g * co))];
}
template <typename T>
__global__ void pack_filter_kernel(const T* __restrict__ w, T* __restrict__ out, ConvGeom g, int for_dgrad) {
    pack_filter_element<T>(w, out, g, for_dgrad, (int)(blockIdx.x * blockDim.x + threadIdx.x));
}
// The layout transform of a tensor and the repacking of the filter in one launch (the filter is a few hundred
// KiB: a launch of its own costs more than the work): the z slices 0 .. N - 1 of the grid transform image n, the
// slices behind them repack 256 filter elements per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void whcn_to_cwhn_pack_kernel(const T* __restrict__ in, T* __restrict__ out, int P, int C, int N,
                                                                const T* __restrict__ w, T* __restrict__ wout, ConvGeom g, int for_dgrad) {
    if ((int)blockIdx.z < N) {
        whcn_to_cwhn_vec_tile<T>(in, out, P, C);
    } else {
        const int block = ((int)(blockIdx.z - N) * (int)gridDim.y + (int)blockIdx.y) * (int)gridDim.x + (int)blockIdx.x;
        pack_filter_element<T>(w, wout, g, for_dgrad, block * 256 + (int)threadIdx.x);
    }
}

// First pass of the fused pullback (bf16; P and C multiples of 8, 16-byte aligned pointers): one pass over delta
// writes dz = delta .* act'(y, pre) as it lies (p contiguous: what the window and the direct filter-gradient kernels
// read), its channel-contiguous copy dzT (what the input-gradient kernels read) and the bias gradient's partial sums,
// where a pass for dz and the bias gradient followed by a transposing copy reads dz once more.  A workgroup walks
// `chunk` tiles of 64 positions x 64 channels of one image; a tile goes through LDS as fp32 (rows of 65 words: the
// 64 lanes of a wave hit 64 banks in both phases).  Phase 1: 16-byte vectors along p, dz stored, per-channel sums
// kept in registers; phase 2: eight channels of one position per thread, 16 bytes of dzT.  The eight threads of a
// channel add their sums in a fixed order; partial[(n * gridDim.x + blockIdx.x) * C + c].  The z slices behind
// the N images repack the filter for the input-gradient kernel (as in whcn_to_cwhn_pack_kernel).
template <int ACT>
__global__ __launch_bounds__(256) void conv_dz_cwhn_pack_kernel(const bf16_t* __restrict__ delta, const bf16_t* __restrict__ y,
                                                                const bf16_t* __restrict__ pre, bf16_t* dz, bf16_t* __restrict__ dzT,
                                                                float* __restrict__ partial, int P, int C, int N, int chunk,
                                                                const bf16_t* __restrict__ w, bf16_t* __restrict__ wout, ConvGeom g) {
    if ((int)blockIdx.z >= N) {
        const int block = ((int)(blockIdx.z - N) * (int)gridDim.y + (int)blockIdx.y) * (int)gridDim.x + (int)blockIdx.x;
        pack_filter_element<bf16_t>(w, wout, g, 1, block * 256 + (int)threadIdx.x);
        return;
    }
    constexpr int PITCH = 65;
    __shared__ float tile[64 * PITCH];
    const int n = blockIdx.z, c0 = blockIdx.y * 64;
    const size_t image = (size_t)n * C * P;
    float bsum[2] = {0.0f, 0.0f};
    const int tiles_p = (P + 63) / 64;
    const int t_end = min(tiles_p, ((int)blockIdx.x + 1) * chunk);
    for (int tp = blockIdx.x * chunk; tp < t_end; ++tp) {
        const int p0 = tp * 64;
        float r[2][8];
        bool ok[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {                 // loads first, then the stores
            const int idx = threadIdx.x + it * 256, cl = idx >> 3, pv = idx & 7;
            ok[it] = c0 + cl < C && p0 + pv * 8 < P;
            if (ok[it]) {
                dx_vec<bf16_t, ACT, 8>(delta, y, pre, image + (size_t)(c0 + cl) * P + p0 + pv * 8, r[it]);
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) r[it][k] = 0.0f;
            }
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = threadIdx.x + it * 256, cl = idx >> 3, pv = idx & 7;
            if (ok[it] && dz != nullptr) store_vec<bf16_t, 8>(dz, image + (size_t)(c0 + cl) * P + p0 + pv * 8, r[it]);
            float t = 0.0f;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                tile[cl * PITCH + pv * 8 + k] = r[it][k];
                t += r[it][k];
            }
            bsum[it] += t;
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = threadIdx.x + it * 256, pl = idx >> 3, cv = idx & 7;
            if (p0 + pl < P && c0 + cv * 8 < C) {
                float v[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) v[k] = tile[(cv * 8 + k) * PITCH + pl];
                store_vec<bf16_t, 8>(dzT, image + (size_t)(p0 + pl) * C + c0 + cv * 8, v);
            }
        }
        __syncthreads();
    }
    if (partial != nullptr) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = threadIdx.x + it * 256, cl = idx >> 3, pv = idx & 7;
            // the eight threads of a channel are neighbouring lanes: (((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7)))
            float t = bsum[it];
            t += __shfl_xor(t, 1);
            t += __shfl_xor(t, 2);
            t += __shfl_xor(t, 4);
            if (pv == 0 && c0 + cl < C) partial[((size_t)n * gridDim.x + blockIdx.x) * C + c0 + cl] = t;
        }
    }
}

// dbias[c] = sum over slices of partial[slice][c]: one workgroup per channel, thread t adds slices t, t + 256, ...;
// the threads' sums are added in a fixed order (within a wave, then the four waves in turn).
// What is left of the bias gradient after conv_dz_cwhn_pack_kernel: `slices` partial sums per channel.  Either a launch of
// its own or extra workgroups of the launch that adds up the filter gradient's partial sums (both are a few microseconds).
struct BiasPartials {
    const float* partial = nullptr;
    bf16_t* dbias = nullptr;
    int C = 0, slices = 0;
};
__device__ __forceinline__ void conv_dbias_finalize_channel(const float* __restrict__ partial, bf16_t* dbias, int C, int S, int c) {
    __shared__ float sw[4];
    float t = 0.0f;
    for (int sl = threadIdx.x; sl < S; sl += 256) t += partial[(size_t)sl * C + c];
    t = wave_sum(t);
    if ((threadIdx.x & 63) == 0) sw[threadIdx.x >> 6] = t;
    __syncthreads();
    if (threadIdx.x == 0) st(dbias + c, ((sw[0] + sw[1]) + sw[2]) + sw[3]);
}
__global__ __launch_bounds__(256) void conv_dbias_finalize_kernel(const float* __restrict__ partial, bf16_t* dbias, int C, int S) {
    conv_dbias_finalize_channel(partial, dbias, C, S, (int)blockIdx.x);
}

// dw[a, b, ci, g*Cout_g + col] = sum over slices of partial[slice][m' = t*Cin_g + ci][col].
// A thread owns 4 consecutive m' (one 16-byte load per slice, eight slices in flight); slices are
// added in order.
template <typename T>
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ partial, T* __restrict__ dw, ConvGeom g,
                                                           int grp, int slices, int reduce_blocks, BiasPartials bp) {
    if ((int)blockIdx.x >= reduce_blocks) {       // workgroups behind the reduction: one channel of the bias gradient each
        conv_dbias_finalize_channel(bp.partial, bp.dbias, bp.C, bp.slices, (int)blockIdx.x - reduce_blocks);
        return;
    }
    const int Mrows = g.kW * g.kH * g.Cin_g;
    const int total = Mrows * g.Cout_g;
    const int idx = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (idx >= total) return;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool vec = (total & 3) == 0;                 // then idx + 3 < total and every slice row is 16-byte aligned
    if (vec) {
        int sl = 0;
        for (; sl + 8 <= slices; sl += 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4*>(partial + (size_t)(sl + u) * total + idx);
#pragma unroll
            for (int u = 0; u < 8; ++u) { acc[0] += v[u].x; acc[1] += v[u].y; acc[2] += v[u].z; acc[3] += v[u].w; }
        }
        for (; sl < slices; ++sl) {
            const float4 v = *reinterpret_cast<const float4*>(partial + (size_t)sl * total + idx);
            acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
        }
    } else {
        for (int sl = 0; sl < slices; ++sl)
            for (int e = 0; e < 4; ++e)
                if (idx + e < total) acc[e] += partial[(size_t)sl * total + idx + e];
    }
    for (int e = 0; e < 4; ++e) {
        const int id = idx + e;
        if (id >= total) break;
        const int m = id % Mrows, col = id / Mrows;
        const int t = m / g.Cin_g, ci = m - t * g.Cin_g;
        const int ka = t % g.kW, kb = t / g.kW;
        const int a = g.flip ? ka : g.kW - 1 - ka, b = g.flip ? kb : g.kH - 1 - kb;
        st(dw + a + g.kW * (b + g.kH * (ci + g.Cin_g * (grp * g.Cout_g + col))), acc[e]);
    }
}

// ----------------------------------------------------------------------------- host helpers
static int make_geom(const luxhip_conv_dims_t* d, ConvGeom* g) {
    LUX_INVALID_IF(d == nullptr, "conv: dims must not be NULL");
    LUX_INVALID_IF(d->W <= 0 || d->H <= 0 || d->Cin <= 0 || d->N < 0 || d->kW <= 0 || d->kH <= 0 || d->Cout <= 0,
                   "conv: non-positive dimension");
    LUX_INVALID_IF(d->stride_w <= 0 || d->stride_h <= 0 || d->dil_w <= 0 || d->dil_h <= 0 || d->groups <= 0,
                   "conv: stride, dilation and groups must be positive");
    LUX_INVALID_IF(d->pad_w_lo < 0 || d->pad_w_hi < 0 || d->pad_h_lo < 0 || d->pad_h_hi < 0, "conv: negative padding");
    LUX_INVALID_IF(d->Cin % d->groups != 0 || d->Cout % d->groups != 0, "conv: channels must be divisible by groups");
    const int64_t ow = (d->W + d->pad_w_lo + d->pad_w_hi - d->dil_w * (d->kW - 1) - 1) / d->stride_w + 1;
    const int64_t oh = (d->H + d->pad_h_lo + d->pad_h_hi - d->dil_h * (d->kH - 1) - 1) / d->stride_h + 1;
    LUX_INVALID_IF(ow <= 0 || oh <= 0, "conv: empty output");
    const long double big = 2147483648.0L;
    LUX_UNSUPPORTED_IF((long double)d->W * d->H * d->Cin * std::max<int64_t>(d->N, 1) >= big ||
                           (long double)ow * oh * d->Cout * std::max<int64_t>(d->N, 1) >= big,
                       "conv: tensors of 2^31 or more elements are not supported");
    g->W = (int)d->W; g->H = (int)d->H; g->Cin = (int)d->Cin; g->N = (int)d->N; g->kW = (int)d->kW; g->kH = (int)d->kH;
    g->Cout = (int)d->Cout; g->OW = (int)ow; g->OH = (int)oh; g->sw = (int)d->stride_w; g->sh = (int)d->stride_h;
    g->pw = (int)d->pad_w_lo; g->ph = (int)d->pad_h_lo; g->dw = (int)d->dil_w; g->dh = (int)d->dil_h;
    g->groups = (int)d->groups; g->Cin_g = (int)(d->Cin / d->groups); g->Cout_g = (int)(d->Cout / d->groups);
    g->flip = d->flipkernel != 0;
    return LUXHIP_OK;
}

static inline size_t align256(size_t b) { return (b + 255) & ~size_t(255); }

template <typename T>
static int transpose_to_cwhn(hipStream_t s, const T* in, T* out, int P, int C, int N) {
    ProfScope ps("whcn_to_cwhn_kernel", s);
    constexpr int V = 16 / (int)sizeof(T);
    const bool vec = P % V == 0 && C % V == 0 && aligned16(in) && aligned16(out);
    const int tile = vec ? 64 : 32;
    dim3 grid((unsigned)ceil_div(P, tile), (unsigned)ceil_div(C, tile), (unsigned)N);
    LUX_UNSUPPORTED_IF(grid.y > 65535 || grid.z > 65535, "conv: too many channels or images for the layout transform");
    if (vec) whcn_to_cwhn_vec_kernel<T><<<grid, 256, 0, s>>>(in, out, P, C);
    else whcn_to_cwhn_kernel<T><<<grid, 256, 0, s>>>(in, out, P, C);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// out (C x P, C contiguous) = transpose of in (P x C, P contiguous); for the GEMM dispatch, which
// turns large operands into the K-major layout its fastest kernel reads
int transpose_matrix_bf16(hipStream_t s, const bf16_t* in, bf16_t* out, int64_t P, int64_t C) {
    LUX_UNSUPPORTED_IF(P >= (1ll << 31) || C >= (1ll << 31), "matrix too large for the layout transform");
    return transpose_to_cwhn<bf16_t>(s, in, out, (int)P, (int)C, 1);
}

template <typename T>
static int pack_filter(hipStream_t s, const T* w, T* out, const ConvGeom& g, int for_dgrad) {
    ProfScope ps("pack_filter_kernel", s);
    const int total = g.kW * g.kH * g.Cin_g * g.Cout;
    pack_filter_kernel<T><<<(unsigned)ceil_div(total, 256), 256, 0, s>>>(w, out, g, for_dgrad);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// transpose_to_cwhn(in -> out) and pack_filter(w -> wout) in one launch where the 16-byte transform applies
template <typename T>
static int transpose_and_pack(hipStream_t s, const T* in, T* out, int P, int C, int N, const T* w, T* wout, const ConvGeom& g, int for_dgrad) {
    constexpr int V = 16 / (int)sizeof(T);
    const bool vec = P % V == 0 && C % V == 0 && aligned16(in) && aligned16(out);
    const int64_t gx = ceil_div(P, 64), gy = ceil_div(C, 64);
    const int64_t pack_blocks = ceil_div((int64_t)g.kW * g.kH * g.Cin_g * g.Cout, 256);
    const int64_t gz = N + ceil_div(pack_blocks, gx * gy);
    if (!vec || N < 1 || gy > 65535 || gz > 65535) {
        int rc = transpose_to_cwhn<T>(s, in, out, P, C, N);
        if (rc != LUXHIP_OK) return rc;
        return pack_filter<T>(s, w, wout, g, for_dgrad);
    }
    ProfScope ps("whcn_to_cwhn_kernel", s);
    whcn_to_cwhn_pack_kernel<T><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), 256, 0, s>>>(in, out, P, C, N, w, wout, g, for_dgrad);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// Tiles of 64 positions that one workgroup of conv_dz_cwhn_pack_kernel walks: as many as leave about four workgroups
// per compute unit, eight at most (each workgroup contributes one slice of partial sums per channel)
static int dz_cwhn_chunk(int P, int C, int N) {
    const int64_t tiles = ceil_div(P, 64) * ceil_div(C, 64) * N;
    return (int)std::min<int64_t>(8, std::max<int64_t>(1, tiles / (4 * (int64_t)std::max(1, num_cus()))));
}
static size_t dz_cwhn_partial_bytes(int P, int C, int N) {
    const int64_t groups = ceil_div(ceil_div(P, 64), dz_cwhn_chunk(P, C, N));
    return align256((size_t)groups * N * C * sizeof(float));
}
static bool dz_cwhn_ok(int P, int C, int N, const void* delta, const void* y, const void* pre, const void* dz, const void* dzT) {
    return P % 8 == 0 && C % 8 == 0 && N >= 1 && aligned16(delta) && aligned16(y) && aligned16(pre) && aligned16(dz) && aligned16(dzT) &&
           ceil_div(C, 64) <= 65535 && N + 4096 <= 65535;
}
// dz (may be NULL for the identity: dz is delta), dzT, the bias gradient (if dbias != NULL) and, if wout != NULL, the filter
// repacked for the input-gradient kernel
static int conv_dz_cwhn_pack(hipStream_t s, int act, const ConvGeom& g, const bf16_t* delta, const bf16_t* y, const bf16_t* pre,
                             bf16_t* dz, bf16_t* dzT, float* partial, bf16_t* dbias, const bf16_t* w, bf16_t* wout, BiasPartials* later) {
    const int P = g.OW * g.OH, C = g.Cout, N = g.N;
    const int chunk = dz_cwhn_chunk(P, C, N);
    const int64_t gx = ceil_div(ceil_div(P, 64), chunk), gy = ceil_div(C, 64);
    const int64_t pack_blocks = wout != nullptr ? ceil_div((int64_t)g.kW * g.kH * g.Cin_g * g.Cout, 256) : 0;
    const int64_t gz = N + ceil_div(pack_blocks, gx * gy);
    LUX_UNSUPPORTED_IF(gz > 65535, "conv: filter too large for the combined layout pass");
    float* const part = dbias != nullptr ? partial : nullptr;
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)gz);
#define LAUNCH_DZC(A) conv_dz_cwhn_pack_kernel<A><<<grid, 256, 0, s>>>(delta, y, pre, dz, dzT, part, P, C, N, chunk, w, wout, g)
    {
        ProfScope ps("conv_dz_cwhn_pack_kernel", s);
        LUX_DISPATCH_ACT(act, LAUNCH_DZC);
    }
#undef LAUNCH_DZC
    LUX_CHECK_LAUNCH();
    if (dbias != nullptr) {
        if (later != nullptr) {           // the caller adds the channels' sums to a later launch
            later->partial = partial; later->dbias = dbias; later->C = C; later->slices = (int)(gx * N);
            return LUXHIP_OK;
        }
        ProfScope ps2("conv_dbias_finalize_kernel", s);
        conv_dbias_finalize_kernel<<<(unsigned)C, 256, 0, s>>>(partial, dbias, C, (int)(gx * N));
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

template <typename T>
static void fill_gather(GatherK<T>& q, const ConvGeom& g, bool dgrad) {
    constexpr int V = GemmTraits<T>::VEC;
    q.kW = g.kW; q.sw = g.sw; q.sh = g.sh; q.pw = g.pw; q.ph = g.ph; q.dw = g.dw; q.dh = g.dh;
    q.dgrad = dgrad;
    if (!dgrad) {            // rows: output positions; source: xT
        q.Ctot = g.Cin; q.Cg = g.Cin_g; q.P = g.OW; q.PQ = g.OW * g.OH; q.SP = g.W; q.SQ = g.H;
    } else {                 // rows: input positions; source: dyT
        q.Ctot = g.Cout; q.Cg = g.Cout_g; q.P = g.W; q.PQ = g.W * g.H; q.SP = g.OW; q.SQ = g.OH;
    }
    q.M = q.PQ * g.N;
    q.divP = FastDiv((uint32_t)q.P); q.divPQ = FastDiv((uint32_t)q.PQ); q.divCg = FastDiv((uint32_t)q.Cg);
    q.divkW = FastDiv((uint32_t)g.kW); q.divsw = FastDiv((uint32_t)g.sw); q.divsh = FastDiv((uint32_t)g.sh);
    q.vec_ok = (q.Cg % V == 0) && (q.Ctot % V == 0);
}

// fprop (dgrad == false): out = y; dgrad: out = dx.  src is the channel-contiguous activation,
// wm the packed filter (all groups), zeros a few zero bytes in device memory.
template <typename T>
static int run_conv_gemm(hipStream_t s, const ConvGeom& g, bool dgrad, const T* src, const T* wm, const T* bias, T* out,
                         T* pre, int act, const void* zeros) {
    const int Tt = g.kW * g.kH;
    const int Cg = dgrad ? g.Cout_g : g.Cin_g;
    const int64_t src_elems = dgrad ? (int64_t)g.OW * g.OH * g.Cout * g.N : (int64_t)g.W * g.H * g.Cin * g.N;
    // whole-tap stages: a K stage never straddles a filter tap; the transposed-convolution index
    // map of dgrad is only that simple for unit stride
    const bool tap_path = Cg % GemmTraits<T>::BK == 0 && (!dgrad || (g.sw == 1 && g.sh == 1)) && aligned16(src) &&
                          aligned16(wm) && src_elems < (int64_t(1) << 30);
    for (int grp = 0; grp < g.groups; ++grp) {
        const int Ncols = dgrad ? g.Cin_g : g.Cout_g;
        const int K = Tt * Cg;
        Operand<T> Wm;
        Wm.p = wm + (size_t)grp * Ncols * K;
        Wm.sr = K; Wm.sk = 1; Wm.rows = Ncols;
        Wm.vec_ok = aligned16(Wm.p) && ((size_t)K * sizeof(T)) % 16 == 0;
        int rc;
        if constexpr (sizeof(T) == 2) {
            // unit stride and dilation, output as large as the input: the kernel that keeps a tile's input window in LDS
            if (option_conv_tile() <= 2 && g.sw == 1 && g.sh == 1 && g.dw == 1 && g.dh == 1 && g.OW == g.W && g.OH == g.H) {
                cpatch::Problem p;
                p.src = reinterpret_cast<const bf16_t*>(src) + (size_t)grp * Cg;
                p.wm = reinterpret_cast<const bf16_t*>(Wm.p);
                p.bias = reinterpret_cast<const bf16_t*>(bias);
                p.out = reinterpret_cast<bf16_t*>(out); p.pre = reinterpret_cast<bf16_t*>(pre); p.zero = zeros;
                p.Ctot = dgrad ? g.Cout : g.Cin; p.Cg = Cg; p.P = g.W; p.Q = g.H; p.N = g.N;
                p.kW = g.kW; p.kH = g.kH; p.pad_w = g.pw; p.pad_h = g.ph; p.dgrad = dgrad;
                p.Ncols = Ncols; p.col_off = grp * Ncols; p.Ctot_out = dgrad ? g.Cin : g.Cout; p.act = act;
                if (cpatch::applicable(p)) {
                    if ((rc = cpatch::launch(s, p)) != LUXHIP_OK) return rc;
                    continue;
                }
            }
        }
        if (tap_path) {
            ConvTapArgs<T> a;
            TapGeom<T>& q = a.tap;
            q.kW = g.kW; q.sw = g.sw; q.sh = g.sh; q.pw = g.pw; q.ph = g.ph; q.dw = g.dw; q.dh = g.dh;
            q.dgrad = dgrad;
            q.Cg = Cg;
            if (!dgrad) { q.Ctot = g.Cin; q.P = g.OW; q.PQ = g.OW * g.OH; q.SP = g.W; q.SQ = g.H; }
            else { q.Ctot = g.Cout; q.P = g.W; q.PQ = g.W * g.H; q.SP = g.OW; q.SQ = g.OH; }
            q.M = q.PQ * g.N;
            q.divP = FastDiv((uint32_t)q.P); q.divPQ = FastDiv((uint32_t)q.PQ); q.divCg = FastDiv((uint32_t)q.Cg);
            q.divkW = FastDiv((uint32_t)g.kW);
            q.src = src + (size_t)grp * Cg;
            q.zero = zeros;
            a.Wm = Wm; a.K = K; a.Ncols = Ncols;
            a.out = out; a.pre = pre; a.bias = bias;
            a.Ctot_out = dgrad ? g.Cin : g.Cout;
            a.col_off = grp * Ncols;
            a.act = act;
            a.m_begin = 0;
            rc = launch_conv_tap_any<T>(s, a);
        } else {
            ConvGemmArgs<T> a;
            fill_gather(a.gather, g, dgrad);
            a.gather.src = src;
            a.gather.c_off = grp * a.gather.Cg;
            a.gather.vec_ok = a.gather.vec_ok && aligned16(src);
            a.K = K; a.Ncols = Ncols; a.Wm = Wm;
            a.out = out; a.pre = pre; a.bias = bias;
            a.Ctot_out = dgrad ? g.Cin : g.Cout;
            a.col_off = grp * a.Ncols;
            a.act = act;
            rc = launch_conv_gemm_any<T>(s, a);
        }
        if (rc != LUXHIP_OK) return rc;
    }
    return LUXHIP_OK;
}

template <typename T>
static int wgrad_plan(const ConvGeom& g, int* slices, int* kslice, bool* small) {
    constexpr int BK = GemmTraits<T>::BK;
    const int Mrows = g.kW * g.kH * g.Cin_g;
    *small = Mrows <= 64 || g.Cout_g <= 64;
    const int tile = *small ? 64 : 128;
    const int64_t tiles = ceil_div(Mrows, tile) * ceil_div(g.Cout_g, tile);
    const int64_t Ktotal = (int64_t)g.OW * g.OH * g.N;
    // as many slices as keep every workgroup resident at once (two per compute unit): one more
    // would add a whole round for a single straggler
    int64_t want = std::max<int64_t>(1, 2 * (int64_t)std::max(1, num_cus()) / (tiles * g.groups));
    int64_t ks = ceil_div(ceil_div(Ktotal, want), BK) * BK;
    ks = std::max<int64_t>(ks, 4 * BK);
    *kslice = (int)ks;
    *slices = (int)ceil_div(Ktotal, ks);
    LUX_UNSUPPORTED_IF(*slices > 65535, "conv wgrad: too many k slices");
    return LUXHIP_OK;
}

// The filter gradient with the tile's input window in LDS (bf16, 3 x 3, unit stride and dilation, output as large
// as the input): one partial sum per image.  Pointer alignment is checked again at the launch.
template <typename T>
static bool wgrad_window_shape(const ConvGeom& g) {
    if (sizeof(T) != 2 || option_conv_tile() > 2) return false;
    if (g.kW != 3 || g.kH != 3 || g.sw != 1 || g.sh != 1 || g.dw != 1 || g.dh != 1 || g.OW != g.W || g.OH != g.H) return false;
    wpatch::Problem p;
    p.src = nullptr; p.dz = nullptr; p.partial = nullptr; p.zero = nullptr;
    p.Ctot = g.Cin; p.Cg = g.Cin_g; p.Cout = g.Cout; p.Ncols = g.Cout_g; p.P = g.W; p.Q = g.H; p.N = g.N; p.pad_w = g.pw; p.pad_h = g.ph;
    return wpatch::applicable(p, num_cus() > 0 ? num_cus() : 256);
}

template <typename T>
static size_t wgrad_partial_bytes(const ConvGeom& g) {
    int slices = 1, kslice = 0;
    bool small = false;
    if (wgrad_plan<T>(g, &slices, &kslice, &small) != LUXHIP_OK) return 0;
    if (wgrad_window_shape<T>(g))
        slices = std::max(slices, wpatch::image_lanes(g.N, (g.Cin_g / 64) * ((g.Cout_g + 63) / 64), num_cus() > 0 ? num_cus() : 256));
    return align256((size_t)slices * g.kW * g.kH * g.Cin_g * g.Cout_g * sizeof(float));
}

// bf16 fast path of the filter gradient: conditions under which conv_wgrad_direct_kernel applies
template <typename T>
static bool wgrad_direct_ok(const ConvGeom& g, const void* xT, const void* dy) {
    if (sizeof(T) != 2) return false;
    const int64_t PQ = (int64_t)g.OW * g.OH;
    return PQ % GemmTraits<T>::BK == 0 && g.Cin_g % 8 == 0 && g.Cin % 8 == 0 && aligned16(xT) && aligned16(dy) &&
           (int64_t)g.W * g.H * g.Cin * g.N < (int64_t(1) << 30) && PQ * g.Cout * g.N < (int64_t(1) << 30);
}

// dy: WHCN cotangent (used by the direct bf16 kernel); dyT: its channel-contiguous copy (used by
// the general kernel; may be NULL when wgrad_direct_ok).
template <typename T>
static int run_wgrad(hipStream_t s, const ConvGeom& g, const T* xT, const T* dy, const T* dyT, float* partial, T* dw,
                     const void* zeros, const BiasPartials* bias = nullptr) {
    constexpr int V = GemmTraits<T>::VEC;
    int slices, kslice;
    bool small;
    int rc = wgrad_plan<T>(g, &slices, &kslice, &small);
    if (rc != LUXHIP_OK) return rc;
    const bool direct = wgrad_direct_ok<T>(g, xT, dy);
    const bool window = wgrad_window_shape<T>(g) && aligned16(xT) && aligned16(dy) && aligned16(partial);
    for (int grp = 0; grp < g.groups; ++grp) {
        const int Mrows = g.kW * g.kH * g.Cin_g;
        if (window) {
            if constexpr (sizeof(T) == 2) {
                wpatch::Problem p;
                p.src = reinterpret_cast<const bf16_t*>(xT) + (size_t)grp * g.Cin_g;
                p.dz = reinterpret_cast<const bf16_t*>(dy) + (size_t)grp * g.Cout_g * g.OW * g.OH;
                p.partial = partial; p.zero = zeros;
                p.Ctot = g.Cin; p.Cg = g.Cin_g; p.Cout = g.Cout; p.Ncols = g.Cout_g;
                p.P = g.W; p.Q = g.H; p.N = g.N; p.pad_w = g.pw; p.pad_h = g.ph;
                rc = wpatch::launch(s, p);
                slices = wpatch::image_lanes(g.N, (g.Cin_g / 64) * ((g.Cout_g + 63) / 64), num_cus() > 0 ? num_cus() : 256);
            }
        } else if (direct) {
            if constexpr (sizeof(T) == 2) {
                ConvWgradDirectArgs a;
                WgradGeomA& q = a.A;
                q.src = reinterpret_cast<const bf16_t*>(xT) + (size_t)grp * g.Cin_g;
                q.zero = zeros;
                q.Ctot = g.Cin; q.Cg = g.Cin_g; q.Mrows = Mrows;
                q.OW = g.OW; q.OWOH = g.OW * g.OH; q.SP = g.W; q.SQ = g.H;
                q.kW = g.kW; q.sw = g.sw; q.sh = g.sh; q.pw = g.pw; q.ph = g.ph; q.dw = g.dw; q.dh = g.dh;
                q.divOW = FastDiv((uint32_t)q.OW); q.divOWOH = FastDiv((uint32_t)q.OWOH);
                q.divCg = FastDiv((uint32_t)q.Cg); q.divkW = FastDiv((uint32_t)g.kW);
                WgradGeomB& b = a.B;
                b.dy = reinterpret_cast<const bf16_t*>(dy);
                b.zero = zeros;
                b.PQ = g.OW * g.OH; b.Cout = g.Cout; b.co_off = grp * g.Cout_g; b.Ncols = g.Cout_g;
                b.divPQ = FastDiv((uint32_t)b.PQ);
                a.Ktotal = g.OW * g.OH * g.N; a.kslice = kslice; a.partial = partial;
                rc = launch_conv_wgrad_direct(s, a, slices);
            }
        } else {
            ConvWgradArgs<T> a;
            GatherMN<T>& q = a.gather;
            q.src = xT; q.Ctot = g.Cin; q.c_off = grp * g.Cin_g; q.Cg = g.Cin_g; q.Mrows = Mrows;
            q.OW = g.OW; q.OWOH = g.OW * g.OH; q.SP = g.W; q.SQ = g.H; q.kW = g.kW; q.sw = g.sw; q.sh = g.sh; q.pw = g.pw;
            q.ph = g.ph; q.dw = g.dw; q.dh = g.dh;
            q.vec_ok = (g.Cin_g % V == 0) && (g.Cin % V == 0) && aligned16(xT);
            q.divOW = FastDiv((uint32_t)q.OW); q.divOWOH = FastDiv((uint32_t)q.OWOH); q.divCg = FastDiv((uint32_t)q.Cg);
            q.divkW = FastDiv((uint32_t)g.kW);
            a.dyT = dyT; a.Cout = g.Cout; a.co_off = grp * g.Cout_g; a.Cout_g = g.Cout_g;
            a.Ktotal = g.OW * g.OH * g.N; a.kslice = kslice; a.partial = partial;
            a.dy_vec_ok = (g.Cout % V == 0) && (g.Cout_g % V == 0) && aligned16(dyT);
            rc = launch_conv_wgrad_any<T>(s, a, slices, small);
        }
        if (rc != LUXHIP_OK) return rc;
        ProfScope ps("wgrad_reduce_kernel", s);
        const int total = Mrows * g.Cout_g;
        const int reduce_blocks = (int)ceil_div(total, 1024);
        BiasPartials bp;
        if (bias != nullptr && grp == g.groups - 1) bp = *bias;       // the bias gradient's channels ride on the last group's launch
        wgrad_reduce_kernel<T><<<(unsigned)(reduce_blocks + bp.C), 256, 0, s>>>(partial, dw, g, grp, slices, reduce_blocks, bp);
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

// ----------------------------------------------------------------------------- typed entry points
template <typename T>
static int conv_fwd_t(hipStream_t s, int act, const ConvGeom& g, const T* x, const T* w, const T* bias, T* y, T* pre,
                      T* xt_keep) {
    // xt_keep: caller's buffer of x's size that keeps the channel-contiguous copy of x for the pullback
    const size_t xb = xt_keep ? 0 : align256((size_t)g.W * g.H * g.Cin * g.N * sizeof(T));
    const size_t wb = align256((size_t)g.kW * g.kH * g.Cin_g * g.Cout * sizeof(T));
    Workspace ws;
    int rc = get_workspace(s, xb + wb, &ws);
    if (rc != LUXHIP_OK) return rc;
    T* xT = xt_keep ? xt_keep : reinterpret_cast<T*>(ws.data);
    T* wF = reinterpret_cast<T*>(ws.data + xb);
    if ((rc = transpose_and_pack<T>(s, x, xT, g.W * g.H, g.Cin, g.N, w, wF, g, 0)) != LUXHIP_OK) return rc;
    return run_conv_gemm<T>(s, g, false, xT, wF, bias, y, pre, act, ws.zeros);
}

template <typename T>
static int conv_bwd_data_t(hipStream_t s, const ConvGeom& g, const T* dy, const T* w, T* dx) {
    const size_t yb = align256((size_t)g.OW * g.OH * g.Cout * g.N * sizeof(T));
    const size_t wb = align256((size_t)g.kW * g.kH * g.Cin_g * g.Cout * sizeof(T));
    Workspace ws;
    int rc = get_workspace(s, yb + wb, &ws);
    if (rc != LUXHIP_OK) return rc;
    T* dyT = reinterpret_cast<T*>(ws.data);
    T* wD = reinterpret_cast<T*>(ws.data + yb);
    if ((rc = transpose_and_pack<T>(s, dy, dyT, g.OW * g.OH, g.Cout, g.N, w, wD, g, 1)) != LUXHIP_OK) return rc;
    return run_conv_gemm<T>(s, g, true, dyT, wD, nullptr, dx, nullptr, LUXHIP_ACT_IDENTITY, ws.zeros);
}

template <typename T>
static int conv_bwd_filter_t(hipStream_t s, const ConvGeom& g, const T* x, const T* dy, T* dw) {
    const size_t xb = align256((size_t)g.W * g.H * g.Cin * g.N * sizeof(T));
    const size_t yb = align256((size_t)g.OW * g.OH * g.Cout * g.N * sizeof(T));
    const size_t pb = wgrad_partial_bytes<T>(g);
    Workspace ws;
    int rc = get_workspace(s, xb + yb + pb, &ws);
    if (rc != LUXHIP_OK) return rc;
    T* xT = reinterpret_cast<T*>(ws.data);
    T* dyT = reinterpret_cast<T*>(ws.data + xb);
    float* partial = reinterpret_cast<float*>(ws.data + xb + yb);
    if ((rc = transpose_to_cwhn<T>(s, x, xT, g.W * g.H, g.Cin, g.N)) != LUXHIP_OK) return rc;
    if (!wgrad_direct_ok<T>(g, xT, dy)) {   // the direct kernel reads dy as it is
        if ((rc = transpose_to_cwhn<T>(s, dy, dyT, g.OW * g.OH, g.Cout, g.N)) != LUXHIP_OK) return rc;
    }
    return run_wgrad<T>(s, g, xT, dy, dyT, partial, dw, ws.zeros);
}

template <typename T>
static int fused_conv_bwd_t(hipStream_t s, int dtype, int act, const ConvGeom& g, const T* delta, const T* y,
                            const T* pre, const T* x, const T* w, T* dz, T* dw, T* dx, T* dbias, const T* xt_kept) {
    const size_t xb = xt_kept ? 0 : align256((size_t)g.W * g.H * g.Cin * g.N * sizeof(T));
    const size_t yb = align256((size_t)g.OW * g.OH * g.Cout * g.N * sizeof(T));
    const size_t wb = align256((size_t)g.kW * g.kH * g.Cin_g * g.Cout * sizeof(T));
    const size_t pb = wgrad_partial_bytes<T>(g);
    // bf16: dz, its channel-contiguous copy and the bias gradient in one pass, when both a pass over delta and a
    // transposing copy would run
    bool one_pass = false;
    if constexpr (sizeof(T) == 2)
        one_pass = (act != LUXHIP_ACT_IDENTITY || dbias != nullptr) && (dw != nullptr || dx != nullptr) &&
                   dz_cwhn_ok(g.OW * g.OH, g.Cout, g.N, delta, y, pre, dz, nullptr);
    const size_t bb = one_pass && dbias != nullptr ? dz_cwhn_partial_bytes(g.OW * g.OH, g.Cout, g.N) : 0;
    // reserve everything up front: the bias-gradient pass below uses the start of the same
    // workspace, and the buffer must not be reallocated while pointers into it are live
    Workspace ws;
    int rc = get_workspace(s, xb + yb + wb + pb + bb, &ws);
    if (rc != LUXHIP_OK) return rc;
    const T* xT = xt_kept ? xt_kept : reinterpret_cast<const T*>(ws.data);
    T* dzT = reinterpret_cast<T*>(ws.data + xb);
    T* wD = reinterpret_cast<T*>(ws.data + xb + yb);
    float* partial = reinterpret_cast<float*>(ws.data + xb + yb + wb);
    const T* dzp = delta;
    BiasPartials bias_later;              // set by the single pass when the filter gradient's reduction will finish the bias gradient
    if (one_pass) {
        if constexpr (sizeof(T) == 2) {
            bf16_t* dz_out = act == LUXHIP_ACT_IDENTITY ? nullptr : reinterpret_cast<bf16_t*>(dz);
            rc = conv_dz_cwhn_pack(s, act, g, reinterpret_cast<const bf16_t*>(delta), reinterpret_cast<const bf16_t*>(y),
                                   reinterpret_cast<const bf16_t*>(pre), dz_out, reinterpret_cast<bf16_t*>(dzT),
                                   reinterpret_cast<float*>(ws.data + xb + yb + wb + pb), reinterpret_cast<bf16_t*>(dbias),
                                   reinterpret_cast<const bf16_t*>(w), dx != nullptr ? reinterpret_cast<bf16_t*>(wD) : nullptr,
                                   dw != nullptr ? &bias_later : nullptr);
            if (rc != LUXHIP_OK) return rc;
            if (dz_out) dzp = dz;
        }
    } else {
        if (act != LUXHIP_ACT_IDENTITY || dbias != nullptr) {
            T* dz_out = act == LUXHIP_ACT_IDENTITY ? nullptr : dz;
            rc = bias_act_bwd_dispatch(s, dtype, act, (int64_t)g.OW * g.OH, g.Cout, g.N, delta, y, pre, dz_out, dbias);
            if (rc != LUXHIP_OK) return rc;
            if (dz_out) dzp = dz_out;
        }
        if (dw == nullptr && dx == nullptr) return LUXHIP_OK;
        if (dx != nullptr) rc = transpose_and_pack<T>(s, dzp, dzT, g.OW * g.OH, g.Cout, g.N, w, wD, g, 1);
        else rc = transpose_to_cwhn<T>(s, dzp, dzT, g.OW * g.OH, g.Cout, g.N);
        if (rc != LUXHIP_OK) return rc;
    }
    if (dx != nullptr) {
        if ((rc = run_conv_gemm<T>(s, g, true, dzT, wD, nullptr, dx, nullptr, LUXHIP_ACT_IDENTITY, ws.zeros)) != LUXHIP_OK) return rc;
    }
    if (dw != nullptr) {
        if (!xt_kept && (rc = transpose_to_cwhn<T>(s, x, reinterpret_cast<T*>(ws.data), g.W * g.H, g.Cin, g.N)) != LUXHIP_OK)
            return rc;
        if ((rc = run_wgrad<T>(s, g, xT, dzp, dzT, partial, dw, ws.zeros, bias_later.dbias != nullptr ? &bias_later : nullptr)) != LUXHIP_OK)
            return rc;
    }
    return LUXHIP_OK;
}

static int conv_check(int dtype, int act) {
    LUX_UNSUPPORTED_IF(dtype != LUXHIP_F32 && dtype != LUXHIP_BF16, "unsupported dtype %d", dtype);
    LUX_UNSUPPORTED_IF(act < 0 || act >= LUXHIP_ACT_COUNT, "unsupported activation id %d", act);
    return LUXHIP_OK;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_conv_fwd(luxhip_stream_t s, int dtype, int act, const luxhip_conv_dims_t* d, const void* x, const void* w,
                    const void* bias, void* y, void* pre, void* xt_keep) {
    LUX_REQUIRE_INIT();
    int rc = conv_check(dtype, act);
    if (rc != LUXHIP_OK) return rc;
    ConvGeom g;
    if ((rc = make_geom(d, &g)) != LUXHIP_OK) return rc;
    if (g.N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(x == nullptr || w == nullptr || y == nullptr, "conv_fwd: x, w and y must not be NULL");
    if (dtype == LUXHIP_F32)
        return conv_fwd_t<float>((hipStream_t)s, act, g, (const float*)x, (const float*)w, (const float*)bias, (float*)y, (float*)pre,
                                 (float*)xt_keep);
    return conv_fwd_t<bf16_t>((hipStream_t)s, act, g, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (bf16_t*)y, (bf16_t*)pre,
                              (bf16_t*)xt_keep);
}

int luxhip_conv_bwd_data(luxhip_stream_t s, int dtype, const luxhip_conv_dims_t* d, const void* dy, const void* w, void* dx) {
    LUX_REQUIRE_INIT();
    int rc = conv_check(dtype, 0);
    if (rc != LUXHIP_OK) return rc;
    ConvGeom g;
    if ((rc = make_geom(d, &g)) != LUXHIP_OK) return rc;
    if (g.N == 0) return LUXHIP_OK;
    LUX_INVALID_IF(dy == nullptr || w == nullptr || dx == nullptr, "conv_bwd_data: dy, w and dx must not be NULL");
    if (dtype == LUXHIP_F32) return conv_bwd_data_t<float>((hipStream_t)s, g, (const float*)dy, (const float*)w, (float*)dx);
    return conv_bwd_data_t<bf16_t>((hipStream_t)s, g, (const bf16_t*)dy, (const bf16_t*)w, (bf16_t*)dx);
}

int luxhip_conv_bwd_filter(luxhip_stream_t s, int dtype, const luxhip_conv_dims_t* d, const void* x, const void* dy, void* dw) {
    LUX_REQUIRE_INIT();
    int rc = conv_check(dtype, 0);
    if (rc != LUXHIP_OK) return rc;
    ConvGeom g;
    if ((rc = make_geom(d, &g)) != LUXHIP_OK) return rc;
    LUX_INVALID_IF(dw == nullptr, "conv_bwd_filter: dw must not be NULL");
    if (g.N == 0) return luxhip_fill_zero(dw, (size_t)g.kW * g.kH * g.Cin_g * g.Cout * (dtype == LUXHIP_F32 ? 4 : 2), s);
    LUX_INVALID_IF(x == nullptr || dy == nullptr, "conv_bwd_filter: x and dy must not be NULL");
    if (dtype == LUXHIP_F32) return conv_bwd_filter_t<float>((hipStream_t)s, g, (const float*)x, (const float*)dy, (float*)dw);
    return conv_bwd_filter_t<bf16_t>((hipStream_t)s, g, (const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dw);
}

int luxhip_fused_conv_bwd(luxhip_stream_t s, int dtype, int act, const luxhip_conv_dims_t* d, const void* delta,
                          const void* y, const void* pre, const void* x, const void* w, void* dz, void* dw, void* dx,
                          void* dbias, const void* xt_kept) {
    LUX_REQUIRE_INIT();
    int rc = conv_check(dtype, act);
    if (rc != LUXHIP_OK) return rc;
    ConvGeom g;
    if ((rc = make_geom(d, &g)) != LUXHIP_OK) return rc;
    const size_t esz = dtype == LUXHIP_F32 ? 4 : 2;
    if (g.N == 0) {
        if (dw) { rc = luxhip_fill_zero(dw, (size_t)g.kW * g.kH * g.Cin_g * g.Cout * esz, s); if (rc) return rc; }
        if (dbias) { rc = luxhip_fill_zero(dbias, (size_t)g.Cout * esz, s); if (rc) return rc; }
        return LUXHIP_OK;
    }
    LUX_INVALID_IF(delta == nullptr, "fused_conv_bwd: delta must not be NULL");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && dz == nullptr, "fused_conv_bwd: dz scratch is required");
    LUX_INVALID_IF(act != LUXHIP_ACT_IDENTITY && !act_needs_pre(act) && y == nullptr, "fused_conv_bwd: activation %d needs y", act);
    LUX_INVALID_IF(act_needs_pre(act) && pre == nullptr, "fused_conv_bwd: activation %d needs the pre-activation", act);
    LUX_INVALID_IF((dw != nullptr && x == nullptr && xt_kept == nullptr) || (dx != nullptr && w == nullptr), "fused_conv_bwd: x / w must not be NULL");
    if (dtype == LUXHIP_F32)
        return fused_conv_bwd_t<float>((hipStream_t)s, dtype, act, g, (const float*)delta, (const float*)y, (const float*)pre,
                                       (const float*)x, (const float*)w, (float*)dz, (float*)dw, (float*)dx, (float*)dbias,
                                       (const float*)xt_kept);
    return fused_conv_bwd_t<bf16_t>((hipStream_t)s, dtype, act, g, (const bf16_t*)delta, (const bf16_t*)y, (const bf16_t*)pre,
                                    (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)dz, (bf16_t*)dw, (bf16_t*)dx, (bf16_t*)dbias,
                                    (const bf16_t*)xt_kept);
}

}  // extern "C"
