// Implicit-GEMM convolution kernels (2 spatial dims, WHCN tensors) on the MFMA mainloop of
// gemm_core.h.
//
// The activations are first rewritten channel-contiguous ("CWHN": element (c, w, h, n) at
// ((n*H + h)*W + w)*C + c) by a transpose kernel, and the filter into K-major matrices, so that
// every gathered 16-byte chunk is a run of channels at one spatial position: aligned, and
// either entirely inside the image or entirely padding.
//
//   fprop : y(m=(ow,oh,n), co) = sum_{k=(tap,ci)} xT[pos_in(m,tap)][ci] * wF[co][k]
//   dgrad : dx(m=(iw,ih,n), ci) = sum_{k=(tap,co)} dyT[pos_out(m,tap)][co] * wD[ci][k]
//           (pos_out exists only where (iw + pad - ka*dil) is a multiple of the stride)
//   wgrad : dw(m'=(tap,ci), co) = sum_{k'=(ow,oh,n)} xT[pos_in(k',tap)][ci] * dyT[k'][co]
//           split over k' into slices; fp32 partials are reduced in slice order and scattered
//           into the (kW, kH, Cin/g, Cout) filter layout by wgrad_reduce_kernel.
// "tap" enumerates spatial offsets (ka, kb) = ka + kW*kb; the filter transforms bake in the
// flip: offset ka belongs to filter index a = kW-1-ka for a true convolution (flipkernel == 0)
// and a = ka for cross-correlation.  Outputs are written straight into WHCN: the lanes of a
// half-wave hold 32 consecutive m, which are consecutive in memory.
#pragma once

#include "common.h"
#include "gemm_core.h"

namespace luxhip {

struct ConvGeom {
    int W, H, Cin, N, kW, kH, Cout, OW, OH;
    int sw, sh, pw, ph, dw, dh;
    int groups, Cin_g, Cout_g;
    int flip;
};

// Rows m = (p, q, n) of the implicit im2col matrix, gathered from a channel-contiguous source.
template <typename T>
struct GatherK {
    const T* src;
    int Ctot, c_off, Cg;       // source channel count, first channel of the group, channels per group
    int P, PQ, M;              // row space: p in [0,P), q, n;  PQ = P*Q
    int SP, SQ;                // source spatial extent
    int kW, sw, sh, pw, ph, dw, dh;
    int dgrad, vec_ok;
    FastDiv divP, divPQ, divCg, divkW, divsw, divsh;

    __device__ __forceinline__ bool locate(int m, int k, int64_t& off) const {
        const int n = (int)divPQ.div((uint32_t)m);
        const int rem = m - n * PQ;
        const int q = (int)divP.div((uint32_t)rem);
        const int p = rem - q * P;
        const int t = (int)divCg.div((uint32_t)k);
        const int c = k - t * Cg;
        const int kb = (int)divkW.div((uint32_t)t);
        const int ka = t - kb * kW;
        int sp, sq;
        if (!dgrad) {
            sp = p * sw + ka * dw - pw;
            sq = q * sh + kb * dh - ph;
        } else {
            const int tp = p + pw - ka * dw, tq = q + ph - kb * dh;
            if (tp < 0 || tq < 0) return false;
            sp = (int)divsw.div((uint32_t)tp);
            sq = (int)divsh.div((uint32_t)tq);
            if (sp * sw != tp || sq * sh != tq) return false;
        }
        if (sp < 0 || sp >= SP || sq < 0 || sq >= SQ) return false;
        off = (((int64_t)n * SQ + sq) * SP + sp) * Ctot + c_off + c;
        return true;
    }
};

template <typename T, int ROWS>
struct ConvGatherLoaderK {
    using Tr = GemmTraits<T>;
    static constexpr bool KMAJOR = true;
    static constexpr int CHUNKS = ROWS * Tr::BK / Tr::VEC;
    static constexpr int PER_THREAD = CHUNKS / kGemmThreads;
    u32x4_v reg[PER_THREAD];
    const GatherK<T>& g;
    int m0, K;
    __device__ __forceinline__ ConvGatherLoaderK(const GatherK<T>& gg, int row0, int k_total) : g(gg), m0(row0), K(k_total) {}

    __device__ __forceinline__ void load(int k0) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = threadIdx.x + i * kGemmThreads;
            const int r = id / (Tr::BK / Tr::VEC);
            const int k = k0 + (id % (Tr::BK / Tr::VEC)) * Tr::VEC;
            const int m = m0 + r;
            u32x4_v v = {0u, 0u, 0u, 0u};
            if (m < g.M && k < K) {
                if (g.vec_ok) {          // K % VEC == 0 and chunks never straddle a tap
                    int64_t off;
                    if (g.locate(m, k, off)) v = *reinterpret_cast<const u32x4_v*>(g.src + off);
                } else {
                    T tmp[Tr::VEC];
#pragma unroll
                    for (int e = 0; e < Tr::VEC; ++e) {
                        int64_t off;
                        tmp[e] = (k + e < K && g.locate(m, k + e, off)) ? g.src[off] : T(0);
                    }
                    v = *reinterpret_cast<const u32x4_v*>(tmp);
                }
            }
            reg[i] = v;
        }
    }

    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = threadIdx.x + i * kGemmThreads;
            const int r = id / (Tr::BK / Tr::VEC), k = (id % (Tr::BK / Tr::VEC)) * Tr::VEC;
            *reinterpret_cast<u32x4_v*>(lds + lds_chunk_offset<T, true, ROWS>(r, k)) = reg[i];
        }
    }
};

template <typename T>
struct ConvGemmArgs {
    GatherK<T> gather;
    Operand<T> Wm;                     // filter matrix, K-major, rows = output columns of this group
    int K, Ncols;                      // contraction length, number of output columns (channels of the group)
    // epilogue: element (m=(p,q,n), col) -> out[(m - n*PQ) + PQ*(col_off + col + Ctot_out*n)]
    T* out;
    T* pre;
    const T* bias;                     // per output column (global channel index), may be null
    int Ctot_out, col_off, act;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ float conv_apply_act(int act, float x) {
    switch (act) {
        case LUXHIP_ACT_RELU: return Act<LUXHIP_ACT_RELU>::f(x);
        case LUXHIP_ACT_TANH: return Act<LUXHIP_ACT_TANH>::f(x);
        case LUXHIP_ACT_SIGMOID: return Act<LUXHIP_ACT_SIGMOID>::f(x);
        case LUXHIP_ACT_SWISH: return Act<LUXHIP_ACT_SWISH>::f(x);
        case LUXHIP_ACT_GELU: return Act<LUXHIP_ACT_GELU>::f(x);
        case LUXHIP_ACT_SOFTPLUS: return Act<LUXHIP_ACT_SOFTPLUS>::f(x);
        case LUXHIP_ACT_LOGSIGMOID: return Act<LUXHIP_ACT_LOGSIGMOID>::f(x);
        case LUXHIP_ACT_LISHT: return Act<LUXHIP_ACT_LISHT>::f(x);
        default: return x;
    }
}

// fprop and dgrad share this kernel (the gather loader's `dgrad` flag picks the index map).
template <typename T, int WM, int WN>
__global__ __launch_bounds__(kGemmThreads) void conv_gemm_kernel(ConvGemmArgs<T> a) {
    using ML = GemmMainloop<T, WM, WN, true, true>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    int tm, tn;
    tile_coords(a.tiles_m, a.tiles_n, tm, tn);
    const int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
    const GatherK<T>& g = a.gather;
    ConvGatherLoaderK<T, ML::TILE_M> la(g, m0, a.K);
    typename ML::PlainLoaderB lb(a.Wm, n0, a.K);
    f32x16_v acc[WM][WN];
    ML::run(la, lb, a.K, lds, acc);
    const int PQ = g.PQ, M = g.M;
    const FastDiv divPQ = g.divPQ;
    ML::for_each(acc, m0, n0, [&](int m, int col, float v) {
        if (m < M && col < a.Ncols) {
            const int n = (int)divPQ.div((uint32_t)m);
            const int ch = a.col_off + col;
            if (a.bias) v += ld(a.bias + ch);
            const int64_t off = (int64_t)(m - n * PQ) + (int64_t)PQ * (ch + (int64_t)a.Ctot_out * n);
            if (a.pre) st(a.pre + off, v);
            st(a.out + off, conv_apply_act(a.act, v));
        }
    });
}

template <typename T, int WM, int WN>
int launch_conv_gemm(hipStream_t s, ConvGemmArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, true, true>;
    a.tiles_m = (int)ceil_div(a.gather.M, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.Ncols, ML::TILE_N);
    auto kernel = conv_gemm_kernel<T, WM, WN>;
    static bool attr_set = false;
    if (!attr_set) {
        LUX_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)ML::LDS_BYTES));
        attr_set = true;
    }
    ProfScope ps(a.gather.dgrad ? (sizeof(T) == 2 ? "conv_dgrad_kernel<bf16>" : "conv_dgrad_kernel<f32>")
                                : (sizeof(T) == 2 ? "conv_fprop_kernel<bf16>" : "conv_fprop_kernel<f32>"), s);
    kernel<<<dim3((unsigned)(a.tiles_m * a.tiles_n)), dim3(kGemmThreads), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
int launch_conv_gemm_any(hipStream_t s, ConvGemmArgs<T>& a);   // picks the tile; conv_inst_*.hip

// ----------------------------------------------------------------------------- wgrad
// A(m'=(tap,ci), k'=(ow,oh,n)): MN-major gather from xT (runs of ci at one input position).
template <typename T>
struct GatherMN {
    const T* src;              // xT
    int Ctot, c_off, Cg;       // Cin, g*Cin_g, Cin_g
    int Mrows;                 // taps * Cin_g
    int OW, OWOH;              // k' decoding
    int SP, SQ;                // W, H
    int kW, sw, sh, pw, ph, dw, dh;
    int vec_ok;
    FastDiv divOW, divOWOH, divCg, divkW;

    __device__ __forceinline__ bool locate(int mrow, int kp, int64_t& off) const {
        const int t = (int)divCg.div((uint32_t)mrow);
        const int c = mrow - t * Cg;
        const int kb = (int)divkW.div((uint32_t)t);
        const int ka = t - kb * kW;
        const int n = (int)divOWOH.div((uint32_t)kp);
        const int rem = kp - n * OWOH;
        const int oh = (int)divOW.div((uint32_t)rem);
        const int ow = rem - oh * OW;
        const int sp = ow * sw + ka * dw - pw, sq = oh * sh + kb * dh - ph;
        if (sp < 0 || sp >= SP || sq < 0 || sq >= SQ) return false;
        off = (((int64_t)n * SQ + sq) * SP + sp) * Ctot + c_off + c;
        return true;
    }
};

template <typename T, int ROWS>
struct ConvGatherLoaderMN {
    using Tr = GemmTraits<T>;
    static constexpr bool KMAJOR = false;
    static constexpr int CHUNKS = ROWS * Tr::BK / Tr::VEC;
    static constexpr int PER_THREAD = CHUNKS / kGemmThreads;
    u32x4_v reg[PER_THREAD];
    const GatherMN<T>& g;
    int m0, kbase, Kend;       // Kend = one past the last k' of this slice
    __device__ __forceinline__ ConvGatherLoaderMN(const GatherMN<T>& gg, int row0, int kb, int ke)
        : g(gg), m0(row0), kbase(kb), Kend(ke) {}

    __device__ __forceinline__ void load(int k0) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = threadIdx.x + i * kGemmThreads;
            const int kp = kbase + k0 + id / (ROWS / Tr::VEC);
            const int mrow = m0 + (id % (ROWS / Tr::VEC)) * Tr::VEC;
            u32x4_v v = {0u, 0u, 0u, 0u};
            if (kp < Kend && mrow < g.Mrows) {
                if (g.vec_ok) {
                    int64_t off;
                    if (g.locate(mrow, kp, off)) v = *reinterpret_cast<const u32x4_v*>(g.src + off);
                } else {
                    T tmp[Tr::VEC];
#pragma unroll
                    for (int e = 0; e < Tr::VEC; ++e) {
                        int64_t off;
                        tmp[e] = (mrow + e < g.Mrows && g.locate(mrow + e, kp, off)) ? g.src[off] : T(0);
                    }
                    v = *reinterpret_cast<const u32x4_v*>(tmp);
                }
            }
            reg[i] = v;
        }
    }

    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int id = threadIdx.x + i * kGemmThreads;
            const int k = id / (ROWS / Tr::VEC), r = (id % (ROWS / Tr::VEC)) * Tr::VEC;
            *reinterpret_cast<u32x4_v*>(lds + lds_chunk_offset<T, false, ROWS>(r, k)) = reg[i];
        }
    }
};

template <typename T>
struct ConvWgradArgs {
    GatherMN<T> gather;
    const T* dyT;           // [k'][Cout] channel-contiguous
    int Cout, co_off, Cout_g;
    int Ktotal, kslice;     // OW*OH*N and the k' extent of one slice
    float* partial;         // [slice][Mrows][Cout_g]
    int dy_vec_ok;
    int tiles_m, tiles_n;
};

template <typename T, int WM, int WN>
__global__ __launch_bounds__(kGemmThreads) void conv_wgrad_kernel(ConvWgradArgs<T> a) {
    using ML = GemmMainloop<T, WM, WN, false, false>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    const int tile = blockIdx.x, slice = blockIdx.y;
    const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
    const int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
    const int kbeg = slice * a.kslice, kend = min(kbeg + a.kslice, a.Ktotal);
    const GatherMN<T>& g = a.gather;
    ConvGatherLoaderMN<T, ML::TILE_M> la(g, m0, kbeg, kend);
    Operand<T> B;
    B.p = a.dyT + (int64_t)kbeg * a.Cout + a.co_off;
    B.sr = 1; B.sk = a.Cout; B.rows = a.Cout_g; B.vec_ok = a.dy_vec_ok;
    typename ML::PlainLoaderB lb(B, n0, kend - kbeg);
    f32x16_v acc[WM][WN];
    ML::run(la, lb, kend - kbeg, lds, acc);
    float* out = a.partial + (size_t)slice * g.Mrows * a.Cout_g;
    const int Mrows = g.Mrows, Ncols = a.Cout_g;
    ML::for_each(acc, m0, n0, [&](int m, int col, float v) {
        if (m < Mrows && col < Ncols) out[(size_t)m + (size_t)col * Mrows] = v;
    });
}

template <typename T, int WM, int WN>
int launch_conv_wgrad(hipStream_t s, ConvWgradArgs<T>& a, int slices) {
    using ML = GemmMainloop<T, WM, WN, false, false>;
    a.tiles_m = (int)ceil_div(a.gather.Mrows, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.Cout_g, ML::TILE_N);
    auto kernel = conv_wgrad_kernel<T, WM, WN>;
    static bool attr_set = false;
    if (!attr_set) {
        LUX_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)ML::LDS_BYTES));
        attr_set = true;
    }
    ProfScope ps(sizeof(T) == 2 ? "conv_wgrad_kernel<bf16>" : "conv_wgrad_kernel<f32>", s);
    kernel<<<dim3((unsigned)(a.tiles_m * a.tiles_n), (unsigned)slices), dim3(kGemmThreads), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
int launch_conv_wgrad_any(hipStream_t s, ConvWgradArgs<T>& a, int slices, bool small);   // conv_inst_*.hip

}  // namespace luxhip
