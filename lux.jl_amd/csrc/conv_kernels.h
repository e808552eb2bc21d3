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

// Epilogue of fprop / dgrad: element (m = (p, q, n), col) -> out[(m - n*PQ) + PQ*(col_off + col +
// Ctot_out*n)], with bias per output channel and the activation.  The image index of a row is
// decoded once per row, the channel terms once per column.  CHECK (tiles that stick out of the
// matrix), the activation mode and HAS_PRE are resolved once per tile.
template <class ML, typename T, int WM, int WN, bool CHECK, int ACT_MODE, bool HAS_PRE>
__device__ __forceinline__ void conv_epilogue_as(const f32x16_v (&acc)[WM][WN], int m0, int n0, int M, int PQ, FastDiv divPQ,
                                                 int Ncols, int col_off, int Ctot_out, const T* bias, T* out, T* pre, int act) {
    const int mb = ML::lane_m(m0), nb = ML::lane_n(n0);
    int64_t rowoff[WM];
    bool mok[WM];
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int m = mb + i * 32;
        mok[i] = !CHECK || m < M;
        const int n = (int)divPQ.div((uint32_t)(mok[i] ? m : 0));
        rowoff[i] = (int64_t)(m - n * PQ) + (int64_t)PQ * Ctot_out * n;
    }
    static_for<WN * 16>([&](auto JR) {
        {
            constexpr int j = decltype(JR)::value / 16, r = decltype(JR)::value % 16;
            const int col = nb + j * 32 + ((r >> 2) << 3) + (r & 3);
            if (!CHECK || col < Ncols) {
                const float b = bias ? ld(bias + col_off + col) : 0.0f;
                const int64_t coloff = (int64_t)PQ * (col_off + col);
                float v[WM];
#pragma unroll
                for (int i = 0; i < WM; ++i) v[i] = acc[i][j][r] + b;
                if constexpr (HAS_PRE) {
#pragma unroll
                    for (int i = 0; i < WM; ++i)
                        if (!CHECK || mok[i]) st(pre + coloff + rowoff[i], v[i]);
                }
                if constexpr (ACT_MODE == 1) act_vec_as<LUXHIP_ACT_RELU>(v);
                else if constexpr (ACT_MODE == 2) act_vec(act, v);
#pragma unroll
                for (int i = 0; i < WM; ++i)
                    if (!CHECK || mok[i]) st(out + coloff + rowoff[i], v[i]);
            }
        }
    });
}
template <class ML, typename T, int WM, int WN>
__device__ __forceinline__ void conv_epilogue(const f32x16_v (&acc)[WM][WN], int m0, int n0, int M, int PQ, FastDiv divPQ,
                                              int Ncols, int col_off, int Ctot_out, const T* bias, T* out, T* pre, int act) {
    const bool check = m0 + ML::TILE_M > M || n0 + ML::TILE_N > Ncols;
    const bool has_pre = pre != nullptr;
    // activation: 0 none, 1 relu (inline), 2 any (dispatched per column of the accumulator tile)
#define LUX_CONV_EPI(C, A, P) conv_epilogue_as<ML, T, WM, WN, C, A, P>(acc, m0, n0, M, PQ, divPQ, Ncols, col_off, Ctot_out, bias, out, pre, act)
    if (check) {                                 // rare: general variants
        if (has_pre) LUX_CONV_EPI(true, 2, true);
        else LUX_CONV_EPI(true, 2, false);
    } else if (has_pre) {
        LUX_CONV_EPI(false, 2, true);
    } else if (act == LUXHIP_ACT_IDENTITY) {
        LUX_CONV_EPI(false, 0, false);
    } else if (act == LUXHIP_ACT_RELU) {
        LUX_CONV_EPI(false, 1, false);
    } else {
        LUX_CONV_EPI(false, 2, false);
    }
#undef LUX_CONV_EPI
}

// fprop and dgrad share this kernel (the gather loader's `dgrad` flag picks the index map).
// Persistent: workgroup b handles tiles b, b + gridDim.x, ...
template <typename T, int WM, int WN>
__global__ __launch_bounds__(kGemmThreads) void conv_gemm_kernel(ConvGemmArgs<T> a) {
    using ML = GemmMainloop<T, WM, WN, true, true>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    const GatherK<T>& g = a.gather;
    const int total = a.tiles_m * a.tiles_n;
    for (int t = blockIdx.x; t < total; t += gridDim.x) {
        int tm, tn;
        tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
        const int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
        ConvGatherLoaderK<T, ML::TILE_M> la(g, m0, a.K);
        typename ML::PlainLoaderB lb(a.Wm, n0, a.K);
        f32x16_v acc[WM][WN];
        ML::run(la, lb, a.K, lds, acc);
        conv_epilogue<ML, T, WM, WN>(acc, m0, n0, g.M, g.PQ, g.divPQ, a.Ncols, a.col_off, a.Ctot_out, a.bias, a.out, a.pre, a.act);
        __syncthreads();   // every wave is done with the LDS stages before the next tile refills them
    }
}

template <typename T, int WM, int WN>
int launch_conv_gemm(hipStream_t s, ConvGemmArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, true, true>;
    a.tiles_m = (int)ceil_div(a.gather.M, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.Ncols, ML::TILE_N);
    auto kernel = conv_gemm_kernel<T, WM, WN>;
    static ResidentOnce ro;    // workgroups that fit the device at once
    const int resident = ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return err == hipSuccess ? persistent_grid(kernel, kGemmThreads, ML::LDS_BYTES, int64_t(1) << 40) : 0;
    });
    LUX_CHECK_HIP(ro.error);
    const int grid = (int)std::min<int64_t>((int64_t)a.tiles_m * a.tiles_n, resident);
    ProfScope ps(a.gather.dgrad ? (sizeof(T) == 2 ? "conv_dgrad_kernel<bf16>" : "conv_dgrad_kernel<f32>")
                                : (sizeof(T) == 2 ? "conv_fprop_kernel<bf16>" : "conv_fprop_kernel<f32>"), s);
    kernel<<<dim3((unsigned)grid), dim3(kGemmThreads), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// ----------------------------------------------------------------------------- whole-tap stages
// When the channels per group are a multiple of BK, a K stage lies inside one filter tap: the
// tap (ka, kb) and first channel of a stage are uniform scalars, and the (p, q, n) decode of a
// thread's rows does not depend on the stage, so it is done once.  Element offset of row m at
// the stage that starts at k0:  pos0(m) + tap_delta(k0)  with
//   pos0      = ((n*SQ + qs)*SP + ps)*Ctot     (ps, qs: source position for tap offset 0)
//   tap_delta = (dq*SP + dp)*Ctot + c0         (dp, dq: the tap's shift of that position)
// valid when 0 <= ps+dp < SP and 0 <= qs+dq < SQ.  fprop: ps = p*sw, dp = ka*dw - pw.  dgrad
// (unit stride only): ps = p, dp = pw - ka*dw.
template <typename T>
struct TapGeom {
    const T* src;              // channel-contiguous source, first channel of the group
    const void* zero;          // 16 zero bytes in device memory (padding and rows past M)
    int Ctot, Cg;
    int P, PQ, M;
    int SP, SQ;
    int kW, sw, sh, pw, ph, dw, dh;
    int dgrad;
    FastDiv divP, divPQ, divCg, divkW;
};

template <int N>
struct TapRows {
    int pos0[N], ps[N], qs[N];
    template <typename T>
    __device__ __forceinline__ void init(const TapGeom<T>& g, int m_first, int m_step) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int m = m_first + i * m_step;
            if (m < g.M) {
                const int n = (int)g.divPQ.div((uint32_t)m);
                const int rem = m - n * g.PQ;
                const int q = (int)g.divP.div((uint32_t)rem);
                const int p = rem - q * g.P;
                ps[i] = g.dgrad ? p : p * g.sw;
                qs[i] = g.dgrad ? q : q * g.sh;
                // ps, qs may exceed the source extent (strided windows); the 64-bit product keeps pos0 exact
                pos0[i] = (int)((((int64_t)n * g.SQ + qs[i]) * g.SP + ps[i]) * g.Ctot);
            } else {
                ps[i] = -(1 << 24);   // never valid
                qs[i] = 0;
                pos0[i] = 0;
            }
        }
    }
};

struct TapStage {
    int dp, dq, delta;
    template <typename T>
    __device__ __forceinline__ TapStage(const TapGeom<T>& g, int k0) {
        const int t = (int)g.divCg.div((uint32_t)k0);
        const int c0 = k0 - t * g.Cg;
        const int kb = (int)g.divkW.div((uint32_t)t);
        const int ka = t - kb * g.kW;
        dp = g.dgrad ? g.pw - ka * g.dw : ka * g.dw - g.pw;
        dq = g.dgrad ? g.ph - kb * g.dh : kb * g.dh - g.ph;
        delta = (dq * g.SP + dp) * g.Ctot + c0;
    }
};

// bf16, straight into LDS (same slot assignment as DirectLoader<true, ROWS, THREADS>)
template <int ROWS, int THREADS>
struct ConvDirectLoaderK {
    using T = bf16_t;
    static constexpr bool KMAJOR = true;
    static constexpr int BK = GemmTraits<bf16_t>::BK, CPR = BK / 8;
    static constexpr int INSTR = ROWS * CPR / THREADS, STEP = THREADS / CPR;
    static_assert(INSTR >= 1 && (ROWS * CPR) % THREADS == 0 && STEP % 16 == 0, "stage must split evenly over the workgroup");
    const TapGeom<T>& g;
    TapRows<INSTR> rows;
    int chunk_el;          // element offset of this thread's 16-byte chunk inside a row's stage
    uint32_t lds_off;
    __device__ __forceinline__ ConvDirectLoaderK(const TapGeom<T>& gg, int m0) : g(gg) {
        const int q = threadIdx.x, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int row = q / CPR, slot = q % CPR;
        chunk_el = (slot ^ ((row >> 2) & 3)) * 8;     // STEP is a multiple of 16: same swizzle for every i
        lds_off = (uint32_t)w * 1024u;
        move_to(m0);
    }
    __device__ __forceinline__ void move_to(int m0) { rows.init(g, m0 + (int)threadIdx.x / CPR, STEP); }
    __device__ __forceinline__ void issue(int k0, T* lds_tile) const {
        typedef __attribute__((address_space(3))) void* lds_vp;
        typedef const __attribute__((address_space(1))) void* glb_vp;
        const TapStage st(g, k0);
        char* l = reinterpret_cast<char*>(lds_tile) + lds_off;
#pragma unroll
        for (int i = 0; i < INSTR; ++i) {
            const bool valid = (unsigned)(rows.ps[i] + st.dp) < (unsigned)g.SP && (unsigned)(rows.qs[i] + st.dq) < (unsigned)g.SQ;
            const T* src = g.src + ((int64_t)rows.pos0[i] + st.delta + chunk_el);
            const void* p = valid ? static_cast<const void*>(src) : g.zero;
            __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(l + i * (THREADS * 16)), 16, 0, 0);
        }
    }
};

// any storage type, through registers (interface of TileLoader)
template <typename T, int ROWS, int THREADS>
struct ConvTapLoaderK {
    using Tr = GemmTraits<T>;
    static constexpr bool KMAJOR = true;
    static constexpr int CPR = Tr::BK / Tr::VEC;
    static constexpr int PER_THREAD = ROWS * CPR / THREADS, STEP = THREADS / CPR;
    static_assert(PER_THREAD >= 1 && (ROWS * CPR) % THREADS == 0, "tile must split evenly over the workgroup");
    u32x4_v reg[PER_THREAD];
    const TapGeom<T>& g;
    TapRows<PER_THREAD> rows;
    int chunk_el;
    __device__ __forceinline__ ConvTapLoaderK(const TapGeom<T>& gg, int m0) : g(gg) {
        chunk_el = (threadIdx.x % CPR) * Tr::VEC;
        rows.init(g, m0 + threadIdx.x / CPR, STEP);
    }
    __device__ __forceinline__ ConvTapLoaderK(const ConvTapLoaderK&) = default;
    __device__ __forceinline__ void load(int k0) {
        const TapStage st(g, k0);
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const bool valid = (unsigned)(rows.ps[i] + st.dp) < (unsigned)g.SP && (unsigned)(rows.qs[i] + st.dq) < (unsigned)g.SQ;
            const T* src = g.src + ((int64_t)rows.pos0[i] + st.delta + chunk_el);
            const u32x4_v* p = reinterpret_cast<const u32x4_v*>(valid ? static_cast<const void*>(src) : g.zero);
            reg[i] = *p;
        }
    }
    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int r = threadIdx.x / CPR + i * STEP;
            *reinterpret_cast<u32x4_v*>(lds + lds_chunk_offset<T, true, ROWS>(r, chunk_el)) = reg[i];
        }
    }
};

template <typename T>
struct ConvTapArgs {
    TapGeom<T> tap;
    Operand<T> Wm;                     // filter matrix, K-major, rows = output columns of this group
    int K, Ncols;
    T* out;
    T* pre;
    const T* bias;
    int Ctot_out, col_off, act;
    int tiles_m, tiles_n;
    int m_begin;                       // first row of this launch (rows m_begin .. tap.M are tiled)
};

// Persistent: workgroup b handles tiles b, b + gridDim.x, ...  On the direct-to-LDS path the
// first stages of the next tile are issued before the epilogue of the current one.
template <typename T, int WM, int WN, int NWN, int NST, int NWM>
__global__ __launch_bounds__(NWM * NWN * 64) void conv_tap_kernel(ConvTapArgs<T> a) {
    constexpr bool DIRECT = sizeof(T) == 2;
    using ML = GemmMainloop<T, WM, WN, true, true, DIRECT, NWN, NST, NWM>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    const TapGeom<T>& g = a.tap;
    const int total = a.tiles_m * a.tiles_n;
    f32x16_v acc[WM][WN];
    int tm, tn;
    if constexpr (DIRECT) {
        int t = blockIdx.x;
        tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
        int m0 = a.m_begin + tm * ML::TILE_M, n0 = tn * ML::TILE_N;
        ConvDirectLoaderK<ML::TILE_M, ML::THREADS> la(g, m0);
        DirectLoader<true, ML::TILE_N, ML::THREADS, true> lb(a.Wm, n0, g.zero);
        ML::pipeline_fill(la, lb, a.K, lds);
        for (;;) {
            ML::pipeline_loop(la, lb, a.K, lds, acc);
            const int tnext = t + gridDim.x;
            int m0n = 0, n0n = 0;
            if (tnext < total) {
                tile_coords(tnext, a.tiles_m, a.tiles_n, tm, tn);
                m0n = a.m_begin + tm * ML::TILE_M;
                n0n = tn * ML::TILE_N;
                la.move_to(m0n);
                lb.move_to(a.Wm, n0n);
                ML::pipeline_drain();
                ML::pipeline_fill(la, lb, a.K, lds);
            }
            conv_epilogue<ML, T, WM, WN>(acc, m0, n0, g.M, g.PQ, g.divPQ, a.Ncols, a.col_off, a.Ctot_out, a.bias, a.out, a.pre, a.act);
            if (tnext >= total) break;
            t = tnext; m0 = m0n; n0 = n0n;
        }
    } else {
        for (int t = blockIdx.x; t < total; t += gridDim.x) {
            tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
            const int m0 = a.m_begin + tm * ML::TILE_M, n0 = tn * ML::TILE_N;
            ConvTapLoaderK<T, ML::TILE_M, ML::THREADS> la(g, m0);
            typename ML::PlainLoaderB lb(a.Wm, n0, a.K);
            ML::run(la, lb, a.K, lds, acc);
            conv_epilogue<ML, T, WM, WN>(acc, m0, n0, g.M, g.PQ, g.divPQ, a.Ncols, a.col_off, a.Ctot_out, a.bias, a.out, a.pre, a.act);
            __syncthreads();   // every wave is done with the LDS stages before the next tile refills them
        }
    }
}

// Workgroups of conv_tap_kernel<...> that the device holds at once (0 on error); also raises the
// kernel's dynamic LDS limit on first use.
template <typename T, int WM, int WN, int NWN, int NST, int NWM = 2>
int conv_tap_resident() {
    using ML = GemmMainloop<T, WM, WN, true, true, sizeof(T) == 2, NWN, NST, NWM>;
    static ResidentOnce ro;
    return ro.get([&](hipError_t& err) {
        auto kernel = conv_tap_kernel<T, WM, WN, NWN, NST, NWM>;
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return err == hipSuccess ? persistent_grid(kernel, ML::THREADS, ML::LDS_BYTES, int64_t(1) << 40) : 0;
    });
}

template <typename T, int WM, int WN, int NWN, int NST, int NWM = 2>
int launch_conv_tap(hipStream_t s, ConvTapArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, true, true, sizeof(T) == 2, NWN, NST, NWM>;
    a.tiles_m = (int)ceil_div(a.tap.M - a.m_begin, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.Ncols, ML::TILE_N);
    auto kernel = conv_tap_kernel<T, WM, WN, NWN, NST, NWM>;
    const int resident = conv_tap_resident<T, WM, WN, NWN, NST, NWM>();
    LUX_UNSUPPORTED_IF(resident <= 0, "conv: the kernel does not fit the device");
    const int grid = (int)std::min<int64_t>((int64_t)a.tiles_m * a.tiles_n, resident);
    // a launch that finishes the rows of another one is reported as "<name>+tail"
    static const char* const names[2][2][2] = {
        {{"conv_fprop_kernel<f32>", "conv_fprop_kernel<f32>+tail"}, {"conv_dgrad_kernel<f32>", "conv_dgrad_kernel<f32>+tail"}},
        {{"conv_fprop_kernel<bf16>", "conv_fprop_kernel<bf16>+tail"}, {"conv_dgrad_kernel<bf16>", "conv_dgrad_kernel<bf16>+tail"}}};
    ProfScope ps(names[sizeof(T) == 2][a.tap.dgrad ? 1 : 0][a.m_begin > 0], s);
    kernel<<<dim3((unsigned)grid), dim3(ML::THREADS), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T>
int launch_conv_tap_any(hipStream_t s, ConvTapArgs<T>& a);   // picks the tile; conv_inst_*.hip

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
    static ResidentOnce ro;   // here only the one-time raise of the dynamic LDS limit
    ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return 1;
    });
    LUX_CHECK_HIP(ro.error);
    ProfScope ps(sizeof(T) == 2 ? "conv_wgrad_kernel<bf16>" : "conv_wgrad_kernel<f32>", s);
    kernel<<<dim3((unsigned)(a.tiles_m * a.tiles_n), (unsigned)slices), dim3(kGemmThreads), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// ----------------------------------------------------------------------------- wgrad, bf16 straight into LDS
// A(m' = (tap, ci), k' = (ow, oh, n)) gathered from the channel-contiguous xT into the MN-major
// LDS layout: a thread's 16-byte chunk always covers the same 8 channels of the same tap, so
// tap and channel are decoded once; the output position of each load is decoded per stage.
// B(k', co) comes from dy in its original WHCN layout, where the positions of one image and
// channel are contiguous: K-major, no transposed copy of dy, 16-byte LDS reads.  Needs
// OW*OH % BK == 0 (a stage never straddles two images) and slices of whole stages.
struct WgradGeomA {
    const bf16_t* src;         // xT + first channel of the group
    const void* zero;
    int Ctot, Cg, Mrows;
    int OW, OWOH, SP, SQ;
    int kW, sw, sh, pw, ph, dw, dh;
    FastDiv divOW, divOWOH, divCg, divkW;
};

template <int ROWS, int THREADS>
struct WgradDirectLoaderA {
    using T = bf16_t;
    static constexpr bool KMAJOR = false;
    static constexpr int BK = GemmTraits<bf16_t>::BK, CPR = ROWS / 8;
    static constexpr int INSTR = ROWS * BK / 8 / THREADS, STEP = THREADS / CPR;   // STEP: k rows per instruction
    static_assert(INSTR >= 1 && (ROWS * BK / 8) % THREADS == 0 && STEP % 4 == 0, "stage must split evenly over the workgroup");
    const WgradGeomA& g;
    int dpx, dqy;              // tap shift of the source position
    bool valid_m;
    uint32_t lds_off;
    // The stages of a slice are issued in order (k0 = 0, BK, 2 BK, ...): the output position of each load is
    // kept as (ow, oh) and the element offset of its source position at tap shift 0, and moved on by BK
    // positions per stage with two compares (one row wrap at most for rows of at least BK positions).
    mutable int ow[INSTR], oh[INSTR];
    mutable int64_t pos[INSTR];        // ((n * SQ + oh * sh) * SP + ow * sw) * Ctot + the tap's shift and channel
    int64_t d_step, d_row, d_img;      // what BK positions, a row wrap and an image wrap add to pos
    __device__ __forceinline__ WgradDirectLoaderA(const WgradGeomA& gg, int m0, int kb_) : g(gg) {
        const int q = threadIdx.x, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int krow = q / CPR;
        const int slot = q % CPR;
        const int r = (slot * 8) ^ ((krow & 3) << mn_swizzle_shift(ROWS));   // (krow + i*STEP) & 3 == krow & 3
        const int m = m0 + r;
        valid_m = m < g.Mrows;
        const int t = (int)g.divCg.div((uint32_t)(valid_m ? m : 0));
        const int coff = (valid_m ? m : 0) - t * g.Cg;
        const int kb = (int)g.divkW.div((uint32_t)t), ka = t - kb * g.kW;
        dpx = ka * g.dw - g.pw;
        dqy = kb * g.dh - g.ph;
        lds_off = (uint32_t)w * 1024u;
        const int64_t shift = ((int64_t)dqy * g.SP + dpx) * g.Ctot + coff;
#pragma unroll
        for (int i = 0; i < INSTR; ++i) {
            const int kp = kb_ + krow + i * STEP;
            const int n = (int)g.divOWOH.div((uint32_t)kp);
            const int rem = kp - n * g.OWOH;
            oh[i] = (int)g.divOW.div((uint32_t)rem);
            ow[i] = rem - oh[i] * g.OW;
            pos[i] = (((int64_t)n * g.SQ + oh[i] * g.sh) * g.SP + ow[i] * g.sw) * g.Ctot + shift;
        }
        const int OH = g.OWOH / g.OW;
        d_step = (int64_t)BK * g.sw * g.Ctot;
        d_row = ((int64_t)g.sh * g.SP - (int64_t)g.OW * g.sw) * g.Ctot;
        d_img = ((int64_t)g.SQ - (int64_t)OH * g.sh) * g.SP * g.Ctot;
    }
    __device__ __forceinline__ void issue(int /*k0: the next stage in order*/, T* lds_tile) const {
        typedef __attribute__((address_space(3))) void* lds_vp;
        typedef const __attribute__((address_space(1))) void* glb_vp;
        char* l = reinterpret_cast<char*>(lds_tile) + lds_off;
        const int OH = g.OWOH / g.OW;
#pragma unroll
        for (int i = 0; i < INSTR; ++i) {
            const int sp = ow[i] * g.sw + dpx, sq = oh[i] * g.sh + dqy;
            const bool valid = valid_m && (unsigned)sp < (unsigned)g.SP && (unsigned)sq < (unsigned)g.SQ;
            const void* p = valid ? static_cast<const void*>(g.src + pos[i]) : g.zero;
            __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(l + i * (THREADS * 16)), 16, 0, 0);
            // on to the next stage's position
            ow[i] += BK;
            pos[i] += d_step;
            while (ow[i] >= g.OW) {             // once for rows of at least BK positions
                ow[i] -= g.OW;
                pos[i] += d_row;
                if (++oh[i] == OH) {
                    oh[i] = 0;
                    pos[i] += d_img;
                }
            }
        }
    }
};

struct WgradGeomB {
    const bf16_t* dy;          // WHCN
    const void* zero;
    int PQ, Cout, co_off, Ncols;
    FastDiv divPQ;
};

template <int ROWS, int THREADS>
struct WgradDirectLoaderB {
    using T = bf16_t;
    static constexpr bool KMAJOR = true;
    static constexpr int BK = GemmTraits<bf16_t>::BK, CPR = BK / 8;
    static constexpr int INSTR = ROWS * CPR / THREADS, STEP = THREADS / CPR;
    static_assert(INSTR >= 1 && (ROWS * CPR) % THREADS == 0 && STEP % 16 == 0, "stage must split evenly over the workgroup");
    const WgradGeomB& g;
    int kbeg, col0, rows_left;
    int voff;                  // elements: row * PQ + chunk * 8
    uint32_t lds_off;
    __device__ __forceinline__ WgradDirectLoaderB(const WgradGeomB& gg, int n0, int kb_) : g(gg), kbeg(kb_), col0(n0) {
        const int q = threadIdx.x, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int row = q / CPR, slot = q % CPR;
        voff = row * g.PQ + ((slot ^ ((row >> 2) & 3)) << 3);
        rows_left = g.Ncols - n0 - row;
        lds_off = (uint32_t)w * 1024u;
    }
    __device__ __forceinline__ void issue(int k0, T* lds_tile) const {
        typedef __attribute__((address_space(3))) void* lds_vp;
        typedef const __attribute__((address_space(1))) void* glb_vp;
        const int kp = kbeg + k0;                                  // uniform
        const int n = (int)g.divPQ.div((uint32_t)kp);
        const T* base = g.dy + (kp - n * g.PQ) + (int64_t)g.PQ * (g.co_off + col0 + (int64_t)g.Cout * n);
        char* l = reinterpret_cast<char*>(lds_tile) + lds_off;
#pragma unroll
        for (int i = 0; i < INSTR; ++i) {
            const T* src = base + voff + (int64_t)i * STEP * g.PQ;
            const void* p = i * STEP < rows_left ? static_cast<const void*>(src) : g.zero;
            __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(l + i * (THREADS * 16)), 16, 0, 0);
        }
    }
};

struct ConvWgradDirectArgs {
    WgradGeomA A;
    WgradGeomB B;
    int Ktotal, kslice;
    float* partial;            // [slice][Mrows][Ncols]
    int tiles_m, tiles_n, slices;
};

template <int WM, int WN, int NWN, int NST, int NWM>
__global__ __launch_bounds__(NWM * NWN * 64) void conv_wgrad_direct_kernel(ConvWgradDirectArgs a) {
    using ML = GemmMainloop<bf16_t, WM, WN, false, true, true, NWN, NST, NWM>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    bf16_t* lds = reinterpret_cast<bf16_t*>(lds_raw);
    // Workgroups are handed to the eight XCDs in turn (workgroup i to XCD i % 8), each with an L2 of its own.
    // All tiles of a slice read the same positions of x and dy, so they go to the same XCD, one after the
    // other: XCD c takes the slices c, c + 8, ... and runs through the tiles of one before the next.
    const int tiles = a.tiles_m * a.tiles_n;
    int tile, slice;
    {
        const int id = blockIdx.x, xcd = id & 7, j = id >> 3;
        const int whole = (a.slices >> 3) << 3;              // slices that fill whole groups of eight
        if (id < whole * tiles) {
            tile = j % tiles;
            slice = xcd + 8 * (j / tiles);
        } else {                                             // the rest: slice-major
            const int r = id - whole * tiles;
            tile = r % tiles;
            slice = whole + r / tiles;
        }
    }
    const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
    const int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
    const int kbeg = slice * a.kslice, kend = min(kbeg + a.kslice, a.Ktotal);
    WgradDirectLoaderA<ML::TILE_M, ML::THREADS> la(a.A, m0, kbeg);
    WgradDirectLoaderB<ML::TILE_N, ML::THREADS> lb(a.B, n0, kbeg);
    f32x16_v acc[WM][WN];
    ML::run_pipeline(la, lb, kend - kbeg, lds, acc);
    const int Mrows = a.A.Mrows, Ncols = a.B.Ncols;
    float* out = a.partial + (size_t)slice * Mrows * Ncols;
    ML::for_each(acc, m0, n0, [&](int m, int col, float v) {
        if (m < Mrows && col < Ncols) out[(size_t)m + (size_t)col * Mrows] = v;
    });
}

int launch_conv_wgrad_direct(hipStream_t s, ConvWgradDirectArgs& a, int slices);   // conv_inst_wgrad_bf16.hip

template <typename T>
int launch_conv_wgrad_any(hipStream_t s, ConvWgradArgs<T>& a, int slices, bool small);   // conv_inst_*.hip

}  // namespace luxhip
