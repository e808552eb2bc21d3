// Dense GEMM kernel (MFMA mainloop of gemm_core.h + bias / activation / pre-activation
// epilogue) and its tile-size selection.  launch_layout<T, A_KMAJOR, B_KMAJOR> is explicitly
// instantiated in gemm_inst_*.hip, one translation unit per storage type and layout pair, so
// that the heavy kernels compile in parallel.
#pragma once

#include <algorithm>

#include "common.h"
#include "gemm_core.h"
#include "gemm_dense_decl.h"

namespace luxhip {

// Epilogue of one tile: C = act(acc + bias), optional pre-activation copy.  CHECK: bounds tests;
// the activation mode and HAS_PRE are resolved once per tile, so the common cases have no branch per element.
// WM consecutive values of one column -> memory; one store when the lane's rows are consecutive
// (ML::M_STEP == 1), the storage type is bf16 and the destination allows it
template <class ML, typename T, int WM, bool CHECK>
__device__ __forceinline__ void store_column(T* col, const float (&v)[WM], int mb, int M, bool vec) {
    if constexpr (ML::M_STEP == 1 && sizeof(T) == 2 && !CHECK && (WM == 2 || WM == 4)) {
        if (vec) {
            if constexpr (WM == 4) {
                uint2 w;
                w.x = f32x2_to_bf16x2(v[0], v[1]);
                w.y = f32x2_to_bf16x2(v[2], v[3]);
                *reinterpret_cast<uint2*>(col) = w;
            } else {
                *reinterpret_cast<uint32_t*>(col) = f32x2_to_bf16x2(v[0], v[1]);
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < WM; ++i)
        if (!CHECK || mb + i * ML::M_STEP < M) st(col + i * ML::M_STEP, v[i]);
}

template <class ML, typename T, int WM, int WN, bool CHECK, int ACT_MODE, bool HAS_PRE>
__device__ __forceinline__ void dense_epilogue_as(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, int m0, int n0) {
    const int mb = ML::lane_m(m0), nb = ML::lane_n(n0);
    float bv[WM];
#pragma unroll
    for (int i = 0; i < WM; ++i)
        bv[i] = (a.bias && (!CHECK || mb + i * ML::M_STEP < a.M)) ? ld(a.bias + mb + i * ML::M_STEP) : 0.0f;
    const int act = a.act;
    const bool vec = a.c_vec != 0;
    static_for<WN * 16>([&](auto JR) {
        {
            constexpr int j = decltype(JR)::value / 16, r = decltype(JR)::value % 16;
            const int n = nb + j * 32 + ((r >> 2) << 3) + (r & 3);
            if (!CHECK || n < a.N) {
                float v[WM];
#pragma unroll
                for (int i = 0; i < WM; ++i) v[i] = acc[i][j][r] + bv[i];
                if constexpr (HAS_PRE) store_column<ML, T, WM, CHECK>(a.pre + (int64_t)n * a.ldc + mb, v, mb, a.M, vec);
                if constexpr (ACT_MODE == 1) act_vec_as<LUXHIP_ACT_RELU>(v);
                else if constexpr (ACT_MODE == 2) act_vec(act, v);
                store_column<ML, T, WM, CHECK>(a.C + (int64_t)n * a.ldc + mb, v, mb, a.M, vec);
            }
        }
    });
}
template <class ML, typename T, int WM, int WN, bool FULL>
__device__ __forceinline__ void dense_epilogue(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, int m0, int n0) {
    // activation: 0 none, 1 relu (inline), 2 any (dispatched per column of the accumulator tile)
    if (a.pre != nullptr) dense_epilogue_as<ML, T, WM, WN, !FULL, 2, true>(acc, a, m0, n0);
    else if (a.act == LUXHIP_ACT_IDENTITY) dense_epilogue_as<ML, T, WM, WN, !FULL, 0, false>(acc, a, m0, n0);
    else if (a.act == LUXHIP_ACT_RELU) dense_epilogue_as<ML, T, WM, WN, !FULL, 1, false>(acc, a, m0, n0);
    else dense_epilogue_as<ML, T, WM, WN, !FULL, 2, false>(acc, a, m0, n0);
}

// Persistent: workgroup b handles tiles b, b + gridDim.x, ...  On the direct-to-LDS path the
// first stages of the next tile are issued before the epilogue of the current one, so the
// stores overlap with the loads.
template <typename T, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, bool FULL, int NWN, int NWM>
__global__ __launch_bounds__(NWM * NWN * 64) void dense_gemm_kernel(DenseArgs<T> a) {
    using ML = GemmMainloop<T, WM, WN, A_KMAJOR, B_KMAJOR, FULL, NWN, 0, NWM, true>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    const int total = a.tiles_m * a.tiles_n;
    f32x16_v acc[WM][WN];
    int tm, tn;
    if constexpr (ML::DIRECT) {
        int t = blockIdx.x;
        tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
        int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
        typename ML::DirectLoaderA la(a.A, m0);
        typename ML::DirectLoaderB lb(a.B, n0);
        ML::pipeline_fill(la, lb, a.K, lds);
        for (;;) {
            ML::pipeline_loop(la, lb, a.K, lds, acc);
            const int tnext = t + gridDim.x;
            int m0n = 0, n0n = 0;
            if (tnext < total) {
                tile_coords(tnext, a.tiles_m, a.tiles_n, tm, tn);
                m0n = tm * ML::TILE_M;
                n0n = tn * ML::TILE_N;
                la.move_to(a.A, m0n);
                lb.move_to(a.B, n0n);
                ML::pipeline_drain();
                ML::pipeline_fill(la, lb, a.K, lds);
            }
            dense_epilogue<ML, T, WM, WN, FULL>(acc, a, m0, n0);
            if (tnext >= total) break;
            t = tnext; m0 = m0n; n0 = n0n;
        }
    } else {
        for (int t = blockIdx.x; t < total; t += gridDim.x) {
            tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
            const int m0 = tm * ML::TILE_M, n0 = tn * ML::TILE_N;
            ML::run(a.A, a.B, a.K, m0, n0, lds, acc);
            dense_epilogue<ML, T, WM, WN, FULL>(acc, a, m0, n0);
            __syncthreads();   // every wave is done with the LDS stages before the next tile refills them
        }
    }
}

template <typename T, int WM, int WN, bool AK, bool BKM, bool FULL, int NWN = 2, int NWM = 2>
int launch_cfg_full(hipStream_t s, DenseArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, AK, BKM, FULL, NWN, 0, NWM>;
    a.tiles_m = (int)ceil_div(a.M, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.N, ML::TILE_N);
    auto kernel = dense_gemm_kernel<T, WM, WN, AK, BKM, FULL, NWN, NWM>;
    static ResidentOnce ro;    // workgroups that fit the device at once
    const int resident = ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return err == hipSuccess ? persistent_grid(kernel, ML::THREADS, ML::LDS_BYTES, int64_t(1) << 40) : 0;
    });
    LUX_CHECK_HIP(ro.error);
    const int grid = (int)std::min<int64_t>((int64_t)a.tiles_m * a.tiles_n, resident);
    ProfScope ps(sizeof(T) == 2 ? (a.tail ? "dense_gemm_kernel<bf16>+tail" : "dense_gemm_kernel<bf16>")
                                : (a.tail ? "dense_gemm_kernel<f32>+tail" : "dense_gemm_kernel<f32>"), s);
    kernel<<<dim3((unsigned)grid), dim3(ML::THREADS), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

// whole, aligned tiles take the kernel variant without bounds checks (big tiles only)
template <typename T, int TILE_M, int TILE_N>
bool whole_tiles(const DenseArgs<T>& a) {
    return a.M % TILE_M == 0 && a.N % TILE_N == 0 && a.K % GemmTraits<T>::BK == 0 && a.K > 0 && a.A.vec_ok && a.B.vec_ok &&
           256 * std::max(a.A.sr, a.A.sk) * (int64_t)sizeof(T) < (1ll << 31) &&
           256 * std::max(a.B.sr, a.B.sk) * (int64_t)sizeof(T) < (1ll << 31);
}

template <typename T, int WM, int WN, bool AK, bool BKM, int NWN = 2>
int launch_cfg(hipStream_t s, DenseArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, AK, BKM, false, NWN>;
    if constexpr (WM * WN >= 4) {
        if (whole_tiles<T, ML::TILE_M, ML::TILE_N>(a)) return launch_cfg_full<T, WM, WN, AK, BKM, true, NWN>(s, a);
    }
    return launch_cfg_full<T, WM, WN, AK, BKM, false, NWN>(s, a);
}

int gemm_tile_override();   // gemm.hip: LUXHIP_GEMM_TILE=82|42|22|11 forces a tile (tuning aid), 0 = automatic

// gemm_inst_bf16_kk.hip: the 256 x 256 kernel for two K-major bf16 operands (gemm_kk256.h); false if the
// problem does not meet its conditions (then *rc is untouched)
bool launch_kk256_if_applicable(hipStream_t s, DenseArgs<bf16_t>& a, int* rc);

// whole 256 x 256 tiles of a large problem
template <typename T, bool AK, bool BKM>
int launch_big_tiles(hipStream_t s, DenseArgs<T>& a) {
    if constexpr (sizeof(T) == 2 && AK && BKM) {
        int rc = LUXHIP_OK;
        if (gemm_tile_override() == 0 && launch_kk256_if_applicable(s, a, &rc)) return rc;
    }
    return launch_cfg_full<T, 4, 2, AK, BKM, true, 4>(s, a);
}

template <typename T, bool AK, bool BKM>
int launch_layout(hipStream_t s, DenseArgs<T>& a) {
    switch (gemm_tile_override()) {
        case 82: return launch_cfg<T, 4, 2, AK, BKM, 4>(s, a);   // 8 waves, 256 x 256
        case 42: return launch_cfg<T, 4, 2, AK, BKM>(s, a);
        case 22: return launch_cfg<T, 2, 2, AK, BKM>(s, a);
        case 11: return launch_cfg<T, 1, 1, AK, BKM>(s, a);
        default: break;
    }
    // bf16 problems of whole 256 x 256 tiles that fill the chip: eight waves, operands streamed
    // straight into LDS.  Otherwise 128 x 128 tiles (two workgroups per compute unit) measured
    // fastest on large problems; 64 x 64 for small ones.
    if constexpr (sizeof(T) == 2) {
        if (whole_tiles<T, 256, 256>(a) && (int64_t)(a.M / 256) * (a.N / 256) >= 128) {
            if constexpr (AK && BKM) {
                // two K-major operands: one launch of the 256 x 256 kernel of gemm_kk256.h.  A last round that
                // is partly empty costs it less than the split below would (the small-tile kernel runs the rest
                // at a quarter of its rate: 0.60 ms against 0.44 ms for 11008 x 8192 x 4096)
                int rc = LUXHIP_OK;
                if (gemm_tile_override() == 0 && launch_kk256_if_applicable(s, a, &rc)) return rc;
            }
            // The 256 x 256 tiles are walked in rounds of one per compute unit.  When the last
            // round would be mostly empty, the matrix is cut along m or n: the part that makes
            // whole rounds keeps the big tiles, the rest (at most 10 % of the tiles) goes to
            // 128 x 128 tiles, which fill the compute units two at a time.
            const int64_t tm = a.M / 256, tn = a.N / 256, cus = num_cus() > 0 ? num_cus() : 256;
            const int64_t rem = (tm * tn) % cus;
            if (rem != 0 && rem * 10 < cus * 7) {
                for (int along_m = 1; along_m >= 0; --along_m) {
                    const int64_t t_cut = along_m ? tm : tn, t_other = along_m ? tn : tm;
                    int64_t keep = t_cut - 1;
                    while (keep > 0 && (keep * t_other) % cus != 0) --keep;
                    if (keep <= 0 || (t_cut - keep) * 10 > t_cut) continue;   // measured: a 7 % rest pays off, a 26 % rest does not
                    DenseArgs<T> big = a, rest = a;
                    const int64_t cut = keep * 256;
                    if (along_m) {
                        big.M = (int)cut;
                        rest.M = a.M - (int)cut;
                        rest.A.p = a.A.p + cut * a.A.sr;
                        rest.C = a.C + cut;
                        if (a.pre) rest.pre = a.pre + cut;
                        if (a.bias) rest.bias = a.bias + cut;
                    } else {
                        big.N = (int)cut;
                        rest.N = a.N - (int)cut;
                        rest.B.p = a.B.p + cut * a.B.sr;
                        rest.C = a.C + cut * a.ldc;
                        if (a.pre) rest.pre = a.pre + cut * a.ldc;
                    }
                    big.A.rows = big.M; big.B.rows = big.N;
                    rest.tail = 1;
                    rest.A.rows = rest.M; rest.B.rows = rest.N;
                    int rc = launch_big_tiles<T, AK, BKM>(s, big);
                    if (rc != LUXHIP_OK) return rc;
                    return launch_cfg<T, 2, 2, AK, BKM>(s, rest);
                }
            }
            return launch_big_tiles<T, AK, BKM>(s, a);
        }
    }
    const int64_t t128 = ceil_div(a.M, 128) * ceil_div(a.N, 128);
    if (a.M > 64 && a.N > 64 && t128 >= 4) return launch_cfg<T, 2, 2, AK, BKM>(s, a);
    return launch_cfg<T, 1, 1, AK, BKM>(s, a);
}

// Batched products, persistent like dense_gemm_kernel: the tiles of all products form one
// sequence (the tiles of one product are neighbours, so its operands stay in the L2 caches);
// workgroup w handles tiles w, w + gridDim.x, ...
template <typename T>
struct BatchTile {
    Operand<T> A, B;
    T* C;
    int64_t coff;   // elements between a.C and this product's C
    int product;    // index of the product
    int m0, n0;
    int K;          // extent of the contraction for this tile (a.structure may shorten it)
    bool store;     // false: the tile is not computed (a.structure == 1, every m > n)
};
template <typename T, int TILE_M, int TILE_N>
__device__ __forceinline__ BatchTile<T> batch_tile(const DenseArgs<T>& a, int t, int tiles) {
    const int b = t / tiles;
    int ti = t - b * tiles;
    // with a triangular structure the tiles of a product differ in cost: the walk through a product
    // starts at a different tile for every product, so that a workgroup (which takes every
    // gridDim.x-th tile of the sequence) does not land on the same tile position each time
    if (a.structure != 0) ti = (ti + (int)((((uint32_t)b * 2654435761u) >> 12) % (uint32_t)tiles)) % tiles;   // multiplicative hash of the product index
    int tm, tn;
    tile_coords(ti, a.tiles_m, a.tiles_n, tm, tn);
    const int i0 = b % a.bdim[0], r0 = b / a.bdim[0];
    const int i1 = r0 % a.bdim[1], i2 = r0 / a.bdim[1];
    BatchTile<T> bt;
    bt.A = a.A;
    bt.B = a.B;
    bt.A.p = a.A.p + i0 * a.bsA[0] + i1 * a.bsA[1] + i2 * a.bsA[2];
    bt.B.p = a.B.p + i0 * a.bsB[0] + i1 * a.bsB[1] + i2 * a.bsB[2];
    bt.coff = i0 * a.bsC[0] + i1 * a.bsC[1] + i2 * a.bsC[2];
    bt.product = b;
    bt.C = a.C + bt.coff;
    bt.m0 = tm * TILE_M;
    bt.n0 = tn * TILE_N;
    bt.K = a.K;
    bt.store = true;
    if (a.structure == 1) {
        // computed: everything up to the end of the block of 128 rows that holds the diagonal of the tile's last column
        // (what the products with structure 2 or 3 read, whatever their own tile size)
        if (bt.m0 >= ((bt.n0 + TILE_N - 1) / 128 + 1) * 128) { bt.store = false; bt.K = 0; }
    } else if (a.structure == 2) {
        bt.K = min(a.K, bt.n0 + TILE_N);
    } else if (a.structure == 3) {
        const int k_lo = min(bt.n0, a.K);        // n0 is a multiple of the tile width, hence of the stage depth
        bt.A.p += (int64_t)k_lo * a.A.sk;
        bt.B.p += (int64_t)k_lo * a.B.sk;
        bt.K = a.K - k_lo;
    }
    return bt;
}

// The tile as fp32 (a.c_f32): the accumulators go to memory unrounded, for results that feed a
// softmax or its pullback, where an error of one bf16 unit in the last place of a logit is a
// relative error of the same size times the logit in the weight.
template <class ML, typename T, int WM, int WN, bool FULL>
__device__ __forceinline__ void store_tile_f32(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, int64_t coff, int m0, int n0) {
    float* C = reinterpret_cast<float*>(a.C) + coff;
    ML::for_each(acc, m0, n0, [&](int m, int n, float v) {
        if (FULL || (m < a.M && n < a.N)) C[(int64_t)n * a.ldc + m] = v;
    });
}

// The softmax rule as the epilogue of the product that computes the cotangent of the attention weights
// (a.ep_probs): C = scale * probs .* (acc - d[n]), d[n] = sum over the column of probs .* acc, which the caller
// has computed as sum_e dO[e, n] O[e, n].  The cotangent itself never goes to memory, and stays fp32.
// The weights and d of a tile do not depend on the product, so their loads are issued before the tile's main loop
// and have arrived when it ends: the epilogue itself only stores.  The loaded words stay as they came from memory
// until the epilogue (unpacking them at the load would put a wait behind every load), and the choice between the
// packed and the element-wise access is made once per tile, not per column, for the same reason.
template <class ML, typename T, int WM, int WN, bool FULL>
struct SoftmaxRuleOperands {
    static constexpr bool CHECK = !FULL;
    static constexpr bool CAN_PACK = ML::M_STEP == 1 && sizeof(T) == 2 && !CHECK && (WM == 2 || WM == 4);
    // packed: pairs of bf16 per word; else one element's bits per word.  A kernel that can pack holds registers for
    // the packed words only; when the destination does not allow them (unaligned), its epilogue loads on the spot.
    uint32_t w[WN * 16][CAN_PACK ? WM / 2 : WM];
    float d[WN * 16];
    bool packed;

    template <bool PACKED>
    __device__ __forceinline__ void load_as(const DenseArgs<T>& a, const T* P, const float* dvec, int mb, int nb) {
        static_for<WN * 16>([&](auto JR) {
            constexpr int c = decltype(JR)::value, j = c / 16, r = c % 16;
            const int n = nb + j * 32 + ((r >> 2) << 3) + (r & 3);
            const int nc = CHECK ? min(n, a.N - 1) : n;       // out-of-range lanes read a valid element and store nothing
            const T* col = P + (int64_t)nc * a.ldc;
            if constexpr (PACKED) {
                if constexpr (WM == 4) {
                    const uint2 v = *reinterpret_cast<const uint2*>(col + mb);
                    w[c][0] = v.x; w[c][1] = v.y;
                } else {
                    w[c][0] = *reinterpret_cast<const uint32_t*>(col + mb);
                }
            } else {
#pragma unroll
                for (int i = 0; i < WM; ++i) {
                    const int m = CHECK ? min(mb + i * ML::M_STEP, a.M - 1) : mb + i * ML::M_STEP;
                    if constexpr (sizeof(T) == 2) w[c][i] = col[m];
                    else w[c][i] = __float_as_uint(col[m]);
                }
            }
            d[c] = dvec[nc];
        });
    }
    __device__ __forceinline__ void load_d(const float* dvec, int nb) {
        static_for<WN * 16>([&](auto JR) {
            constexpr int c = decltype(JR)::value, j = c / 16, r = c % 16;
            d[c] = dvec[nb + j * 32 + ((r >> 2) << 3) + (r & 3)];
        });
    }
    __device__ __forceinline__ void load(const DenseArgs<T>& a, int64_t coff, int product, int m0, int n0) {
        const int mb = ML::lane_m(m0), nb = ML::lane_n(n0);
        const T* P = a.ep_probs + coff;
        const float* dvec = a.ep_d + (int64_t)product * a.N;
        packed = CAN_PACK && a.c_vec != 0;
        if constexpr (CAN_PACK) {
            if (packed) load_as<true>(a, P, dvec, mb, nb);
            else load_d(dvec, nb);
        } else {
            load_as<false>(a, P, dvec, mb, nb);
        }
    }
    template <bool PACKED>
    __device__ __forceinline__ void store_as(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, T* C, int mb, int nb) const {
        const float scale = a.ep_scale;
        static_for<WN * 16>([&](auto JR) {
            constexpr int c = decltype(JR)::value, j = c / 16, r = c % 16;
            const int n = nb + j * 32 + ((r >> 2) << 3) + (r & 3);
            if (!CHECK || n < a.N) {
                float v[WM];
#pragma unroll
                for (int i = 0; i < WM; ++i) {
                    float p;
                    if constexpr (PACKED) p = __uint_as_float((i & 1) ? (w[c][i / 2] & 0xffff0000u) : (w[c][i / 2] << 16));
                    else if constexpr (sizeof(T) == 2) p = __uint_as_float(w[c][i] << 16);
                    else p = __uint_as_float(w[c][i]);
                    v[i] = scale * p * (acc[i][j][r] - d[c]);
                }
                store_column<ML, T, WM, CHECK>(C + (int64_t)n * a.ldc + mb, v, mb, a.M, PACKED);
            }
        });
    }
    __device__ __forceinline__ void store(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, int64_t coff, int m0, int n0) const {
        const int mb = ML::lane_m(m0), nb = ML::lane_n(n0);
        T* C = a.C + coff;
        if constexpr (CAN_PACK) {
            if (packed) store_as<true>(acc, a, C, mb, nb);
            else store_unprepared(acc, a, C, a.ep_probs + coff, mb, nb);
        } else {
            store_as<false>(acc, a, C, mb, nb);
        }
    }
    // nothing was loaded ahead: element-wise loads, column by column (the rare destination that is not 8-byte aligned)
    __device__ __forceinline__ void store_unprepared(const f32x16_v (&acc)[WM][WN], const DenseArgs<T>& a, T* C, const T* P, int mb,
                                                     int nb) const {
        const float scale = a.ep_scale;
        static_for<WN * 16>([&](auto JR) {
            constexpr int c = decltype(JR)::value, j = c / 16, r = c % 16;
            const int n = nb + j * 32 + ((r >> 2) << 3) + (r & 3);
            float v[WM];
#pragma unroll
            for (int i = 0; i < WM; ++i) v[i] = scale * ld(P + (int64_t)n * a.ldc + mb + i * ML::M_STEP) * (acc[i][j][r] - d[c]);
            store_column<ML, T, WM, CHECK>(C + (int64_t)n * a.ldc + mb, v, mb, a.M, false);
        });
    }
};
struct NoOperands {};

// EP: the variant with the softmax rule as its epilogue (a.ep_probs), a kernel of its own so that the plain products
// keep their register budget (and with it two workgroups per compute unit)
template <typename T, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, bool FULL, int NWN, int NWM, bool EP = false>
__global__ __launch_bounds__(NWM * NWN * 64, (EP && FULL) ? 2 : 1) void batched_gemm_kernel(DenseArgs<T> a) {
    using ML = GemmMainloop<T, WM, WN, A_KMAJOR, B_KMAJOR, FULL, NWN, 0, NWM, true>;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    const int tiles = a.tiles_m * a.tiles_n;
    const int total = tiles * a.batch;
    f32x16_v acc[WM][WN];
    std::conditional_t<EP, SoftmaxRuleOperands<ML, T, WM, WN, FULL>, NoOperands> ep;
    if constexpr (ML::DIRECT) {
        int t = blockIdx.x;
        BatchTile<T> cur = batch_tile<T, ML::TILE_M, ML::TILE_N>(a, t, tiles);
        typename ML::DirectLoaderA la(cur.A, cur.m0);
        typename ML::DirectLoaderB lb(cur.B, cur.n0);
        if constexpr (EP) {
            if (cur.store) ep.load(a, cur.coff, cur.product, cur.m0, cur.n0);
        }
        ML::pipeline_fill(la, lb, cur.K, lds);
        for (;;) {
            ML::pipeline_loop(la, lb, cur.K, lds, acc);
            const int tnext = t + gridDim.x;
            DenseArgs<T> out = a;
            out.C = cur.C;
            const int m0 = cur.m0, n0 = cur.n0;
            const int64_t coff = cur.coff;
            const bool store = cur.store;
            if constexpr (EP) {
                // the stores first: they free the registers that take the next tile's weights, whose loads go out
                // ahead of the next tile's stages (the stage waits of the main loop count the youngest loads)
                if (store) ep.store(acc, a, coff, m0, n0);
                if (tnext >= total) break;
                cur = batch_tile<T, ML::TILE_M, ML::TILE_N>(a, tnext, tiles);
                if (cur.store) ep.load(a, cur.coff, cur.product, cur.m0, cur.n0);
                la.move_to(cur.A, cur.m0);
                lb.move_to(cur.B, cur.n0);
                ML::pipeline_drain();
                ML::pipeline_fill(la, lb, cur.K, lds);
            } else {
                if (tnext < total) {
                    cur = batch_tile<T, ML::TILE_M, ML::TILE_N>(a, tnext, tiles);
                    la.move_to(cur.A, cur.m0);
                    lb.move_to(cur.B, cur.n0);
                    ML::pipeline_drain();
                    ML::pipeline_fill(la, lb, cur.K, lds);
                }
                if (store) {
                    if (a.c_f32) store_tile_f32<ML, T, WM, WN, FULL>(acc, a, coff, m0, n0);
                    else dense_epilogue<ML, T, WM, WN, FULL>(acc, out, m0, n0);
                }
                if (tnext >= total) break;
            }
            t = tnext;
        }
    } else {
        for (int t = blockIdx.x; t < total; t += gridDim.x) {
            const BatchTile<T> cur = batch_tile<T, ML::TILE_M, ML::TILE_N>(a, t, tiles);
            if (!cur.store) continue;          // uniform
            if constexpr (EP) ep.load(a, cur.coff, cur.product, cur.m0, cur.n0);
            ML::run(cur.A, cur.B, cur.K, cur.m0, cur.n0, lds, acc);
            DenseArgs<T> out = a;
            out.C = cur.C;
            if constexpr (EP) ep.store(acc, a, cur.coff, cur.m0, cur.n0);
            else if (a.c_f32) store_tile_f32<ML, T, WM, WN, FULL>(acc, a, cur.coff, cur.m0, cur.n0);
            else dense_epilogue<ML, T, WM, WN, FULL>(acc, out, cur.m0, cur.n0);
            __syncthreads();   // every wave is done with the LDS stages before the next tile refills them
        }
    }
}

template <typename T, int WM, int WN, bool AK, bool BKM, bool FULL, bool EP = false>
int launch_batched_cfg(hipStream_t s, DenseArgs<T>& a) {
    using ML = GemmMainloop<T, WM, WN, AK, BKM, FULL, 2, 0, 2>;
    a.tiles_m = (int)ceil_div(a.M, ML::TILE_M);
    a.tiles_n = (int)ceil_div(a.N, ML::TILE_N);
    const int64_t total = (int64_t)a.tiles_m * a.tiles_n * a.batch;
    LUX_UNSUPPORTED_IF(total >= (1ll << 31), "batched_matmul: too many tiles");
    auto kernel = batched_gemm_kernel<T, WM, WN, AK, BKM, FULL, 2, 2, EP>;
    static ResidentOnce ro;
    const int resident = ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ML::LDS_BYTES);
        return err == hipSuccess ? persistent_grid(kernel, ML::THREADS, ML::LDS_BYTES, int64_t(1) << 40) : 0;
    });
    LUX_CHECK_HIP(ro.error);
    ProfScope ps(EP ? "batched_gemm_kernel+softmax_rule" : (sizeof(T) == 2 ? "batched_gemm_kernel<bf16>" : "batched_gemm_kernel<f32>"), s);
    kernel<<<dim3((unsigned)std::min<int64_t>(total, resident)), dim3(ML::THREADS), ML::LDS_BYTES, s>>>(a);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

template <typename T, bool AK, bool BKM>
int launch_batched_layout(hipStream_t s, DenseArgs<T>& a) {
    // 128 x 128 tiles when a product has at least one whole tile of them, 64 x 64 otherwise;
    // the variant without bounds checks when every product is made of whole, aligned tiles
    if (a.ep_probs != nullptr) {
        // the product with the softmax rule as its epilogue has two K-major operands (v' and d_out)
        if constexpr (AK && BKM) {
            if (a.M >= 128 && a.N >= 128) {
                if (whole_tiles<T, 128, 128>(a)) return launch_batched_cfg<T, 2, 2, AK, BKM, true, true>(s, a);
                return launch_batched_cfg<T, 2, 2, AK, BKM, false, true>(s, a);
            }
            return launch_batched_cfg<T, 1, 1, AK, BKM, false, true>(s, a);
        } else {
            return set_error(LUXHIP_INVALID, "the softmax-rule epilogue exists for two K-major operands only");
        }
    }
    if (a.M >= 128 && a.N >= 128) {
        if (whole_tiles<T, 128, 128>(a)) return launch_batched_cfg<T, 2, 2, AK, BKM, true>(s, a);
        return launch_batched_cfg<T, 2, 2, AK, BKM, false>(s, a);
    }
    return launch_batched_cfg<T, 1, 1, AK, BKM, false>(s, a);
}

}  // namespace luxhip
