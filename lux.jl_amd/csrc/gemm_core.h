// LDS-staged MFMA GEMM mainloop for gfx950, shared by the dense and convolution kernels.
//
//   C(m, n) = sum_k A(m, k) * B(k, n),  fp32 accumulation.
//
// A workgroup of 4 waves (2 along m x 2 along n) owns a (2*WM*32) x (2*WN*32) tile of C; each
// wave owns WM x WN MFMA tiles of 32 x 32.  The MFMA "row" dimension is mapped to n and the
// "column" dimension (one column per lane) to m, so that the 32 lanes of a half-wave hold 32
// consecutive m: stores to the column-major C are contiguous and a per-m bias is one value per
// lane.
//
// Storage types:  bf16 -> v_mfma_f32_32x32x16_bf16 (BK = 32 per stage),
//                 fp32 -> v_mfma_f32_32x32x2_f32   (BK = 16 per stage).
//
// Each operand tile is staged global -> registers -> LDS (double buffered, one barrier per
// stage) in the layout that matches how it lies in memory:
//   K-major operand  (k contiguous): LDS [row][BK]; bf16 rows are 64 B (BK = 32) with an XOR
//       swizzle of the 16-byte chunk index by (row/4)%4 so that the ds_read_b128 fragment reads
//       of 16 consecutive rows fall into different banks; fp32 rows are padded by 4 floats.
//   MN-major operand (m or n contiguous, k strided): LDS [k][rows]; bf16 rows are unpadded and
//       their 64-byte granules XOR-swizzled with k&3; fragments are read with
//       ds_read_b64_tr_b16 (the LDS transpose read of gfx950), which hands each lane the 4
//       consecutive k of its own row out of a 4(k) x 16(rows) block (the 4 k-rows of a block
//       then sit in 4 different bank groups); fp32 rows are padded and read with ds_read_b32.
// Whole aligned bf16 tiles skip the registers: global_load_lds_dwordx4 writes 64 lanes x 16
// bytes linearly into LDS, and each lane fetches the chunk that the swizzle wants there.
// The same (lane group, slot) -> k assignment is used for both operands of an MFMA, which is
// all the instruction needs.
#pragma once

#include <algorithm>
#include <type_traits>
#include <utility>

#include "common.h"

namespace luxhip {

// f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N-1>): a loop that is
// expanded by the front end, for bodies the loop unroller gives up on (accumulator registers can
// only be indexed by compile-time constants).
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

typedef __bf16 bf16x8_v __attribute__((ext_vector_type(8)));
typedef float f32x16_v __attribute__((ext_vector_type(16)));
typedef short s16x4_v __attribute__((ext_vector_type(4)));
typedef short s16x8_v __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_v __attribute__((ext_vector_type(4)));

// Activation over a few values at a time: the epilogues branch on the runtime activation id once
// per column of the accumulator tile, and only those few values are live in VGPRs meanwhile.
template <int ACT, int N>
__device__ __forceinline__ void act_vec_as(float (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = Act<ACT>::f(v[i]);
}
template <int N>
__device__ __forceinline__ void act_vec(int act, float (&v)[N]) {
    switch (act) {
        case LUXHIP_ACT_RELU: act_vec_as<LUXHIP_ACT_RELU>(v); break;
        case LUXHIP_ACT_TANH: act_vec_as<LUXHIP_ACT_TANH>(v); break;
        case LUXHIP_ACT_SIGMOID: act_vec_as<LUXHIP_ACT_SIGMOID>(v); break;
        case LUXHIP_ACT_SWISH: act_vec_as<LUXHIP_ACT_SWISH>(v); break;
        case LUXHIP_ACT_GELU: act_vec_as<LUXHIP_ACT_GELU>(v); break;
        case LUXHIP_ACT_SOFTPLUS: act_vec_as<LUXHIP_ACT_SOFTPLUS>(v); break;
        case LUXHIP_ACT_LOGSIGMOID: act_vec_as<LUXHIP_ACT_LOGSIGMOID>(v); break;
        case LUXHIP_ACT_LISHT: act_vec_as<LUXHIP_ACT_LISHT>(v); break;
        default: break;
    }
}

constexpr int kGemmThreads = 256;

template <typename T>
struct GemmTraits;
template <>
struct GemmTraits<bf16_t> {
    static constexpr int BK = 32, VEC = 8, KSTEP = 16;   // KSTEP: k consumed per fragment load
    static constexpr int PAD_MN = 0;    // MN-major rows are swizzled instead of padded
    __host__ __device__ static constexpr int kmajor_stride() { return BK; }
};
template <>
struct GemmTraits<float> {
    static constexpr int BK = 16, VEC = 4, KSTEP = 8;
    static constexpr int PAD_MN = 8;    // 4 k-rows apart = 128 bytes apart modulo the 256-byte bank period
    __host__ __device__ static constexpr int kmajor_stride() { return BK + 4; }
};

// The LDS of gfx950 has 64 banks of 4 bytes (256-byte period).  bf16 swizzles are chosen so that
// the lanes served together hit 256 distinct bytes:
//   K-major rows of 64 bytes: ds_read_b128 serves 16 lanes (16 rows) at a time; rows r and r+4
//       share a bank offset, so the chunk index is XORed with (r/4)%4.
//   MN-major [k][rows]: a transpose read serves two 16-lane blocks at a time, each 4 k-rows x 32
//       bytes at row offsets g and g+32 bytes; XORing the row index with (k%4) << 5 moves the 4
//       k-rows into 4 different 64-byte granules (tiles narrower than 128 rows have only room for
//       32-byte granules).
__host__ __device__ constexpr int mn_swizzle_shift(int rows) { return rows >= 128 ? 5 : 4; }

// elements of one LDS stage of an operand tile with `rows` rows
template <typename T, bool KMAJOR>
__host__ __device__ constexpr int lds_tile_elems(int rows) {
    return KMAJOR ? rows * GemmTraits<T>::kmajor_stride() : GemmTraits<T>::BK * (rows + GemmTraits<T>::PAD_MN);
}

// An operand seen as rows x K: element (r, k) at p[r*sr + k*sk]; one of sr, sk is 1.
template <typename T>
struct Operand {
    const T* p;
    int64_t sr, sk;
    int rows;      // valid rows (M or N)
    int vec_ok;    // 16-byte loads along the contiguous dimension are aligned
};

// ----------------------------------------------------------------------------- global -> registers
// LDS offset (in elements) of the 16-byte chunk that starts at (row r, column k) of a tile.
template <typename T, bool KMAJOR, int ROWS>
__device__ __forceinline__ int lds_chunk_offset(int r, int k) {
    using Tr = GemmTraits<T>;
    if constexpr (KMAJOR) {
        if constexpr (sizeof(T) == 2) return r * Tr::BK + (((k >> 3) ^ ((r >> 2) & 3)) << 3);
        else return r * Tr::kmajor_stride() + k;
    } else {
        if constexpr (sizeof(T) == 2) return k * ROWS + (r ^ ((k & 3) << mn_swizzle_shift(ROWS)));   // r is a multiple of 8
        else return k * (ROWS + Tr::PAD_MN) + r;
    }
}

// Loader policy of the mainloop: load(k0) fetches this thread's share of the stage that starts
// at k0 into registers, store(lds) writes it to the stage buffer.  TileLoader reads a plain
// strided matrix; the convolution kernels provide gathering loaders with the same interface.
template <typename T, bool KMAJOR_, int ROWS, bool FULL = false, int THREADS = kGemmThreads>
struct TileLoader {
    using Tr = GemmTraits<T>;
    static constexpr bool KMAJOR = KMAJOR_;
    static constexpr int CHUNKS = ROWS * Tr::BK / Tr::VEC;
    static constexpr int PER_THREAD = CHUNKS / THREADS;
    static_assert(CHUNKS % THREADS == 0, "tile must split evenly over the workgroup");
    u32x4_v reg[PER_THREAD];
    Operand<T> op;
    int r0, K;
    uint32_t voff;   // FULL: byte offset of this thread's first chunk inside the tile (32-bit)
    __device__ __forceinline__ TileLoader(const Operand<T>& o, int row0, int k_total) : op(o), r0(row0), K(k_total) {
        int r, k;
        coords(threadIdx.x, r, k);
        voff = (uint32_t)(((int64_t)r * op.sr + (int64_t)k * op.sk) * (int64_t)sizeof(T));
    }

    __device__ __forceinline__ static void coords(int id, int& r, int& k) {
        if constexpr (KMAJOR) {
            r = id / (Tr::BK / Tr::VEC);
            k = (id % (Tr::BK / Tr::VEC)) * Tr::VEC;
        } else {
            k = id / (ROWS / Tr::VEC);
            r = (id % (ROWS / Tr::VEC)) * Tr::VEC;
        }
    }

    __device__ __forceinline__ void load(int k0) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            int r, k;
            coords(threadIdx.x + i * THREADS, r, k);
            r += r0;
            k += k0;
            if constexpr (FULL) {
                // whole tiles, aligned: no predication; uniform 64-bit base (scalar registers) plus
                // one 32-bit per-thread offset.  Chunk i of a thread lies a uniform step further.
                constexpr int STEP = KMAJOR ? THREADS / (Tr::BK / Tr::VEC) : THREADS / (ROWS / Tr::VEC);
                const int64_t ubase = KMAJOR ? ((int64_t)(r0 + i * STEP) * op.sr + (int64_t)k0 * op.sk)
                                             : ((int64_t)r0 * op.sr + (int64_t)(k0 + i * STEP) * op.sk);
                const char* up = reinterpret_cast<const char*>(op.p + ubase);
                reg[i] = *reinterpret_cast<const u32x4_v*>(up + voff);
            } else {
                u32x4_v v = {0u, 0u, 0u, 0u};
                const int rem = KMAJOR ? (K - k) : (op.rows - r);     // valid elements along the chunk
                const bool in = KMAJOR ? (r < op.rows) : (k < K);
                if (in && rem > 0) {
                    const T* src = op.p + (int64_t)r * op.sr + (int64_t)k * op.sk;
                    if (op.vec_ok && rem >= Tr::VEC) {
                        v = *reinterpret_cast<const u32x4_v*>(src);
                    } else {
                        T tmp[Tr::VEC];
#pragma unroll
                        for (int e = 0; e < Tr::VEC; ++e) tmp[e] = e < rem ? src[e] : T(0);
                        v = *reinterpret_cast<const u32x4_v*>(tmp);
                    }
                }
                reg[i] = v;
            }
        }
    }

    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            int r, k;
            coords(threadIdx.x + i * THREADS, r, k);
            *reinterpret_cast<u32x4_v*>(lds + lds_chunk_offset<T, KMAJOR, ROWS>(r, k)) = reg[i];
        }
    }
};

// Direct global -> LDS loader for aligned bf16 tiles.  One wave instruction fills 1 KiB of the
// stage linearly (lane i -> byte 16*i after a wave-uniform base); lane i therefore fetches the
// global chunk whose swizzled home is that slot.  BOUNDED: rows at or past op.rows read from
// `zero` (16 zero bytes somewhere in device memory) instead, so partial tiles need no branch.
// PERM_WM > 0 (K-major only): the rows are permuted inside groups of 32 * PERM_WM: LDS row
// 32*i + j of a group holds global row PERM_WM*j + i.  A lane of the MFMA then owns PERM_WM
// consecutive rows of the result instead of rows 32 apart, and the epilogue stores them with one
// instruction.  The LDS layout and the fragment reads do not change.
template <bool KMAJOR_, int ROWS, int THREADS = kGemmThreads, bool BOUNDED = false, int PERM_WM = 0>
struct DirectLoader {
    using T = bf16_t;
    static constexpr bool KMAJOR = KMAJOR_;
    static constexpr int BK = GemmTraits<bf16_t>::BK;
    static constexpr int CPR = KMAJOR ? BK / 8 : ROWS / 8;         // 16-byte chunks per LDS row
    static constexpr int INSTR = ROWS * BK / 8 / THREADS;          // instructions per thread and stage
    static_assert(INSTR >= 1 && (ROWS * BK / 8) % THREADS == 0, "stage must split evenly over the workgroup");
    static constexpr int STEP = THREADS / CPR;                // LDS rows covered per instruction of the workgroup
    static_assert(!BOUNDED || KMAJOR, "row bounds are implemented for K-major operands");
    static_assert(PERM_WM == 0 || (KMAJOR && STEP % (32 * PERM_WM) == 0), "row permutation: whole groups per instruction");
    __device__ __forceinline__ static int global_row(int lds_row) {
        if constexpr (PERM_WM == 0) return lds_row;
        constexpr int G = 32 * PERM_WM;
        const int o = lds_row % G;
        return lds_row - o + (o % 32) * PERM_WM + o / 32;
    }
    const char* base;      // uniform: first element of the tile (row r0, k = 0)
    const char* zero;      // BOUNDED only
    int64_t step_bytes;    // uniform: global distance between consecutive instructions of a thread
    int64_t k_bytes;       // uniform: global distance of one k step
    uint32_t voff;         // per thread
    uint32_t lds_off;      // uniform per wave: byte offset of this wave's first 1 KiB block in the tile
    int rows_left;         // BOUNDED: valid rows from this thread's first row on (may be <= 0)
    __device__ __forceinline__ DirectLoader(const Operand<T>& op, int r0, const void* zero_page = nullptr) {
        const int q = threadIdx.x, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int row = q / CPR, slot = q % CPR;
        if constexpr (KMAJOR) {
            const int chunk = slot ^ ((row >> 2) & 3);
            voff = (uint32_t)(((int64_t)global_row(row) * op.sr + chunk * 8) * 2);
            step_bytes = (int64_t)STEP * op.sr * 2;
            k_bytes = 2;
        } else {
            const int r = (slot * 8) ^ ((row & 3) << mn_swizzle_shift(ROWS));   // row = k within the pass
            voff = (uint32_t)(((int64_t)row * op.sk + r) * 2);
            step_bytes = (int64_t)STEP * op.sk * 2;
            k_bytes = op.sk * 2;
        }
        lds_off = (uint32_t)w * 1024u;
        zero = reinterpret_cast<const char*>(zero_page);
        move_to(op, r0);
    }
    // tile that starts at row r0 of the same operand
    __device__ __forceinline__ void move_to(const Operand<T>& op, int r0) {
        base = reinterpret_cast<const char*>(op.p + (KMAJOR ? (int64_t)r0 * op.sr : (int64_t)r0));
        rows_left = op.rows - r0 - global_row((int)threadIdx.x / CPR);
    }
    // stage starting at k0 -> tile at `lds_tile` (uniform)
    __device__ __forceinline__ void issue(int k0, T* lds_tile) const {
        typedef __attribute__((address_space(3))) void* lds_vp;
        typedef const __attribute__((address_space(1))) void* glb_vp;
        const char* g = base + (int64_t)k0 * k_bytes;
        char* l = reinterpret_cast<char*>(lds_tile) + lds_off;
#pragma unroll
        for (int i = 0; i < INSTR; ++i) {
            const char* src = g + i * step_bytes + voff;
            if constexpr (BOUNDED) src = i * STEP < rows_left ? src : zero;
            __builtin_amdgcn_global_load_lds((glb_vp)src, (lds_vp)(l + i * (THREADS * 16)), 16, 0, 0);
        }
    }
};

// ----------------------------------------------------------------------------- LDS -> fragments
// bf16: fragment of 32 rows x 16 k (one k-step `kk` of the stage) for rows rbase..rbase+31
template <bool KMAJOR, int ROWS>
__device__ __forceinline__ bf16x8_v load_frag_bf16(const bf16_t* lds, int rbase, int kk) {
    const int l = threadIdx.x & 63;
    if constexpr (KMAJOR) {
        const int r = rbase + (l & 31);
        const int chunk = 2 * kk + (l >> 5);
        const u32x4_v v = *reinterpret_cast<const u32x4_v*>(lds + r * 32 + ((chunk ^ ((r >> 2) & 3)) << 3));
        return __builtin_bit_cast(bf16x8_v, v);
    } else {
        constexpr int STRIDE = ROWS;
        const int b = l >> 4, s = l & 15;
        const int r = rbase + ((b & 1) << 4) + ((s & 3) << 2);
        const int k = kk * 16 + ((b >> 1) << 3) + (s >> 2);
        typedef __attribute__((address_space(3))) s16x4_v* lds_ptr;
        const bf16_t* p0 = lds + k * STRIDE + (r ^ ((k & 3) << mn_swizzle_shift(ROWS)));   // k and k+4 share the swizzle
        const s16x4_v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
        const s16x4_v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0 + 4 * STRIDE));
        s16x8_v v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(bf16x8_v, v);
    }
}

// The same fragment read written as assembly, for loops that keep global -> LDS loads in flight: a read the
// compiler can see is made to wait for every such load already requested (the compiler must assume that the
// load overwrites what is read; the stage ring rules that out), which would expose a full memory latency per
// stage.  issue() requests the fragment, ready() is called once the caller's own s_waitcnt lgkmcnt has covered
// it and ties the registers to that point, get() hands the fragment to the MFMA.
template <bool KMAJOR, int ROWS>
__device__ __forceinline__ uint32_t frag_offset_bf16(int rbase, int kk) {   // bytes from the operand tile's start
    const int l = threadIdx.x & 63;
    if constexpr (KMAJOR) {
        const int r = rbase + (l & 31);
        const int chunk = 2 * kk + (l >> 5);
        return 2u * (uint32_t)(r * 32 + ((chunk ^ ((r >> 2) & 3)) << 3));
    } else {
        const int b = l >> 4, s = l & 15;
        const int r = rbase + ((b & 1) << 4) + ((s & 3) << 2);
        const int k = kk * 16 + ((b >> 1) << 3) + (s >> 2);
        return 2u * (uint32_t)(k * ROWS + (r ^ ((k & 3) << mn_swizzle_shift(ROWS))));
    }
}
template <bool KMAJOR, int ROWS> struct FragRegsBf16;
template <int ROWS> struct FragRegsBf16<true, ROWS> {
    static constexpr int READS = 1;
    u32x4_v v;
    __device__ __forceinline__ void issue(uint32_t addr) { asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr)); }
    __device__ __forceinline__ void ready() { asm volatile("" : "+v"(v)); }
    __device__ __forceinline__ bf16x8_v get() const { return __builtin_bit_cast(bf16x8_v, v); }
};
template <int ROWS> struct FragRegsBf16<false, ROWS> {
    static constexpr int READS = 2;
    s16x4_v lo, hi;
    __device__ __forceinline__ void issue(uint32_t addr) {   // k and k + 4 share the swizzle
        asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %2 offset:%3"
                     : "=&v"(lo), "=&v"(hi) : "v"(addr), "n"(4 * ROWS * 2));
    }
    __device__ __forceinline__ void ready() { asm volatile("" : "+v"(lo), "+v"(hi)); }
    __device__ __forceinline__ bf16x8_v get() const {
        const s16x8_v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(bf16x8_v, both);
    }
};
template <int N> __device__ __forceinline__ void wait_lds_reads() {   // at most N of this wave's LDS reads outstanding
    static_assert(N >= 0 && N <= 15, "lgkmcnt range");
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N));
}

// fp32: 4 floats per lane covering one 8-k window `kw`: slot s <-> k = kw*8 + 4*(lane/32) + s
template <bool KMAJOR, int ROWS>
__device__ __forceinline__ void load_frag_f32(const float* lds, int rbase, int kw, float (&f)[4]) {
    const int l = threadIdx.x & 63;
    const int r = rbase + (l & 31), kb = kw * 8 + ((l >> 5) << 2);
    if constexpr (KMAJOR) {
        const float4 v = *reinterpret_cast<const float4*>(lds + r * GemmTraits<float>::kmajor_stride() + kb);
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
    } else {
        constexpr int STRIDE = ROWS + GemmTraits<float>::PAD_MN;
#pragma unroll
        for (int s = 0; s < 4; ++s) f[s] = lds[(kb + s) * STRIDE + r];
    }
}

// ----------------------------------------------------------------------------- tile -> C coordinates
// Tile `id` of `nb` = tiles_m * tiles_n tiles -> (tm, tn).  Workgroups walk the tiles in
// strides of the grid size (a multiple of 8 whenever there are more tiles than workgroups), so
// the tiles with id % 8 == x are all processed on XCD x (consecutive workgroup ids land on
// different XCDs, 8 of them, each with its own L2).  Ids are therefore first regrouped per XCD
// and then walked in groups of 8 tiles along m, which keeps the operand rows and columns that
// one L2 sees close together.
__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int nb = tiles_m * tiles_n;
    const int per = nb >> 3;
    const int lid = id < (per << 3) ? (id & 7) * per + (id >> 3) : id;
    constexpr int GROUP = 8;
    const int in_group = GROUP * tiles_n;
    const int first_m = (lid / in_group) * GROUP;
    const int gsize = min(tiles_m - first_m, GROUP);
    tm = first_m + (lid % in_group) % gsize;
    tn = (lid % in_group) / gsize;
}

// Workgroups of a persistent tile kernel: as many as stay resident at once, at most one per tile.
template <typename Kernel>
inline int persistent_grid(Kernel kernel, int threads, size_t lds_bytes, int64_t tiles) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds_bytes) != hipSuccess || per_cu < 1)
        per_cu = 1;
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    return (int)std::min<int64_t>(tiles, cus * per_cu);
}

// ----------------------------------------------------------------------------- mainloop
// Accumulates the (2*WM*32) x (2*WN*32) tile at (m0, n0).  acc[wm][wn][r] of lane l belongs to
//   m = m0 + wave_m*WM*32 + wm*32 + l%32,   n = n0 + wave_n*WN*32 + wn*32 + 8*(r/4) + 4*(l/32) + r%4.
// NWM x NWN waves per workgroup (along m, along n); wave w sits at (w % NWM, w / NWM).
// PERMUTE: on the direct-to-LDS path with a K-major A, the A rows of each wave are permuted
// (DirectLoader PERM_WM = WM) so that a lane owns WM consecutive m: m = lane_m + i.
template <typename T, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, bool FULL = false, int NWN = 2, int NSTAGES = 0,
          int NWM = 2, bool PERMUTE = false>
struct GemmMainloop {
    using Tr = GemmTraits<T>;
    static constexpr int THREADS = NWM * NWN * 64;
    static constexpr int TILE_M = NWM * WM * 32, TILE_N = NWN * WN * 32;
    using PlainLoaderA = TileLoader<T, A_KMAJOR, TILE_M, FULL, THREADS>;
    using PlainLoaderB = TileLoader<T, B_KMAJOR, TILE_N, FULL, THREADS>;
    static constexpr int A_ELEMS = lds_tile_elems<T, A_KMAJOR>(TILE_M);
    static constexpr int B_ELEMS = lds_tile_elems<T, B_KMAJOR>(TILE_N);
    static constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
    static constexpr bool DIRECT = FULL && sizeof(T) == 2;     // global -> LDS without registers
    static constexpr int NST = NSTAGES > 0 ? NSTAGES : (DIRECT ? 4 : 2);   // LDS stages
    static constexpr size_t LDS_BYTES = NST * (size_t)STAGE_ELEMS * sizeof(T);
    static constexpr int PERM_A = (PERMUTE && DIRECT && A_KMAJOR && WM > 1 && (THREADS / 4) % (32 * WM) == 0) ? WM : 0;
    static constexpr int M_STEP = PERM_A ? 1 : 32;            // distance in m between acc[i] and acc[i + 1] of a lane
    using DirectLoaderA = DirectLoader<A_KMAJOR, TILE_M, THREADS, false, PERM_A>;
    using DirectLoaderB = DirectLoader<B_KMAJOR, TILE_N, THREADS>;

    __device__ __forceinline__ static void run(const Operand<T>& A, const Operand<T>& B, int K, int m0, int n0, T* lds,
                                               f32x16_v (&acc)[WM][WN]) {
        if constexpr (FULL && sizeof(T) == 2) {
            run_direct(A, B, K, m0, n0, lds, acc);
        } else {
            PlainLoaderA la(A, m0, K);
            PlainLoaderB lb(B, n0, K);
            run(la, lb, K, lds, acc);
        }
    }

    __device__ __forceinline__ static void zero(f32x16_v (&acc)[WM][WN]) {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    }

    // All fragment reads of the stage are issued up front (LDS returns in order, so the MFMAs of
    // the first k-step start while the reads of the second are still in flight).
    __device__ __forceinline__ static void compute_bf16(const bf16_t* As, const bf16_t* Bs, int wave_m, int wave_n,
                                                        f32x16_v (&acc)[WM][WN]) {
        constexpr int KK = Tr::BK / 16;
        bf16x8_v fa[KK][WM], fb[KK][WN];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
            for (int j = 0; j < WN; ++j) fb[kk][j] = load_frag_bf16<B_KMAJOR, TILE_N>(Bs, wave_n + j * 32, kk);
#pragma unroll
            for (int i = 0; i < WM; ++i) fa[kk][i] = load_frag_bf16<A_KMAJOR, TILE_M>(As, wave_m + i * 32, kk);
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the reads ahead of the MFMAs (the scheduler would sink them to save registers)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
    }

    // Whole aligned bf16 tiles: stages go from global memory straight into LDS (no staging
    // registers, no ds_write).
    __device__ __forceinline__ static void run_direct(const Operand<T>& A, const Operand<T>& B, int K, int m0, int n0,
                                                      T* lds, f32x16_v (&acc)[WM][WN]) {
        DirectLoaderA la(A, m0);
        DirectLoaderB lb(B, n0);
        run_pipeline(la, lb, K, lds, acc);
    }

    // Direct-to-LDS pipeline over loaders with an issue(k0, lds_tile) method and INSTR loads per
    // thread and stage.  NST LDS stages: while stage kt is consumed, stages kt+1 .. kt+NST-2 are
    // in flight or landed and stage kt+NST-1 is issued into the buffer that stage kt-1 has just
    // left.  One barrier per stage.  K must be a multiple of BK.
    //   pipeline_fill : issues the first NST-1 stages of a tile.  All waves must have finished
    //                   reading the LDS stages of the previous tile (pipeline_drain).
    //   pipeline_loop : consumes all stages of the tile; acc is overwritten.
    // Other vector-memory operations of the wave that are still outstanding (the previous tile's
    // epilogue stores) only make the vmcnt waits more conservative: loads return in order.
    template <class LA, class LB>
    __device__ __forceinline__ static void pipeline_fill(const LA& la, const LB& lb, int K, T* lds) {
        static_assert(sizeof(T) == 2, "direct-to-LDS staging is implemented for bf16");
        const int KT = K / Tr::BK;
#pragma unroll
        for (int st = 0; st < NST - 1; ++st)
            if (st < KT) {
                la.issue(st * Tr::BK, lds + st * STAGE_ELEMS);
                lb.issue(st * Tr::BK, lds + st * STAGE_ELEMS + A_ELEMS);
            }
    }
    __device__ __forceinline__ static void pipeline_drain() {
        __builtin_amdgcn_s_waitcnt(0xF | (0x7 << 4) | (0x3 << 14));   // lgkmcnt(0): own LDS reads returned
        __builtin_amdgcn_s_barrier();
    }
    // The barrier of a stage sits between its k groups (16 k each), not in front of it: behind the barrier the
    // fragments of the next stage's first group are requested, then the MFMAs of this stage's last group run
    // while those reads are in flight; the matrix pipe does not drain at the stage boundary.
    template <class LA, class LB>
    __device__ __forceinline__ static void pipeline_loop(const LA& la, const LB& lb, int K, T* lds, f32x16_v (&acc)[WM][WN]) {
        const int w = threadIdx.x >> 6;
        const int wave_m = (w % NWM) * (WM * 32), wave_n = (w / NWM) * (WN * 32);
        zero(acc);
        constexpr int KK = Tr::BK / 16;
        static_assert(KK == 2, "a stage has two k groups");
        constexpr int IPS = LA::INSTR + LB::INSTR;               // load instructions per thread and stage
        constexpr int PENDING = (NST - 2) * IPS;                 // loads of later stages that may stay in flight
        static_assert(PENDING < 64, "vmcnt range");
        // s_waitcnt vmcnt(PENDING) lgkmcnt(0): expcnt left at its maximum; lgkmcnt(0) retires this wave's
        // LDS reads of the stage before the barrier lets other waves refill its buffer
        constexpr int WAIT_IMM = (PENDING & 0xF) | (0x7 << 4) | ((PENDING >> 4) << 14);
        const int KT = K / Tr::BK;
        using FA = FragRegsBf16<A_KMAJOR, TILE_M>;
        using FB = FragRegsBf16<B_KMAJOR, TILE_N>;
        constexpr int GROUP_READS = WM * FA::READS + WN * FB::READS;   // LDS read instructions of one k group
        static_assert(GROUP_READS <= 15, "lgkmcnt range");
        FA fa[KK][WM];
        FB fb[KK][WN];
        const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds);
        uint32_t off_a[KK][WM], off_b[KK][WN];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
            for (int i = 0; i < WM; ++i) off_a[kk][i] = lds_addr + frag_offset_bf16<A_KMAJOR, TILE_M>(wave_m + i * 32, kk);
#pragma unroll
            for (int j = 0; j < WN; ++j)
                off_b[kk][j] = lds_addr + (uint32_t)A_ELEMS * 2u + frag_offset_bf16<B_KMAJOR, TILE_N>(wave_n + j * 32, kk);
        }
        auto read = [&](int kk, int stage) {
            const uint32_t sb = (uint32_t)stage * (uint32_t)(STAGE_ELEMS * 2);
#pragma unroll
            for (int j = 0; j < WN; ++j) fb[kk][j].issue(off_b[kk][j] + sb);
#pragma unroll
            for (int i = 0; i < WM; ++i) fa[kk][i].issue(off_a[kk][i] + sb);
        };
        auto mma = [&](int kk) {                                 // the caller's wait has covered group kk
#pragma unroll
            for (int j = 0; j < WN; ++j) fb[kk][j].ready();
#pragma unroll
            for (int i = 0; i < WM; ++i) fa[kk][i].ready();
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[kk][j].get(), fa[kk][i].get(), acc[i][j], 0, 0, 0);
        };
        int cur = 0, fill = NST - 1;                             // buffer of stage kt, buffer to refill
        // stage 0 has landed (every wave's share: barrier); its first fragments
        if (NST - 2 < KT) __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        else __builtin_amdgcn_s_waitcnt(0);                      // fewer stages than the pipeline holds
        __builtin_amdgcn_s_barrier();
        read(0, 0);
        for (int kt = 0; kt < KT; ++kt) {
            // the buffer of stage kt - 1 was released at that stage's barrier
            if (kt + NST - 1 < KT) {
                la.issue((kt + NST - 1) * Tr::BK, lds + fill * STAGE_ELEMS);
                lb.issue((kt + NST - 1) * Tr::BK, lds + fill * STAGE_ELEMS + A_ELEMS);
            }
            read(1, cur);
            wait_lds_reads<GROUP_READS>();                       // the first group is in, the second may be on its way
            mma(0);
            __builtin_amdgcn_sched_barrier(0);
            cur = cur + 1 == NST ? 0 : cur + 1;
            fill = fill + 1 == NST ? 0 : fill + 1;
            if (kt + 1 < KT) {
                // stage kt + 1 has landed, this wave's reads of stage kt have returned
                if (kt + NST - 1 < KT) __builtin_amdgcn_s_waitcnt(WAIT_IMM);
                else __builtin_amdgcn_s_waitcnt(0);              // tail: fewer stages are in flight
                // bare barrier: __syncthreads() would add a fence that drains every load in flight
                __builtin_amdgcn_s_barrier();
                read(0, cur);
            } else {
                wait_lds_reads<0>();
            }
            mma(1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    template <class LA, class LB>
    __device__ __forceinline__ static void run_pipeline(const LA& la, const LB& lb, int K, T* lds, f32x16_v (&acc)[WM][WN]) {
        pipeline_fill(la, lb, K, lds);
        pipeline_loop(la, lb, K, lds, acc);
    }

    // k range [0, K) in stages of BK; the loaders decide what a stage contains
    template <class LoaderA, class LoaderB>
    __device__ __forceinline__ static void run(LoaderA& la, LoaderB& lb, int K, T* lds, f32x16_v (&acc)[WM][WN]) {
        static_assert(LoaderA::KMAJOR == A_KMAJOR && LoaderB::KMAJOR == B_KMAJOR, "loader layout mismatch");
        const int w = threadIdx.x >> 6;
        const int wave_m = (w % NWM) * (WM * 32), wave_n = (w / NWM) * (WN * 32);
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

        const int KT = (K + Tr::BK - 1) / Tr::BK;
        auto compute = [&](const T* As, const T* Bs) {
            if constexpr (sizeof(T) == 2) {
#pragma unroll
                for (int kk = 0; kk < Tr::BK / 16; ++kk) {
                    bf16x8_v fa[WM], fb[WN];
#pragma unroll
                    for (int i = 0; i < WM; ++i) fa[i] = load_frag_bf16<A_KMAJOR, TILE_M>(As, wave_m + i * 32, kk);
#pragma unroll
                    for (int j = 0; j < WN; ++j) fb[j] = load_frag_bf16<B_KMAJOR, TILE_N>(Bs, wave_n + j * 32, kk);
#pragma unroll
                    for (int i = 0; i < WM; ++i)
#pragma unroll
                        for (int j = 0; j < WN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int kw = 0; kw < Tr::BK / 8; ++kw) {
                    float fa[WM][4], fb[WN][4];
#pragma unroll
                    for (int i = 0; i < WM; ++i) load_frag_f32<A_KMAJOR, TILE_M>(As, wave_m + i * 32, kw, fa[i]);
#pragma unroll
                    for (int j = 0; j < WN; ++j) load_frag_f32<B_KMAJOR, TILE_N>(Bs, wave_n + j * 32, kw, fb[j]);
#pragma unroll
                    for (int s = 0; s < 4; ++s)
#pragma unroll
                        for (int i = 0; i < WM; ++i)
#pragma unroll
                            for (int j = 0; j < WN; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][s], fa[i][s], acc[i][j], 0, 0, 0);
                }
            }
        };
        // Global loads run two stages ahead of the MFMAs (two register sets), LDS is double
        // buffered: while stage kt is consumed from one LDS buffer, stage kt+1 waits in the
        // first register set for its LDS slot and stage kt+2 is in flight into the second.
        LoaderA la2 = la;
        LoaderB lb2 = lb;
        T* buf0 = lds;
        T* buf1 = lds + STAGE_ELEMS;
        la.load(0);
        lb.load(0);
        la.store(buf0);
        lb.store(buf0 + A_ELEMS);
        if (KT > 1) { la.load(Tr::BK); lb.load(Tr::BK); }
        if (KT > 2) { la2.load(2 * Tr::BK); lb2.load(2 * Tr::BK); }
        __syncthreads();
        int kt = 0;
        for (; kt + 2 <= KT; kt += 2) {
            // even stage: buf0 holds kt, set 1 holds kt+1, set 2 holds kt+2
            compute(buf0, buf0 + A_ELEMS);
            la.store(buf1);
            lb.store(buf1 + A_ELEMS);
            if (kt + 3 < KT) { la.load((kt + 3) * Tr::BK); lb.load((kt + 3) * Tr::BK); }
            __syncthreads();
            // odd stage: buf1 holds kt+1, set 2 holds kt+2, set 1 holds kt+3
            compute(buf1, buf1 + A_ELEMS);
            if (kt + 2 < KT) {
                la2.store(buf0);
                lb2.store(buf0 + A_ELEMS);
                if (kt + 4 < KT) { la2.load((kt + 4) * Tr::BK); lb2.load((kt + 4) * Tr::BK); }
            }
            __syncthreads();
        }
        if (kt < KT) compute(buf0, buf0 + A_ELEMS);   // odd number of stages: the last one sits in buf0
    }

    // First m and n of this lane inside the tile at (m0, n0); element acc[i][j][r] belongs to
    // m = lane_m + M_STEP*i,  n = lane_n + 32*j + 8*(r/4) + r%4.
    __device__ __forceinline__ static int lane_m(int m0) {
        return m0 + ((threadIdx.x >> 6) % NWM) * (WM * 32) + (threadIdx.x & 31) * (PERM_A ? WM : 1);
    }
    __device__ __forceinline__ static int lane_n(int n0) {
        return n0 + ((threadIdx.x >> 6) / NWM) * (WN * 32) + (((threadIdx.x & 63) >> 5) << 2);
    }

    // Calls f(m, n, value) for every element of the tile owned by this lane.
    template <typename F>
    __device__ __forceinline__ static void for_each(const f32x16_v (&acc)[WM][WN], int m0, int n0, F&& f) {
        const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
        const int mb = lane_m(m0);
        const int nb = n0 + (w / NWM) * (WN * 32) + ((l >> 5) << 2);
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) f(mb + i * M_STEP, nb + j * 32 + ((r >> 2) << 3) + (r & 3), acc[i][j][r]);
    }
};

}  // namespace luxhip
