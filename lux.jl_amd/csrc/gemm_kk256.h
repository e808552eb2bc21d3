// bf16 GEMM for large problems with both operands K-major (k contiguous): 256 x 256 tiles on eight
// waves, K consumed in steps of 64.
//
// What shapes this kernel (all measured on the device):
//   * the global -> LDS stream is the scarcest resource.  A row segment of 128 bytes (one cache line)
//     per row and step moves 20 % more bytes per second than two segments of 64, so a step covers
//     64 k, and an operand tile of a step is one "block" of 256 rows x 128 bytes = 32 KiB;
//   * LDS holds a ring of five blocks (the whole 160 KiB): the two blocks of the step being consumed,
//     the two of the next step and the A block of the step after;
//   * loads issued in bursts at the step boundary queue up behind each other in the memory system and
//     come back late; one load instruction in front of every eight MFMAs keeps the stream even
//     (1450 -> 1740 TFLOP/s on 8192^3);
//   * fragment reads run one k group (16) ahead of the MFMAs, and the step's barrier sits before the
//     last quarter of its MFMAs, so the matrix pipe has work while the first reads of the next step
//     are in flight.
//
// LDS layout of a block: row r at r * 128 bytes, its eight 16-byte chunks XORed with (r / 2) % 8:
// the sixteen lanes that a ds_read_b128 serves together (lanes 0-3, 12-15, 20-23, 24-27 and so on)
// then fall into sixteen different bank groups.  Rows of A are permuted inside each wave's 128 rows
// (LDS row 16 j + u holds row 8 u + j) so that a lane of the accumulator owns eight consecutive m and
// stores them with one 16-byte instruction.
#pragma once

#include "common.h"
#include "gemm_core.h"
#include "gemm_dense_decl.h"

namespace luxhip {
namespace kk256 {

constexpr int THREADS = 512, TILE = 256, BK = 64, RING = 5;
constexpr int BLOCK_BYTES = TILE * BK * 2;                 // 32 KiB
constexpr size_t LDS_BYTES = (size_t)RING * BLOCK_BYTES;   // 160 KiB
constexpr int SM = 8, SN = 4;                              // 16 x 16 accumulator tiles per wave: 128 (m) x 64 (n)
typedef float f32x4_v __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) void* lds_vp;
typedef const __attribute__((address_space(1))) void* glb_vp;

// What the kernel reads of a DenseArgs (scalar registers are scarce in its loop).
struct Args {
    const bf16_t *A, *B, *bias;
    bf16_t *C, *pre;
    int64_t lda, ldb, ldc;      // elements
    int K, act, tiles_m, tiles_n;
};

// Keeps the compiler from hoisting everything derived from `v` out of the loops (it would hold one
// register per k group and operand for what is a single XOR at the point of use).
__device__ __forceinline__ uint32_t at_use(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

// One block: 256 rows x 128 bytes of a K-major operand, four load instructions per thread.  Thread q
// fills LDS row q / 8 + 64 i with instruction i.  PERM: LDS row 16 u + j of a wave's 128 rows holds row
// 8 j + u of the tile, which makes instruction i fetch tile row g + {0, 4, 128, 132}[i] for the thread's
// g; without it row q / 8 + 64 i.  Either way: one per-thread offset, and a uniform row distance per
// instruction that is added to the uniform pointer (tile base + k).
template <bool PERM>
struct BlockLoader {
    uint32_t voff;           // per thread: byte offset of its chunk of instruction 0 inside the tile at k = 0
    uint32_t lds_off;        // uniform per wave
    int64_t step[4];         // uniform: byte distance of instruction i's rows from instruction 0's
    __device__ __forceinline__ BlockLoader(int64_t ld) {
        const int q = threadIdx.x, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int row = q >> 3, slot = q & 7;                                      // LDS row of instruction 0
        const int chunk = slot ^ ((row >> 1) & 7);                                 // (row + 64 i) / 2 % 8 is the same for every i
        const int grow = PERM ? (((row & 15) << 3) | (row >> 4)) : row;
        voff = (uint32_t)(((int64_t)grow * ld + chunk * 8) * 2);
        lds_off = (uint32_t)w * 1024u;
#pragma unroll
        for (int i = 0; i < 4; ++i) step[i] = (PERM ? ((i & 1) * 4 + (i >> 1) * 128) : 64 * i) * ld * 2;
    }
    // instruction i of the block at `g` (uniform: tile base + k) -> LDS block `dst`
    __device__ __forceinline__ void issue(int i, const char* g, char* dst) const {
        // cache policy sc0 sc1 (the data is used once per compute unit: nothing is gained by keeping it in the
        // vector L1); measured 2.5-3.7 % faster than the default policy, the non-temporal policies 20 % slower
        __builtin_amdgcn_global_load_lds((glb_vp)(g + step[i] + at_use(voff)), (lds_vp)(dst + lds_off + i * 8192), 16, 0, 17);
    }
};

// C = act(acc + bias), optional pre-activation copy.  Lane l of wave (wm, wn) owns
//   m = m0 + wm * 128 + 8 * (l % 16) + i,  n = n0 + wn * 64 + 16 * j + 4 * (l / 16) + r   for acc[i][j][r].
template <int ACT_MODE, bool HAS_PRE>
__device__ __forceinline__ void epilogue_as(const f32x4_v (&acc)[SM][SN], const Args& a, int m0, int n0) {
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int mb = m0 + (w & 1) * 128 + 8 * (l & 15);
    const int nb = n0 + (w >> 1) * 64 + 4 * (l >> 4);
    float bv[SM];
    if (a.bias) {
        Vec<bf16_t>::load(a.bias + mb, bv);
    } else {
#pragma unroll
        for (int i = 0; i < SM; ++i) bv[i] = 0.0f;
    }
    const int act = a.act;
    static_for<SN * 4>([&](auto JR) {
        constexpr int j = decltype(JR)::value / 4, r = decltype(JR)::value % 4;
        const int n = nb + 16 * j + r;
        float v[SM];
#pragma unroll
        for (int i = 0; i < SM; ++i) v[i] = acc[i][j][r] + bv[i];
        if constexpr (HAS_PRE) Vec<bf16_t>::store(a.pre + (int64_t)n * a.ldc + mb, v);
        if constexpr (ACT_MODE == 1) act_vec_as<LUXHIP_ACT_RELU>(v);
        else if constexpr (ACT_MODE == 2) act_vec(act, v);
        Vec<bf16_t>::store(a.C + (int64_t)n * a.ldc + mb, v);
    });
}
__device__ __forceinline__ void epilogue(const f32x4_v (&acc)[SM][SN], const Args& a, int m0, int n0) {
    if (a.pre != nullptr) epilogue_as<2, true>(acc, a, m0, n0);
    else if (a.act == LUXHIP_ACT_IDENTITY) epilogue_as<0, false>(acc, a, m0, n0);
    else if (a.act == LUXHIP_ACT_RELU) epilogue_as<1, false>(acc, a, m0, n0);
    else epilogue_as<2, false>(acc, a, m0, n0);
}

// Persistent: workgroup b takes tiles b, b + gridDim.x, ...; the first blocks of the next tile are
// requested before the epilogue of the current one.
//
// Blocks of a tile: b = 2 s is the A block of step s, b = 2 s + 1 its B block; block b lives in ring slot
// b % 5.  Schedule of step kt (the same for every step, so the loop body has one branch, for the last step):
//   loads, two in front of every k group: block 2 kt + 3 (instructions 2, 3), block 2 kt + 4 (all four), and
//   behind the boundary block 2 kt + 5 (instructions 0, 1); the tile's prologue supplies blocks 0, 1, 2 and
//   the first half of block 3.  Blocks past the end of K are loaded all the same, from the last step's
//   columns (valid memory, a free slot, never read): no special cases for the tail.
//   boundary, before the last k group: every wave's reads of step kt have returned and the blocks of step
//   kt + 1 have landed (loads return in order: at most the four instructions of block 2 kt + 4 are left).
__global__ __launch_bounds__(THREADS) void dense_gemm_kk256_kernel(Args a) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    char* lds = reinterpret_cast<char*>(lds_raw);
    const int total = a.tiles_m * a.tiles_n;
    const int w = threadIdx.x >> 6;
    const int wave_m = (w & 1) * 128, wave_n = (w >> 1) * 64;
    const int KT = a.K / BK;
    const int64_t lda_b = a.lda * 2, ldb_b = a.ldb * 2;
    const int klast = (KT - 1) * BK * 2;                       // byte offset of the last step's columns

    int t = blockIdx.x, tm, tn;
    tile_coords(t, a.tiles_m, a.tiles_n, tm, tn);
    int m0 = tm * TILE, n0 = tn * TILE;
    const BlockLoader<true> la(a.lda);
    const BlockLoader<false> lb(a.ldb);
    const char* ga = reinterpret_cast<const char*>(a.A) + (int64_t)m0 * lda_b;      // uniform: the tile's rows, k = 0
    const char* gb = reinterpret_cast<const char*>(a.B) + (int64_t)n0 * ldb_b;
    // blocks 0, 1, 2 and the first half of block 3 of the tile at (ga, gb)
    auto issue_prologue = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) la.issue(i, ga, lds);
#pragma unroll
        for (int i = 0; i < 4; ++i) lb.issue(i, gb, lds + BLOCK_BYTES);
#pragma unroll
        for (int i = 0; i < 4; ++i) la.issue(i, ga + 128, lds + 2 * BLOCK_BYTES);
        lb.issue(0, gb + 128, lds + 3 * BLOCK_BYTES);
        lb.issue(1, gb + 128, lds + 3 * BLOCK_BYTES);
    };
    issue_prologue();

    // this lane's byte offset inside a block for k group 0 (its rows' swizzle does not depend on the fragment)
    const uint32_t lane15 = threadIdx.x & 15, laneq = (threadIdx.x & 63) >> 4;
    const uint32_t offA = (wave_m + lane15) * 128 + ((laneq ^ ((lane15 >> 1) & 7)) << 4);
    const uint32_t offB = (wave_n + lane15) * 128 + ((laneq ^ ((lane15 >> 1) & 7)) << 4);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds);   // LDS byte address

    f32x4_v acc[SM][SN];
    bf16x8_v fa[2][SM], fb[2][SN];
    for (;;) {
#pragma unroll
        for (int i = 0; i < SM; ++i)
#pragma unroll
            for (int j = 0; j < SN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
        // blocks 0 and 1 have landed: at most the six load instructions of blocks 2 and 3 are outstanding
        // (loads return in order; the previous tile's stores, issued after the prologue, only make the
        // count more conservative)
        __builtin_amdgcn_s_waitcnt(6 | (0x7 << 4));
        __builtin_amdgcn_s_barrier();

        // Fragment (16 rows x 32 k) of k group g: lane l reads row l % 16 of the fragment, chunk 4 g + l / 16,
        // swizzled: ((4 g + q) ^ s) << 4 = ((q ^ s) << 4) ^ (g << 6).  The reads are written as assembly:
        // left to the compiler, every read would be followed by a wait for *all* outstanding LDS reads before
        // the first MFMA, and by another before each global -> LDS load (which it must assume to overwrite what
        // is being read; the ring's barriers rule that out).  Their completion is awaited by frags_ready().
        // The reads of a fragment set come in two parts: the B fragments and the first four A fragments, then,
        // once the MFMAs have consumed half of the set in use, the last four A fragments into registers that
        // have just become free (twenty fragments live instead of twenty-four).
        auto reads_1 = [&](uint32_t slot_a, uint32_t slot_b, int g, int set) {
            const uint32_t aA = lds_addr + slot_a + (at_use(offA) ^ (uint32_t)(g << 6));
            const uint32_t aB = lds_addr + slot_b + (at_use(offB) ^ (uint32_t)(g << 6));
            asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:2048\n\tds_read_b128 %2, %4 offset:4096\n\tds_read_b128 %3, %4 offset:6144"
                         : "=&v"(fb[set][0]), "=&v"(fb[set][1]), "=&v"(fb[set][2]), "=&v"(fb[set][3]) : "v"(aB));
            asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:2048\n\tds_read_b128 %2, %4 offset:4096\n\tds_read_b128 %3, %4 offset:6144"
                         : "=&v"(fa[set][0]), "=&v"(fa[set][1]), "=&v"(fa[set][2]), "=&v"(fa[set][3]) : "v"(aA));
        };
        auto reads_2 = [&](uint32_t slot_a, int g, int set) {
            const uint32_t aA = lds_addr + slot_a + (at_use(offA) ^ (uint32_t)(g << 6));
            asm volatile("ds_read_b128 %0, %4 offset:8192\n\tds_read_b128 %1, %4 offset:10240\n\tds_read_b128 %2, %4 offset:12288\n\tds_read_b128 %3, %4 offset:14336"
                         : "=&v"(fa[set][4]), "=&v"(fa[set][5]), "=&v"(fa[set][6]), "=&v"(fa[set][7]) : "v"(aA));
        };
        // The twelve reads of `set` have returned when at most `younger` LDS reads issued after them are
        // outstanding (LDS reads return in order); naming the fragments as operands keeps their MFMAs behind
        // the wait.
#define KK256_READY(set, younger)                                                                                          \
        asm volatile("s_waitcnt lgkmcnt(" #younger ")"                                                                     \
                     : "+v"(fb[set][0]), "+v"(fb[set][1]), "+v"(fb[set][2]), "+v"(fb[set][3]), "+v"(fa[set][0]), "+v"(fa[set][1]), \
                       "+v"(fa[set][2]), "+v"(fa[set][3]), "+v"(fa[set][4]), "+v"(fa[set][5]), "+v"(fa[set][6]), "+v"(fa[set][7]))
        auto mfmas = [&](int set, int i0) {      // two rows of accumulator tiles: eight MFMAs
#pragma unroll
            for (int i = i0; i < i0 + 2; ++i)
#pragma unroll
                for (int j = 0; j < SN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
        };
#define KK256_FENCE() __builtin_amdgcn_sched_barrier(0)
        const int tnext = t + gridDim.x;
        int m0n = 0, n0n = 0;
        // ring slots (byte offsets) of the blocks of the current step and of those being loaded
        uint32_t sA = 0, sB = BLOCK_BYTES;                     // blocks 2 kt, 2 kt + 1
        auto next_slot = [](uint32_t s_, int by) {             // (slot + by) % RING in bytes, by < RING
            const uint32_t v = s_ + (uint32_t)by * BLOCK_BYTES;
            return v >= RING * BLOCK_BYTES ? v - RING * BLOCK_BYTES : v;
        };
        int k1 = 128, k2 = 256;                                // byte offsets of the columns of steps kt + 1, kt + 2
        reads_1(sA, sB, 0, 0);
        reads_2(sA, 0, 0);
        for (int kt = 0; kt < KT; ++kt) {
            const int k1c = min(k1, klast), k2c = min(k2, klast);
            char* const d3 = lds + next_slot(sA, 3);           // block 2 kt + 3: B of step kt + 1
            char* const d4 = lds + next_slot(sA, 4);           // block 2 kt + 4: A of step kt + 2
            reads_1(sA, sB, 1, 1);
            lb.issue(2, gb + k1c, d3);
            KK256_READY(0, 8);                                  // set 0 (both parts) is older than the eight reads above
            KK256_FENCE(); mfmas(0, 0); KK256_FENCE();
            lb.issue(3, gb + k1c, d3);
            KK256_FENCE(); mfmas(0, 2); KK256_FENCE();
            reads_2(sA, 1, 1);                                  // into the registers of the A fragments just used up
            la.issue(0, ga + k2c, d4);
            KK256_FENCE(); mfmas(0, 4); KK256_FENCE();
            la.issue(1, ga + k2c, d4);
            KK256_FENCE(); mfmas(0, 6); KK256_FENCE();
            la.issue(2, ga + k2c, d4);
            KK256_READY(1, 0);
            KK256_FENCE(); mfmas(1, 0); KK256_FENCE();
            la.issue(3, ga + k2c, d4);
            KK256_FENCE(); mfmas(1, 2); KK256_FENCE();
            // Boundary (the MFMAs stay outside every branch: accumulator tuples that differ between the arms
            // of a branch end up copied or spilled).
            if (kt + 1 < KT) {
                __builtin_amdgcn_s_waitcnt(4 | (0x7 << 4));     // vmcnt(4) lgkmcnt(0)
                __builtin_amdgcn_s_barrier();
                // block 2 kt + 5 (B of step kt + 2) takes the slot of the A block just released
                lb.issue(0, gb + k2c, lds + sA);
                const uint32_t freed = sA;
                sA = next_slot(sA, 2);
                sB = next_slot(sB, 2);
                reads_1(sA, sB, 0, 0);
                reads_2(sA, 0, 0);
                KK256_FENCE(); mfmas(1, 4); KK256_FENCE();
                lb.issue(1, gb + k2c, lds + freed);
            } else {
                // last step: nothing of this tile may still be on its way into the ring (the loads past the end
                // of K) when the next tile's blocks are requested, and every wave has read its last fragments
                __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));     // vmcnt(0) lgkmcnt(0)
                __builtin_amdgcn_s_barrier();
                if (tnext < total) {
                    tile_coords(tnext, a.tiles_m, a.tiles_n, tm, tn);
                    m0n = tm * TILE;
                    n0n = tn * TILE;
                    ga = reinterpret_cast<const char*>(a.A) + (int64_t)m0n * lda_b;
                    gb = reinterpret_cast<const char*>(a.B) + (int64_t)n0n * ldb_b;
                    issue_prologue();
                }
                KK256_FENCE(); mfmas(1, 4); KK256_FENCE();
            }
            k1 += 128;
            k2 += 128;
            KK256_FENCE(); mfmas(1, 6); KK256_FENCE();
        }
#undef KK256_READY
#undef KK256_FENCE
        epilogue(acc, a, m0, n0);
        if (tnext >= total) break;
        t = tnext; m0 = m0n; n0 = n0n;
    }
}

// The kernel's conditions: whole tiles, K in whole steps and long enough to fill the ring, 16-byte
// loads of the bias and stores of eight consecutive m.
inline bool applicable(const DenseArgs<bf16_t>& a) {
    const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    return a.M % TILE == 0 && a.N % TILE == 0 && a.K % BK == 0 && a.K >= 2 * BK && a.A.sk == 1 && a.B.sk == 1 && a.A.vec_ok &&
           a.B.vec_ok && al16(a.C) && al16(a.pre) && al16(a.bias) && a.ldc % 8 == 0 &&
           256 * a.A.sr * 2 < (int64_t(1) << 31) && 256 * a.B.sr * 2 < (int64_t(1) << 31);
}

inline int launch(hipStream_t s, DenseArgs<bf16_t>& a) {
    a.tiles_m = a.M / TILE;
    a.tiles_n = a.N / TILE;
    static ResidentOnce ro;
    ro.get([&](hipError_t& err) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(dense_gemm_kk256_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)LDS_BYTES);
        return 1;
    });
    LUX_CHECK_HIP(ro.error);
    const int64_t cus = num_cus() > 0 ? num_cus() : 256;
    const int grid = (int)std::min<int64_t>((int64_t)a.tiles_m * a.tiles_n, cus);   // the ring fills the LDS: one workgroup per compute unit
    Args k;
    k.A = a.A.p; k.B = a.B.p; k.bias = a.bias; k.C = a.C; k.pre = a.pre;
    k.lda = a.A.sr; k.ldb = a.B.sr; k.ldc = a.ldc;
    k.K = a.K; k.act = a.act; k.tiles_m = a.tiles_m; k.tiles_n = a.tiles_n;
    ProfScope ps(a.tail ? "dense_gemm_kernel<bf16>+tail" : "dense_gemm_kernel<bf16>", s);
    dense_gemm_kk256_kernel<<<dim3((unsigned)grid), dim3(THREADS), LDS_BYTES, s>>>(k);
    LUX_CHECK_LAUNCH();
    return LUXHIP_OK;
}

}  // namespace kk256
}  // namespace luxhip
