// bf16 3 x 3 convolution (fprop and dgrad) for unit stride, unit dilation and "same" output size, with the
// input window of a tile held in LDS: 256 or 272 output positions x 128 output channels per tile on eight waves.
//
// An implicit GEMM that gathers its A operand per filter tap reads every input element nine times from
// L2; here a tile first brings the rows of the image that it needs ("patch": the rows of its output
// positions plus the halo, 64 channels at a time) into LDS once, and the nine taps read it at shifted
// addresses.  What is left of the global -> LDS stream is the patch (about 6.5 KiB per step instead of
// 32 KiB) and the filter slice of the step (16 KiB).
//
// LDS (160 KiB, one workgroup per compute unit):
//   two patch buffers of 464 positions x 128 bytes (64 channels) + 2 KiB of zeros each, used in turn by the
//   successive 64-channel parts ("halves") of the successive tiles: while the taps of one half are
//   multiplied, the next half (of the same tile or of the workgroup's next tile) is loaded; the zeros are read
//   in place of a patch row above or below the image;
//   a ring of five filter half-blocks (64 output channels x 64 k = 8 KiB each, rows of 128 bytes with their
//   16-byte chunks XORed with (row / 2) % 8); a step (one tap of one half, 64 k) consumes two, one per half
//   of the waves, and the loads run three to four half-blocks ahead: a step requests the first half-block of
//   the step after the next between its MFMAs and the second one right behind its barrier.
//
// Patch layout: position x = pr * pitch + pc (row pr, column pc of the patch, pitch = P + 2 with zero-filled halo
// columns) belongs to the group x / 16 of 2 KiB, which holds its sixteen positions chunk by chunk: 16-byte chunk
// c of position x at (x / 16) * 2048 + c * 256 + (x % 16) * 16.  The sixteen lanes that read one chunk of
// sixteen consecutive positions then touch sixteen different 16-byte columns of the banks wherever the run
// starts: no tap and no wrap into the next image row causes a bank conflict, and the second k group of a
// step (chunks 4-7) is the same address + 1024.  The zeros behind a buffer are its "group 29": a tap row
// outside the image is read at position 464.  Per tile a lane keeps the position of each of its four output
// positions under each of the three tap rows (or 464); a tap's address is three instructions from there.
//
// Work split: the output positions are cut into runs of 16 ("fragments"), every workgroup takes the same number
// of consecutive fragments (one more for the first few) and cuts its share into tiles of at most 17: 12544
// fragments on 256 compute units are 49 each, three tiles of 17 + 16 + 16, where tiles of 16 dealt out in turn
// would leave 240 compute units idle for a quarter of the time.  The seventeenth fragment of a tile is
// multiplied by two waves on different SIMDs on top of their own four.
//
// One step: 32 MFMAs 16x16x32 per wave (wave tile 64 positions x 64 channels, two k groups of 32); the
// fragments of a k group are read while the MFMAs of the one before run; the step's barrier sits before its
// last eight MFMAs; a load instruction in front of every eight MFMAs.  The nine taps of a half are unrolled.
#pragma once

#include "common.h"
#include "gemm_core.h"

namespace luxhip {
namespace cpatch {

constexpr int THREADS = 512, TILE_N = 128, TAPS = 9;
constexpr int MAX_FRAGS = 17, TILE_M_MAX = 16 * MAX_FRAGS;           // fragments of 16 output positions per tile
constexpr int PATCH_PIX = 464, PATCH_BYTES = PATCH_PIX * 128;          // 59392: 29 groups of 16 positions
constexpr int ZERO_REL = PATCH_BYTES, ZERO_BYTES = 2048;               // behind each patch buffer
constexpr int BUF_STRIDE = PATCH_BYTES + ZERO_BYTES;                   // 61440
constexpr int RING_OFF = 2 * BUF_STRIDE, HB_BYTES = 8192, RING = 5;    // 122880
constexpr size_t LDS_BYTES = (size_t)RING_OFF + (size_t)RING * HB_BYTES;   // 163840
constexpr int PATCH_INSTR = 8;                     // load instructions per thread and patch (58 blocks of 1 KiB on 8 waves)
typedef float f32x4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_vp;
typedef const __attribute__((address_space(1))) void* glb_vp;

struct Args {
    const bf16_t* src;       // channel-contiguous source (C, P, Q, N), first channel of the group
    const bf16_t* wm;        // filter rows of the group: [Ncols][9 * Cg], k = tap * Cg + channel
    const bf16_t* bias;      // or null; indexed with col_off + column
    bf16_t* out;             // (P, Q, Ctot_out, N)
    bf16_t* pre;             // or null
    const void* zero;        // 16 zero bytes in device memory
    int Ctot, Cg;            // channels of the source (all groups), of this group
    int P, Q, NQ, PQ, M;     // row length, rows per image, rows in all, positions per image, positions in all
    int kW, kH, H;           // filter extent, 64-channel parts of Cg
    int rev, hlo, dq_min;    // dgrad walks the taps backwards; halo columns on the left; first source row relative to the output row
    int pitch;               // P + kW - 1
    int Ncols, col_off, Ctot_out, act;
    int frags, groups_m, tiles_n;   // fragments of 16 positions in all; workgroups that share them; tiles along the output channels
    int staged;                     // the epilogue may go through LDS: PQ % 8 == 0, no pre-activation output, out 16-byte aligned
    FastDiv divP, divQ, divPQ, divPitch;
};

// The kernel is compiled by the one source file that defines LUXHIP_CONV_PATCH_KERNEL.
#ifdef LUXHIP_CONV_PATCH_KERNEL
__device__ __forceinline__ uint32_t at_use(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

// ANY_ACT false: identity or relu only.  The epilogue is unrolled over the accumulator tiles, and with every activation
// inlined into each copy the kernel grows to several times the instruction cache, which the workgroup then refills
// from L2 after every tile.
template <bool ANY_ACT>
__global__ __launch_bounds__(THREADS) void conv_patch_kernel(Args a) {
    extern __shared__ __align__(128) unsigned char lds_raw[];
    char* lds = reinterpret_cast<char*>(lds_raw);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds);   // LDS byte address
    const int tid = threadIdx.x, l = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = (w & 3) * 64, wave_n = (w >> 2) * 64;
    // this workgroup's fragments [frag0, frag0 + nfrag) and its tiles
    const int bm = blockIdx.x % a.groups_m, tn = blockIdx.x / a.groups_m;
    const int fbase = a.frags / a.groups_m, frem = a.frags % a.groups_m;
    const int frag0 = bm * fbase + min(bm, frem), nfrag = fbase + (bm < frem ? 1 : 0);
    const int ntile = (nfrag + MAX_FRAGS - 1) / MAX_FRAGS, tbase = nfrag / ntile, trem = nfrag % ntile;
    // tile i: first output position and number of fragments
    auto tile_first = [&](int i) { return 16 * (frag0 + i * tbase + min(i, trem)); };
    auto tile_frags = [&](int i) { return tbase + (i < trem ? 1 : 0); };
    const int Cg2 = a.Cg * 2;                                        // bytes of a tap's channels in a filter row
    const int K2 = TAPS * Cg2;                                       // bytes of a filter row
    const int64_t row_bytes = (int64_t)a.P * a.Ctot * 2;             // bytes of an image row of the source

    if (tid < 2 * (ZERO_BYTES / 16)) {
        const int b = tid / (ZERO_BYTES / 16), i = tid % (ZERO_BYTES / 16);
        *reinterpret_cast<u32x4_v*>(lds + b * BUF_STRIDE + ZERO_REL + i * 16) = u32x4_v{0u, 0u, 0u, 0u};
    }

    // ---- patch loader: instruction i of this thread fills 1 KiB block g = w + 8 i (the last instruction: blocks
    // 56 and 57, four waves each, the same bytes): positions 16 (g / 2) + l % 16, chunk 4 (g % 2) + l / 16
    int32_t poff[PATCH_INSTR], prv[PATCH_INSTR];
#pragma unroll
    for (int i = 0; i < PATCH_INSTR; ++i) {
        const int g = i < PATCH_INSTR - 1 ? w + 8 * i : 56 + (w & 1);
        const int x = 16 * (g >> 1) + (l & 15), c = 4 * (g & 1) + (l >> 4);
        const int pr = (int)a.divPitch.div((uint32_t)x), pc = x - pr * a.pitch;
        const int ps = pc - a.hlo;
        poff[i] = ((pr * a.P + ps) * a.Ctot + 8 * c) * 2;
        prv[i] = (unsigned)ps < (unsigned)a.P ? pr : -(1 << 28);     // a halo column never passes the row test
    }
    // pb: source bytes of row `rbase`, column 0, first channel of the half; the patch rows are rbase, rbase + 1, ...
    auto patch_issue = [&](int i, const char* pb, int rbase, int buf) {
        const bool valid = (unsigned)(rbase + prv[i]) < (unsigned)a.NQ;
        const char* q = pb + (int32_t)at_use((uint32_t)poff[i]);
        const void* p = valid ? static_cast<const void*>(q) : a.zero;
        const int g = i < PATCH_INSTR - 1 ? w + 8 * i : 56 + (w & 1);
        __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(lds + buf * BUF_STRIDE + g * 1024), 16, 0, 0);
    };
    auto patch_base = [&](int tile, int h, int& rbase) -> const char* {
        rbase = (int)a.divP.div((uint32_t)tile_first(tile)) + a.dq_min;
        return reinterpret_cast<const char*>(a.src) + (int64_t)rbase * row_bytes + h * 128;
    };

    // ---- filter loader: one instruction per thread and half-block (64 rows: row tid / 8, 16-byte chunk tid % 8);
    // rows past the last output channel read the last one's (their products go to columns that are never stored)
    const int last_row = a.Ncols - 1 - tn * TILE_N;                  // of this workgroup's (up to 128) output channels
    const int brow0 = min(tid >> 3, last_row), brow1 = min(64 + (tid >> 3), last_row);
    const uint32_t bchunk = (uint32_t)(((tid & 7) ^ (((tid >> 3) >> 1) & 7)) << 4);
    const uint32_t boff0 = (uint32_t)(brow0 * K2) + bchunk, boff1 = (uint32_t)(brow1 * K2) + bchunk;
    int ring_b = 0;
    // half-block `hb` (0: rows 0-63, 1: rows 64-127) of the step whose columns start at gp
    auto filter_issue = [&](const char* gp, int hb) {
        __builtin_amdgcn_global_load_lds((glb_vp)(gp + at_use(hb ? boff1 : boff0)), (lds_vp)(lds + RING_OFF + ring_b * HB_BYTES + w * 1024), 16, 0,
                                         0);
        ring_b = ring_b + 1 == RING ? 0 : ring_b + 1;
    };
    // filter bytes of this workgroup's columns, first channel, tap 0
    const char* const gp_first = reinterpret_cast<const char*>(a.wm) + (int64_t)tn * TILE_N * K2;

    // ---- fragment reads
    const uint32_t lane15 = l & 15, laneq = l >> 4;
    // B: row 16 j + l % 16 of the wave's half-block, chunk 4 g + l / 16 for k group g (g = 1: XOR 64)
    const uint32_t offB = (uint32_t)(lane15 * 128 + ((laneq ^ ((lane15 >> 1) & 7)) << 4));

    // the bias of this lane's four columns (channel n0 + wave_n + 16 j + l % 16), read once: a load inside the epilogue
    // would have to wait for the stores issued before it
    float bias_v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = tn * TILE_N + wave_n + 16 * j + (int)lane15;
        bias_v[j] = a.bias != nullptr && col < a.Ncols ? ld(a.bias + a.col_off + col) : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(bias_v[j]));       // the wait for these loads belongs here, before the tile loop
    int tile = 0;
    int hc = 0;                              // halves consumed so far by this workgroup: patch buffer hc & 1
    const char* gp_cur = gp_first;
    // prologue: the first patch, four filter half-blocks (steps 0 and 1)
    {
        int rbase;
        const char* pb = patch_base(tile, 0, rbase);
#pragma unroll
        for (int i = 0; i < PATCH_INSTR; ++i) patch_issue(i, pb, rbase, 0);
        filter_issue(gp_cur, 0);
        filter_issue(gp_cur, 1);
        filter_issue(gp_cur + Cg2, 0);
        filter_issue(gp_cur + Cg2, 1);
    }
    const bool upper = wave_n != 0;          // this wave's columns are in the second half-block of a step
    // the two waves (on different SIMDs) that take the seventeenth fragment of a tile, one per half of the columns
    const bool extra_wave = w == 3 || w == 6;
    int slot0 = 0, slot1 = 1;                // ring slots of the two half-blocks of the current step

    f32x4_v acc[4][4], accE[4];
    bf16x8_v fa[2][4], fb[2][4], faE[2];
    for (;;) {
        const int m0 = tile_first(tile), n0 = tn * TILE_N;
        const int m_end = min(a.M, m0 + 16 * tile_frags(tile));
        const bool extra = extra_wave && tile_frags(tile) > 16;
        const int r_first = (int)a.divP.div((uint32_t)m0);
        const int tnext = tile + 1;
        const int total = ntile;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) accE[j][r] = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
        // this lane's patch positions: fragment f (output position m0 + wave_m + 16 f + l % 16) under tap row jb, first
        // tap column; 464 (the zeros) where that row lies outside the image
        uint32_t xrow[5][3];
#pragma unroll
        for (int f = 0; f < 5; ++f) {
            const int m = m0 + (f < 4 ? wave_m + 16 * f : 256) + (int)lane15;
            const int mc = min(m, a.M - 1);
            const int R = (int)a.divP.div((uint32_t)mc), p = mc - R * a.P;
            const int q = R - (int)a.divQ.div((uint32_t)R) * a.Q;
            const int x0 = (R - r_first) * a.pitch + p;
#pragma unroll
            for (int jb = 0; jb < 3; ++jb) {
                const bool valid = m < a.M && (unsigned)(q + a.dq_min + jb) < (unsigned)a.Q;
                xrow[f][jb] = valid ? (uint32_t)(x0 + jb * a.pitch) : (uint32_t)PATCH_PIX;
            }
        }
        const uint32_t lq8 = laneq << 8;
        // LDS address of fragment f under tap t (k group 0; k group 1: + 1024) in the buffer at `bufbase`
        auto a_addr = [&](int f, int t, uint32_t bufbase) -> uint32_t {
            const int kb = t / 3, ka = t - 3 * kb;                               // kW = kH = 3
            const uint32_t x = at_use(xrow[f][a.rev ? 2 - kb : kb]) + (uint32_t)(a.rev ? 2 - ka : ka);
            return bufbase + (x << 4) + (__umul24(x >> 4, 1792u) + lq8);   // 24-bit multiply: full rate (the 32-bit one takes four times as long)
        };
#define CP_READ_A(set, a0, a1, a2, a3, OFF)                                                                         \
        asm volatile("ds_read_b128 %0, %4 offset:" #OFF "\n\tds_read_b128 %1, %5 offset:" #OFF "\n\tds_read_b128 %2, %6 offset:" #OFF \
                     "\n\tds_read_b128 %3, %7 offset:" #OFF                                                          \
                     : "=&v"(fa[set][0]), "=&v"(fa[set][1]), "=&v"(fa[set][2]), "=&v"(fa[set][3])                  \
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3))
#define CP_READ_B(set, ab)                                                                                          \
        asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:2048\n\tds_read_b128 %2, %4 offset:4096\n\t" \
                     "ds_read_b128 %3, %4 offset:6144"                                                              \
                     : "=&v"(fb[set][0]), "=&v"(fb[set][1]), "=&v"(fb[set][2]), "=&v"(fb[set][3]) : "v"(ab))
        // the eight reads of `set` have returned when at most `younger` LDS reads issued after them are outstanding
#define CP_READY(set, younger)                                                                                      \
        asm volatile("s_waitcnt lgkmcnt(" #younger ")"                                                              \
                     : "+v"(fa[set][0]), "+v"(fa[set][1]), "+v"(fa[set][2]), "+v"(fa[set][3]), "+v"(fb[set][0]),   \
                       "+v"(fb[set][1]), "+v"(fb[set][2]), "+v"(fb[set][3]))
#define CP_FENCE() __builtin_amdgcn_sched_barrier(0)
        // the seventeenth fragment: one more read behind the eight of a set (so the waits above cover it), four more MFMAs
#define CP_READ_E(set, ae, OFF) asm volatile("ds_read_b128 %0, %1 offset:" #OFF : "=&v"(faE[set]) : "v"(ae))
#define CP_MFMA_E(set)                                                                                               \
        do {                                                                                                        \
            asm volatile("" : "+v"(faE[set]));                                                                      \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                           \
                accE[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(faE[set], fb[set][j], accE[j], 0, 0, 0);          \
        } while (0)
        auto mfmas = [&](int set, int i0) {      // two rows of accumulator tiles: eight MFMAs
#pragma unroll
            for (int i = i0; i < i0 + 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
        };

        // the patch of the first half and the two half-blocks of the first step have landed: of the loads
        // issued so far at most the two youngest (the half-blocks of the second step) are outstanding
        __builtin_amdgcn_s_waitcnt(2 | (0x7 << 4));          // vmcnt(2) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();

        uint32_t aA[5], aN[5];
        {
            const uint32_t bufbase = lds_addr + (uint32_t)(hc & 1) * BUF_STRIDE;
#pragma unroll
            for (int f = 0; f < 5; ++f) aA[f] = a_addr(f, 0, bufbase);
        }
        CP_READ_A(0, aA[0], aA[1], aA[2], aA[3], 0);
        CP_READ_B(0, lds_addr + RING_OFF + (uint32_t)(upper ? slot1 : slot0) * HB_BYTES + at_use(offB));
        if (extra) CP_READ_E(0, aA[4], 0);

        for (int h = 0; h < a.H; ++h) {
            // the half after this one: where its patch and its filter blocks come from
            int h_p = h + 1, tile_p = tile;
            if (h_p == a.H) { h_p = 0; tile_p = tnext; }
            const bool have_p = tile_p < total;
            int rbase_p = 0;
            const char* pb_p = nullptr;
            const char* gp_next = gp_cur;                    // past the last tile: the same blocks again, never read
            if (have_p) {
                pb_p = patch_base(tile_p, h_p, rbase_p);
                gp_next = h_p != 0 ? gp_cur + 128 : gp_first;
            }
            const uint32_t buf_cur = lds_addr + (uint32_t)(hc & 1) * BUF_STRIDE, buf_next = lds_addr + (uint32_t)((hc + 1) & 1) * BUF_STRIDE;
            static_for<TAPS>([&](auto TT) {
                constexpr int t = decltype(TT)::value;
                CP_READ_A(1, aA[0], aA[1], aA[2], aA[3], 1024);
                CP_READ_B(1, lds_addr + RING_OFF + (uint32_t)(upper ? slot1 : slot0) * HB_BYTES + (at_use(offB) ^ 64u));
                if (extra) CP_READ_E(1, aA[4], 1024);
                CP_READY(0, 8);
                CP_FENCE(); mfmas(0, 0); CP_FENCE();
                {
                    const uint32_t nb = t + 1 < TAPS ? buf_cur : buf_next;
#pragma unroll
                    for (int f = 0; f < 5; ++f) aN[f] = a_addr(f, (t + 1) % TAPS, nb);
                }
                CP_FENCE(); mfmas(0, 2); CP_FENCE();
                if (extra) CP_MFMA_E(0);
                CP_FENCE();
                // first half-block of the step after the next
                filter_issue(t + 2 < TAPS ? gp_cur + (t + 2) * Cg2 : gp_next + (t + 2 - TAPS) * Cg2, 0);
                CP_READY(1, 0);
                CP_FENCE(); mfmas(1, 0); CP_FENCE();
                // boundary: every wave's reads of this step have returned, and everything that the next step reads
                // has landed (loads return in order: only the half-block requested last may be outstanding)
                __builtin_amdgcn_s_waitcnt(1 | (0x7 << 4));      // vmcnt(1) lgkmcnt(0)
                __builtin_amdgcn_s_barrier();
                // Requested first thing behind the barrier, so that they have a whole step to arrive (the boundary of the
                // next step waits for them): the second half-block of the step after the next, into the slot this
                // barrier has released, and a block of the next half's patch.
                filter_issue(t + 2 < TAPS ? gp_cur + (t + 2) * Cg2 : gp_next + (t + 2 - TAPS) * Cg2, 1);
                if constexpr (t < PATCH_INSTR) {
                    if (have_p) patch_issue(t, pb_p, rbase_p, (hc + 1) & 1);
                }
                slot0 = slot0 + 2 >= RING ? slot0 + 2 - RING : slot0 + 2;
                slot1 = slot1 + 2 >= RING ? slot1 + 2 - RING : slot1 + 2;
                CP_READ_A(0, aN[0], aN[1], aN[2], aN[3], 0);
                CP_READ_B(0, lds_addr + RING_OFF + (uint32_t)(upper ? slot1 : slot0) * HB_BYTES + at_use(offB));
                CP_FENCE(); mfmas(1, 2); CP_FENCE();
                if (extra) {
                    // the set's reads were complete at the boundary; its registers are not among those just requested
                    CP_MFMA_E(1);
                    CP_READ_E(0, aN[4], 0);
                }
                CP_FENCE();
#pragma unroll
                for (int f = 0; f < 5; ++f) aA[f] = aN[f];
            });
            ++hc;
            gp_cur = gp_next;
        }

        // ---- epilogue: lane l owns positions m0 + wave_m + 16 i + 4 (l / 16) + r and channel n0 + wave_n + 16 j + l % 16
        if (a.staged) {
            // Through LDS, sixteen channels at a time, so that a store instruction writes whole 128-byte lines (64
            // positions of a channel) instead of sixteen pieces of 32 bytes: the wave's 2304 bytes lie in the patch
            // buffer of the half just finished, which nobody reads after that half's last boundary and which the
            // loads of the half after the next only enter behind the next tile's first barrier.  Rows of 144 bytes
            // (64 positions + 16 bytes) keep the writes (lane l: channel l % 16) and the reads (lane l: channel l / 8
            // and l / 8 + 8, positions 8 (l % 8) .. + 7) free of bank conflicts.
            char* st = lds + ((hc - 1) & 1) * BUF_STRIDE + w * 2304;
            const int mq = m0 + wave_m + 8 * (l & 7);
            const bool qok = mq < m_end;                                // m_end and PQ are multiples of 8 here
            const int img = (int)a.divPQ.div((uint32_t)(qok ? mq : 0));
            const uint32_t rowoffq = (uint32_t)(mq - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img;
            const int act = a.act;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = bias_v[j];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = acc[i][j][r] + b;
                    if (act == LUXHIP_ACT_RELU) act_vec_as<LUXHIP_ACT_RELU>(v);
                    else if constexpr (ANY_ACT) { if (act != LUXHIP_ACT_IDENTITY) act_vec(act, v); }
                    uint2 ov;
                    ov.x = f32x2_to_bf16x2(v[0], v[1]);
                    ov.y = f32x2_to_bf16x2(v[2], v[3]);
                    *reinterpret_cast<uint2*>(st + lane15 * 144 + (16 * i + 4 * laneq) * 2) = ov;
                }
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const int c = (l >> 3) + 8 * hh;
                    const uint4 val = *reinterpret_cast<const uint4*>(st + c * 144 + (l & 7) * 16);
                    const int col = n0 + wave_n + 16 * j + c;
                    if (qok && col < a.Ncols)
                        *reinterpret_cast<uint4*>(a.out + ((uint32_t)a.PQ * (uint32_t)(a.col_off + col) + rowoffq)) = val;
                }
            }
        } else {
            const int mrow = m0 + wave_m + 4 * (int)laneq;
            const int ncol = n0 + (upper ? 64 : 0) + (int)lane15;
            // element offsets inside one image's block of the output fit 32 bits (the tensor has fewer than 2^31 elements)
            uint32_t rowoff[4];
            bool mok[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = mrow + 16 * i;
                mok[i] = m < m_end;                                    // m_end and PQ are multiples of 4: all four or none
                const int img = (int)a.divPQ.div((uint32_t)(mok[i] ? m : 0));
                rowoff[i] = (uint32_t)(m - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img;
            }
            const int act = a.act;
            const bool has_pre = a.pre != nullptr;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = ncol + 16 * j;
                if (col < a.Ncols) {
                    const float b = bias_v[j];
                    const uint32_t coloff = (uint32_t)a.PQ * (uint32_t)(a.col_off + col);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (!mok[i]) continue;
                        float v[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = acc[i][j][r] + b;
                        if (has_pre) {
                            uint2 pv;
                            pv.x = f32x2_to_bf16x2(v[0], v[1]);
                            pv.y = f32x2_to_bf16x2(v[2], v[3]);
                            *reinterpret_cast<uint2*>(a.pre + (coloff + rowoff[i])) = pv;
                        }
                        if (act == LUXHIP_ACT_RELU) act_vec_as<LUXHIP_ACT_RELU>(v);
                        else if constexpr (ANY_ACT) { if (act != LUXHIP_ACT_IDENTITY) act_vec(act, v); }
                        uint2 ov;
                        ov.x = f32x2_to_bf16x2(v[0], v[1]);
                        ov.y = f32x2_to_bf16x2(v[2], v[3]);
                        *reinterpret_cast<uint2*>(a.out + (coloff + rowoff[i])) = ov;
                    }
                }
            }
        }
        if (extra) {            // the seventeenth fragment: positions m0 + 256 + 4 (l / 16) + r
            const int m = m0 + 256 + 4 * (int)laneq;
            if (m < m_end) {
                const int img = (int)a.divPQ.div((uint32_t)m);
                const uint32_t rowoffE = (uint32_t)(m - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img;
                const int ncol = n0 + (upper ? 64 : 0) + (int)lane15;
                const int act = a.act;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int col = ncol + 16 * j;
                    if (col < a.Ncols) {
                        const float b = bias_v[j];
                        const uint32_t off = (uint32_t)a.PQ * (uint32_t)(a.col_off + col) + rowoffE;
                        float v[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = accE[j][r] + b;
                        if (a.pre != nullptr) {
                            uint2 pv;
                            pv.x = f32x2_to_bf16x2(v[0], v[1]);
                            pv.y = f32x2_to_bf16x2(v[2], v[3]);
                            *reinterpret_cast<uint2*>(a.pre + off) = pv;
                        }
                        if (act == LUXHIP_ACT_RELU) act_vec_as<LUXHIP_ACT_RELU>(v);
                        else if constexpr (ANY_ACT) { if (act != LUXHIP_ACT_IDENTITY) act_vec(act, v); }
                        uint2 ov;
                        ov.x = f32x2_to_bf16x2(v[0], v[1]);
                        ov.y = f32x2_to_bf16x2(v[2], v[3]);
                        *reinterpret_cast<uint2*>(a.out + off) = ov;
                    }
                }
            }
        }
        if (tnext >= total) break;
        tile = tnext;
    }
#undef CP_READ_E
#undef CP_MFMA_E
#undef CP_READ_A
#undef CP_READ_B
#undef CP_READY
#undef CP_FENCE
    // the half-blocks requested past the last step are still on their way into the ring
    __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));
}
#endif  // LUXHIP_CONV_PATCH_KERNEL

struct Problem {
    const bf16_t *src, *wm, *bias;
    bf16_t *out, *pre;
    const void* zero;
    int Ctot, Cg, P, Q, N, kW, kH, pad_w, pad_h;   // pad: the padding of the forward convolution on the low side
    bool dgrad;
    int Ncols, col_off, Ctot_out, act;
};

// Unit stride and dilation with an output as large as the input are the caller's to check.
inline bool applicable(const Problem& p) {
    const auto al = [](const void* q, uintptr_t n) { return (reinterpret_cast<uintptr_t>(q) & (n - 1)) == 0; };
    const int T = p.kW * p.kH, pitch = p.P + p.kW - 1;
    const int64_t PQ = (int64_t)p.P * p.Q;
    if (p.kW != 3 || p.kH != 3 || p.Cg % 64 != 0 || p.Ctot % 8 != 0 || PQ % 4 != 0 || p.N < 1) return false;
    const int rows = (p.P - 1 + TILE_M_MAX - 1) / p.P + 1 + (p.kH - 1);      // image rows under a tile that starts at the end of a row, plus halo
    if ((int64_t)rows * pitch > PATCH_PIX) return false;
    if ((int64_t)(rows + 1) * p.P * p.Ctot * 2 >= (int64_t(1) << 31) || (int64_t)TILE_N * T * p.Cg * 2 >= (int64_t(1) << 31)) return false;
    return al(p.src, 16) && al(p.wm, 16) && al(p.out, 8) && al(p.pre, 8);
}

int launch(hipStream_t s, const Problem& p);    // conv_inst_patch_bf16.hip

}  // namespace cpatch
}  // namespace luxhip
