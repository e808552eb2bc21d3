// The 3 x 3 window convolution of conv_patch.h in tiles of 64 output channels: the same patch buffers, patch layout,
// work split into fragments of 16 output positions and ring of filter half-blocks, but the eight waves of a
// workgroup share the 64 columns and split the tile's positions: wave w owns the fragments 2 w and 2 w + 1 (wave tile
// 32 positions x 64 channels, 16 MFMAs 16x16x32 per step), the seventeenth fragment of a tile is multiplied
// by the waves 0-3 (one per SIMD), each for 16 of the 64 columns.  A step (one tap of 64 channels) consumes one
// filter half-block (64 output channels x 64 k); the loads run four half-blocks ahead.  With the kernel for 128
// columns, half of the waves of such a problem would multiply columns that are never stored.
#pragma once

#include "conv_patch.h"

namespace luxhip {
namespace cpatch {

// The kernel is compiled by the one source file that defines LUXHIP_CONV_PATCH_KERNEL.
#ifdef LUXHIP_CONV_PATCH_KERNEL
// ANY_ACT false: identity or relu only.  The epilogue is unrolled over the accumulator tiles, and with every activation
// inlined into each copy the kernel grows to several times the instruction cache, which the workgroup then refills
// from L2 after every tile.
template <bool ANY_ACT>
__global__ __launch_bounds__(THREADS) void conv_patch_narrow_kernel(Args a) {
    extern __shared__ __align__(128) unsigned char lds_raw[];
    char* lds = reinterpret_cast<char*>(lds_raw);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds);   // LDS byte address
    const int tid = threadIdx.x, l = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = w * 32;
    // this workgroup's fragments [frag0, frag0 + nfrag) and its tiles
    const int bm = blockIdx.x % a.groups_m, tn = blockIdx.x / a.groups_m;   // tn: which 64 output channels
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
    const int brow0 = min(tid >> 3, a.Ncols - 1 - tn * 64);
    const uint32_t boff0 = (uint32_t)(brow0 * K2) + (uint32_t)(((tid & 7) ^ (((tid >> 3) >> 1) & 7)) << 4);
    int ring_b = 0;
    // the half-block of the step whose columns start at gp
    auto filter_issue = [&](const char* gp) {
        __builtin_amdgcn_global_load_lds((glb_vp)(gp + at_use(boff0)), (lds_vp)(lds + RING_OFF + ring_b * HB_BYTES + w * 1024), 16, 0, 0);
        ring_b = ring_b + 1 == RING ? 0 : ring_b + 1;
    };
    // filter bytes of this workgroup's columns, first channel, tap 0
    const char* const gp_first = reinterpret_cast<const char*>(a.wm) + (int64_t)tn * 64 * K2;

    // ---- fragment reads
    const uint32_t lane15 = l & 15, laneq = l >> 4;
    // B: row 16 j + l % 16 of the step's half-block, chunk 4 g + l / 16 for k group g (g = 1: XOR 64)
    const uint32_t offB = (uint32_t)(lane15 * 128 + ((laneq ^ ((lane15 >> 1) & 7)) << 4));

    // the bias of this lane's columns (16 j + l % 16, and 16 w + l % 16 for the seventeenth fragment), read once: a
    // load inside the epilogue would have to wait for the stores issued before it
    float bias_v[4], bias_e;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = tn * 64 + 16 * j + (int)lane15;
        bias_v[j] = a.bias != nullptr && col < a.Ncols ? ld(a.bias + a.col_off + col) : 0.0f;
    }
    {
        const int col = tn * 64 + 16 * (w & 3) + (int)lane15;
        bias_e = a.bias != nullptr && col < a.Ncols ? ld(a.bias + a.col_off + col) : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(bias_v[j]));       // the wait for these loads belongs here, before the tile loop
    asm volatile("" : "+v"(bias_e));
    int tile = 0;
    int hc = 0;                              // halves consumed so far by this workgroup: patch buffer hc & 1
    const char* gp_cur = gp_first;
    // prologue: the first patch and the half-blocks of the first four steps
    {
        int rbase;
        const char* pb = patch_base(tile, 0, rbase);
#pragma unroll
        for (int i = 0; i < PATCH_INSTR; ++i) patch_issue(i, pb, rbase, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) filter_issue(gp_cur + i * Cg2);
    }
    // the waves (one per SIMD) that share the seventeenth fragment of a tile: wave w takes the columns 16 w .. 16 w + 15
    const bool extra_wave = w < 4;
    const uint32_t offE = (uint32_t)w * 2048u;
    int slot = 0;                            // ring slot of the current step's half-block

    f32x4_v acc[2][4], accE;
    bf16x8_v fa[2][2], fb[2][4], faE[2], fbE[2];
    for (;;) {
        const int m0 = tile_first(tile);
        const int m_end = min(a.M, m0 + 16 * tile_frags(tile));
        const bool extra = extra_wave && tile_frags(tile) > 16;
        const int r_first = (int)a.divP.div((uint32_t)m0);
        const int tnext = tile + 1;
        const int total = ntile;
#pragma unroll
        for (int r = 0; r < 4; ++r) accE[r] = 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
        // this lane's patch positions: fragment f (output position m0 + wave_m + 16 f + l % 16; f = 2: the seventeenth
        // of the tile) under tap row jb, first tap column; 464 (the zeros) where that row lies outside the image
        uint32_t xrow[3][3];
#pragma unroll
        for (int f = 0; f < 3; ++f) {
            const int m = m0 + (f < 2 ? wave_m + 16 * f : 256) + (int)lane15;
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
#define CPN_READ_A(set, a0, a1, OFF)                                                                                \
        asm volatile("ds_read_b128 %0, %2 offset:" #OFF "\n\tds_read_b128 %1, %3 offset:" #OFF                      \
                     : "=&v"(fa[set][0]), "=&v"(fa[set][1]) : "v"(a0), "v"(a1))
#define CPN_READ_B(set, ab)                                                                                         \
        asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:2048\n\tds_read_b128 %2, %4 offset:4096\n\t" \
                     "ds_read_b128 %3, %4 offset:6144"                                                              \
                     : "=&v"(fb[set][0]), "=&v"(fb[set][1]), "=&v"(fb[set][2]), "=&v"(fb[set][3]) : "v"(ab))
        // the six reads of `set` have returned when at most `younger` LDS reads issued after them are outstanding
#define CPN_READY(set, younger)                                                                                     \
        asm volatile("s_waitcnt lgkmcnt(" #younger ")"                                                              \
                     : "+v"(fa[set][0]), "+v"(fa[set][1]), "+v"(fb[set][0]), "+v"(fb[set][1]), "+v"(fb[set][2]),   \
                       "+v"(fb[set][3]))
#define CPN_FENCE() __builtin_amdgcn_sched_barrier(0)
        // the seventeenth fragment: two more reads behind the six of a set (so the waits above cover them), one more MFMA
#define CPN_READ_E(set, ae, OFF, be)                                                                                \
        asm volatile("ds_read_b128 %0, %2 offset:" #OFF "\n\tds_read_b128 %1, %3" : "=&v"(faE[set]), "=&v"(fbE[set]) : "v"(ae), "v"(be))
#define CPN_MFMA_E(set)                                                                                              \
        do {                                                                                                        \
            asm volatile("" : "+v"(faE[set]), "+v"(fbE[set]));                                                      \
            accE = __builtin_amdgcn_mfma_f32_16x16x32_bf16(faE[set], fbE[set], accE, 0, 0, 0);                      \
        } while (0)
        auto mfmas = [&](int set) {              // the wave tile under one k group: eight MFMAs
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
        };

        // the first patch and the half-block of the first step have landed: of the loads issued so far at most the
        // three youngest (half-blocks further ahead) are outstanding.  Later tiles start behind the boundary of the
        // step before, which has covered their patch and first half-block; their barrier keeps the next patch loads
        // out of the buffer in which slower waves still turn their results around.
        if (tile == 0) __builtin_amdgcn_s_waitcnt(3 | (0x7 << 4));      // vmcnt(3) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0xF | (0x7 << 4) | (0x3 << 14));   // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();

        uint32_t aA[3], aN[3];
        {
            const uint32_t bufbase = lds_addr + (uint32_t)(hc & 1) * BUF_STRIDE;
#pragma unroll
            for (int f = 0; f < 3; ++f) aA[f] = a_addr(f, 0, bufbase);
        }
        {
            const uint32_t sb = lds_addr + RING_OFF + (uint32_t)slot * HB_BYTES + at_use(offB);
            CPN_READ_A(0, aA[0], aA[1], 0);
            CPN_READ_B(0, sb);
            if (extra) CPN_READ_E(0, aA[2], 0, sb + offE);
        }

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
                {
                    const uint32_t sb = lds_addr + RING_OFF + (uint32_t)slot * HB_BYTES + (at_use(offB) ^ 64u);
                    CPN_READ_A(1, aA[0], aA[1], 1024);
                    CPN_READ_B(1, sb);
                    if (extra) CPN_READ_E(1, aA[2], 1024, sb + offE);
                }
                // the half-block of the step four ahead goes where the step before this one read
                filter_issue(t + 4 < TAPS ? gp_cur + (t + 4) * Cg2 : gp_next + (t + 4 - TAPS) * Cg2);
                // the next half's patch is requested in the first two steps, behind the step's half-block: the waits
                // of the steps 0-3 then leave it in flight, and it has four steps' time before a wait covers it
                if constexpr (t < 2) {
                    if (have_p) {
#pragma unroll
                        for (int i = 0; i < PATCH_INSTR / 2; ++i) patch_issue(t * (PATCH_INSTR / 2) + i, pb_p, rbase_p, (hc + 1) & 1);
                    }
                }
                CPN_READY(0, 6);
                CPN_FENCE(); mfmas(0); CPN_FENCE();
                {
                    const uint32_t nb = t + 1 < TAPS ? buf_cur : buf_next;
#pragma unroll
                    for (int f = 0; f < 3; ++f) aN[f] = a_addr(f, (t + 1) % TAPS, nb);
                }
                if (extra) CPN_MFMA_E(0);
                CPN_FENCE();
                CPN_READY(1, 0);
                // boundary: every wave's reads of this step have returned, and the half-block of the next step
                // (requested three steps ago, first in its step) has landed.  Loads return in order; younger than
                // that half-block are those of the three steps since and, while a next half exists, the patch
                // blocks requested behind the half-blocks of the steps 0 and 1, four each.  Stores of the tile before
                // that sit in between only make the wait cover more.  After the last tap the half-block of the next
                // half's first step and the whole next patch are older than the three that may stay in flight.
                {
                    constexpr int with_patch = t == 0 || t == 4 ? 7 : t >= 1 && t <= 3 ? 11 : 3;
                    if (have_p) __builtin_amdgcn_s_waitcnt(with_patch | (0x7 << 4));
                    else __builtin_amdgcn_s_waitcnt(3 | (0x7 << 4));
                }
                __builtin_amdgcn_s_barrier();
                slot = slot + 1 == RING ? 0 : slot + 1;
                {
                    const uint32_t sb = lds_addr + RING_OFF + (uint32_t)slot * HB_BYTES + at_use(offB);
                    CPN_READ_A(0, aN[0], aN[1], 0);
                    CPN_READ_B(0, sb);
                    if (extra) CPN_READ_E(0, aN[2], 0, sb + offE);
                }
                CPN_FENCE(); mfmas(1); CPN_FENCE();
                if (extra) CPN_MFMA_E(1);
                CPN_FENCE();
#pragma unroll
                for (int f = 0; f < 3; ++f) aA[f] = aN[f];
            });
            ++hc;
            gp_cur = gp_next;
        }

        // ---- epilogue: lane l owns positions m0 + wave_m + 16 i + 4 (l / 16) + r and channel 16 j + l % 16
        if (a.staged) {
            // Through LDS, sixteen channels at a time, so that a store instruction writes 64 contiguous bytes per channel
            // (the wave's 32 positions) instead of sixteen pieces of 32 bytes: the wave's 1280 bytes lie in the patch
            // buffer of the half just finished, which nobody reads after that half's last boundary and which the
            // loads of the half after the next only enter behind the next tile's first barrier.  Rows of 80 bytes
            // keep the writes (lane l: channel l % 16) and the reads (lane l: channel l / 4, positions 8 (l % 4) .. + 7)
            // free of bank conflicts.
            char* st = lds + ((hc - 1) & 1) * BUF_STRIDE + w * 1280;
            const int mq = m0 + wave_m + 8 * (l & 3);
            const bool qok = mq < m_end;                                // m_end and PQ are multiples of 8 here
            const int img = (int)a.divPQ.div((uint32_t)(qok ? mq : 0));
            const uint32_t rowoffq = (uint32_t)(mq - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img;
            const int act = a.act;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = bias_v[j];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = acc[i][j][r] + b;
                    if (act == LUXHIP_ACT_RELU) act_vec_as<LUXHIP_ACT_RELU>(v);
                    else if constexpr (ANY_ACT) { if (act != LUXHIP_ACT_IDENTITY) act_vec(act, v); }
                    uint2 ov;
                    ov.x = f32x2_to_bf16x2(v[0], v[1]);
                    ov.y = f32x2_to_bf16x2(v[2], v[3]);
                    *reinterpret_cast<uint2*>(st + lane15 * 80 + (16 * i + 4 * laneq) * 2) = ov;
                }
                const int c = l >> 2;
                const uint4 val = *reinterpret_cast<const uint4*>(st + c * 80 + (l & 3) * 16);
                const int col = tn * 64 + 16 * j + c;
                if (qok && col < a.Ncols) *reinterpret_cast<uint4*>(a.out + ((uint32_t)a.PQ * (uint32_t)(a.col_off + col) + rowoffq)) = val;
            }
        } else {
            const int mrow = m0 + wave_m + 4 * (int)laneq;
            // element offsets inside one image's block of the output fit 32 bits (the tensor has fewer than 2^31 elements)
            uint32_t rowoff[2];
            bool mok[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int m = mrow + 16 * i;
                mok[i] = m < m_end;                                    // m_end and PQ are multiples of 4: all four or none
                const int img = (int)a.divPQ.div((uint32_t)(mok[i] ? m : 0));
                rowoff[i] = (uint32_t)(m - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img;
            }
            const int act = a.act;
            const bool has_pre = a.pre != nullptr;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = tn * 64 + (int)lane15 + 16 * j;
                if (col < a.Ncols) {
                    const float b = bias_v[j];
                    const uint32_t coloff = (uint32_t)a.PQ * (uint32_t)(a.col_off + col);
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
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
        if (extra) {            // the seventeenth fragment: positions m0 + 256 + 4 (l / 16) + r, channel 16 w + l % 16
            const int m = m0 + 256 + 4 * (int)laneq;
            const int col = tn * 64 + 16 * w + (int)lane15;
            if (m < m_end && col < a.Ncols) {
                const int img = (int)a.divPQ.div((uint32_t)m);
                const uint32_t off = (uint32_t)(m - img * a.PQ) + (uint32_t)a.PQ * (uint32_t)a.Ctot_out * (uint32_t)img +
                                     (uint32_t)a.PQ * (uint32_t)(a.col_off + col);
                const float b = bias_e;
                const int act = a.act;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = accE[r] + b;
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
        if (tnext >= total) break;
        tile = tnext;
    }
#undef CPN_READ_E
#undef CPN_MFMA_E
#undef CPN_READ_A
#undef CPN_READ_B
#undef CPN_READY
#undef CPN_FENCE
    // the half-blocks requested past the last step are still on their way into the ring
    __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));
}
#endif  // LUXHIP_CONV_PATCH_KERNEL

}  // namespace cpatch
}  // namespace luxhip
