// bf16 filter gradient of a 3 x 3 convolution with unit stride and dilation and "same" output size, with the
// input window of a tile held in LDS.
//
//   dw[tap, ci, co] = sum over the output positions m of  x[position(m) + tap, ci] * dz[m, co]
//
// The gather-per-tap kernel loads, for every tile of 128 (tap, ci) rows, the shifted input again: nine
// times the input through L2, and about 25 address instructions per 16-byte load.  Here a workgroup takes one
// image, 64 input channels and 64 output channels and walks over the image in tiles of 256 positions; the
// rows of the image under a tile (plus the halo) are brought into LDS once, and all nine taps read them at
// shifted addresses.  The accumulators of a workgroup are the whole 9 x 64 x 64 block of dw for its
// channels (144 registers per lane).  Workgroup "lane" i of a part takes the images i, i + lanes, ... and writes one
// partial sum at the end; wgrad_reduce_kernel adds the lanes in order.  There are as many lanes as images while
// that keeps the workgroups within two per compute unit, otherwise fewer (a multiple of eight): the partial sums
// then stay a small multiple of the filter's size however large the batch is.
//
// Waves: wave w owns the 16 input channels 16 (w % 4) .. + 15 and every second 32-position step of the
// contraction (w / 4 selects which); the two waves of a channel block add their accumulators through LDS at
// the end.  Per step a wave reads nine A fragments (16 channels x 32 positions, one per tap, each two
// transposing reads ds_read_b64_tr_b16 from the channel-contiguous patch) and four B fragments (32 positions x
// 16 output channels from dz as it lies in memory: positions contiguous) for 36 MFMAs 16x16x32.
//
// LDS: two patch buffers (the next tile loads while this one is multiplied), each four planes (one per block of
// 16 channels) of 480 positions x 32 bytes: the 4 positions x 32 bytes that a 16-lane group reads are 128
// contiguous bytes; then a ring of eight dz blocks (64 output channels x 32 positions = 4 KiB per step; rows in
// groups of sixteen, chunk by chunk, as the patch of the forward kernel).  One barrier per four steps.
#pragma once

#include "common.h"
#include "gemm_core.h"

namespace luxhip {
namespace wpatch {

constexpr int THREADS = 512, TILE_PX = 256, STEP_PX = 32, SUPER = 4;     // positions per tile, per step; steps per barrier
constexpr int PATCH_PIX = 464, PLANE_POS = 480, PLANE_BYTES = PLANE_POS * 32, BUF_BYTES = 4 * PLANE_BYTES;   // 61440
constexpr int RING_OFF = 2 * BUF_BYTES, BLK_BYTES = 4096, RING = 8;     // 122880 + 32768
constexpr size_t LDS_BYTES = (size_t)RING_OFF + (size_t)RING * BLK_BYTES;   // 155648
constexpr int PATCH_INSTR = 8;                  // 60 blocks of 1 KiB (4 planes x 15 groups of 32 positions) on 8 waves
constexpr int TAPS = 9;
typedef float f32x4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_vp;
typedef const __attribute__((address_space(1))) void* glb_vp;

struct Args {
    const bf16_t* src;       // channel-contiguous x (C, P, Q, N), first channel of the group
    const bf16_t* dz;        // (P, Q, Cout, N), first output channel of the group
    float* partial;          // [lane][column][9 * Cg]
    const void* zero;        // 16 zero bytes in device memory
    int Ctot, Cg, Cout, Ncols;   // channels of x (all groups), of the group; output channels in all, of the group
    int P, Q, PQ, N, lanes;  // lanes: workgroups per part, each walks the images lane, lane + lanes, ...
    int pad_w, pad_h, pitch;     // pitch = P + 2
    int H, CB;                   // 64-channel parts of Cg, of Ncols
    FastDiv divP, divPitch;
};

#ifdef LUXHIP_CONV_WGRAD_PATCH_KERNEL
__device__ __forceinline__ uint32_t at_use(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

__global__ __launch_bounds__(THREADS) void conv_wgrad_patch_kernel(Args a) {
    extern __shared__ __align__(128) unsigned char lds_raw[];
    char* lds = reinterpret_cast<char*>(lds_raw);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds);   // LDS byte address
    const int tid = threadIdx.x, l = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wa = w & 3, ks = w >> 2;                 // channel block, which steps
    // The parts of an image (64 input x 64 output channels each) read the same input and the same dz: they go to one
    // XCD (workgroup i runs on XCD i % 8), next to each other in its order of dispatch, so that its L2 serves the repeats.
    const int parts = a.CB * a.H;
    const int slot = blockIdx.x >> 3;
    const int lane = (slot / parts) * 8 + (blockIdx.x & 7), part = slot % parts;
    if (lane >= a.N) return;                                // the last group of eight may be incomplete
    const int cb = part % a.CB, h = part / a.CB;
    const int steps = a.PQ / STEP_PX;                  // of the image
    const int tiles = (a.PQ + TILE_PX - 1) / TILE_PX;
    const int64_t row_bytes = (int64_t)a.P * a.Ctot * 2;

    // ---- patch loader: instruction i of this thread fills 1 KiB block b = 8 i + w (the last instruction: blocks
    // 56-59, two waves each, the same bytes): plane b / 15, positions 32 (b % 15) + l / 2, 16-byte half l % 2
    int32_t poff[PATCH_INSTR], prv[PATCH_INSTR];
#pragma unroll
    for (int i = 0; i < PATCH_INSTR; ++i) {
        const int b = i < PATCH_INSTR - 1 ? 8 * i + w : 56 + (w & 3);
        const int plane = b / 15, x = 32 * (b % 15) + (l >> 1);
        const int pr = (int)a.divPitch.div((uint32_t)x), pc = x - pr * a.pitch;
        const int ps = pc - a.pad_w;
        poff[i] = ((pr * a.P + ps) * a.Ctot + 16 * plane + 8 * (l & 1)) * 2;
        prv[i] = ((unsigned)ps < (unsigned)a.P && x < PATCH_PIX) ? pr : -(1 << 28);   // halo columns and the tail never pass the row test
    }
    const char* src_img = reinterpret_cast<const char*>(a.src) + ((int64_t)lane * a.Q * row_bytes) + h * 128;
    // patch of tile `ti` of the image into buffer `buf`: rows q_first - pad_h .. of the image
    auto patch_issue = [&](int i, int ti, int buf) {
        const int q0 = (int)a.divP.div((uint32_t)(ti * TILE_PX)) - a.pad_h;
        const bool valid = (unsigned)(q0 + prv[i]) < (unsigned)a.Q;
        const char* q = src_img + (int64_t)q0 * row_bytes + (int32_t)at_use((uint32_t)poff[i]);
        const void* p = valid ? static_cast<const void*>(q) : a.zero;
        const int b = i < PATCH_INSTR - 1 ? 8 * i + w : 56 + (w & 3);
        __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(lds + buf * BUF_BYTES + (b / 15) * PLANE_BYTES + (b % 15) * 1024), 16, 0, 0);
    };

    // ---- dz loader: per group of four steps a wave loads two 1 KiB blocks: rows 16 (w % 4) .. + 15 of the steps
    // w / 4 and 2 + w / 4 of the group; lane: row l % 16, 16-byte chunk (8 positions) l / 16
    const int zrow = 16 * (w & 3) + (l & 15);
    const bool zrow_ok = cb * 64 + zrow < a.Ncols;
    const char* dz_row = reinterpret_cast<const char*>(a.dz) +
                         (((int64_t)lane * a.Cout + cb * 64 + (zrow_ok ? zrow : 0)) * a.PQ + 8 * (l >> 4)) * 2;
    auto dz_issue = [&](int step) {              // step of the image (uniform); past the image: zeros
        const void* p = (step < steps && zrow_ok) ? static_cast<const void*>(dz_row + (int64_t)step * (STEP_PX * 2)) : a.zero;
        __builtin_amdgcn_global_load_lds((glb_vp)p, (lds_vp)(lds + RING_OFF + (step & (RING - 1)) * BLK_BYTES + (w & 3) * 1024), 16, 0, 0);
    };

    // ---- fragment reads
    const int g = l >> 4, s = l & 15;
    // A: this lane's address supplies 4 channels (8 bytes) of one position: channel quad s % 4, position 8 g + s / 4 of the step
    const uint32_t a_lane = (uint32_t)(wa * PLANE_BYTES + (s & 3) * 8);
    // B: row (output channel) 16 j + s of the block, chunk g
    const uint32_t b_lane = (uint32_t)(g * 256 + s * 16);

    f32x4_v acc[TAPS][4];
#pragma unroll
    for (int t = 0; t < TAPS; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][j][r] = 0.0f;

    for (int n = lane;;) {
    // prologue of an image: the first tile's patch, the dz blocks of the first four steps
#pragma unroll
    for (int i = 0; i < PATCH_INSTR; ++i) patch_issue(i, 0, 0);
    dz_issue(w >> 2);
    dz_issue(2 + (w >> 2));

    for (int ti = 0; ti < tiles; ++ti) {
        const int buf = ti & 1;
        const int q_first = (int)a.divP.div((uint32_t)(ti * TILE_PX));
        // this lane's patch byte offsets (first tap) of its positions in this wave's four steps of the tile:
        // step 2 u + ks, positions 8 g + s / 4 (first read) and + 4 (second read)
        uint32_t xb[4][2];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) {
                const int m = min(ti * TILE_PX + (2 * u + ks) * STEP_PX + 8 * g + (s >> 2) + 4 * hi, a.PQ - 1);
                const int q = (int)a.divP.div((uint32_t)m), p = m - q * a.P;
                xb[u][hi] = (uint32_t)(((q - q_first) * a.pitch + p) * 32) + a_lane;
            }
        const int tile_steps = min(TILE_PX / STEP_PX, steps - ti * (TILE_PX / STEP_PX));
        const int supers = (tile_steps + SUPER - 1) / SUPER;
        for (int S = 0; S < supers; ++S) {
            const int step0 = ti * (TILE_PX / STEP_PX) + S * SUPER;      // first step of the group, of the image
            // the dz blocks of this group have landed (requested a group ago), and at a tile's first group its patch;
            // loads of the next tile's patch requested since may stay in flight
            if (S == 0 || ti + 1 >= tiles) __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));
            else __builtin_amdgcn_s_waitcnt(4 | (0x7 << 4));             // vmcnt(4) lgkmcnt(0): the four patch loads are the youngest
            __builtin_amdgcn_s_barrier();
            // the next group's dz blocks, then half of the next tile's patch
            dz_issue(step0 + SUPER + (w >> 2));
            dz_issue(step0 + SUPER + 2 + (w >> 2));
            if (ti + 1 < tiles) {
                if (S == 0) {
                    patch_issue(0, ti + 1, buf ^ 1); patch_issue(1, ti + 1, buf ^ 1);
                    patch_issue(2, ti + 1, buf ^ 1); patch_issue(3, ti + 1, buf ^ 1);
                } else {
                    patch_issue(4, ti + 1, buf ^ 1); patch_issue(5, ti + 1, buf ^ 1);
                    patch_issue(6, ti + 1, buf ^ 1); patch_issue(7, ti + 1, buf ^ 1);
                }
            }
            const uint32_t patch = lds_addr + (uint32_t)buf * BUF_BYTES;
            const uint32_t row_step = (uint32_t)a.pitch * 32u;                // one tap row further down the patch
#pragma unroll
            for (int v = 0; v < 2; ++v) {                                // this wave's two steps of the group
                const int sl = 2 * v + ks;                               // step inside the group
                const int u = S * 2 + v;                                 // index of the step among this wave's four of the tile
                const uint32_t blk = lds_addr + RING_OFF + (uint32_t)((step0 + sl) & (RING - 1)) * BLK_BYTES + b_lane;
                const uint32_t x0 = patch + (u == 0 ? xb[0][0] : u == 1 ? xb[1][0] : u == 2 ? xb[2][0] : xb[3][0]);
                const uint32_t x1 = patch + (u == 0 ? xb[0][1] : u == 1 ? xb[1][1] : u == 2 ? xb[2][1] : xb[3][1]);
                // The reads are written as assembly: left to the compiler, the first of them would wait for every
                // global -> LDS load just requested (it must assume that they overwrite what is read; the ring and
                // the two patch buffers rule that out).  22 reads per step, in the order B0-B3, then per tap the
                // two halves of its A fragment; LDS reads return in order.
                u32x4_v fb[4];
                s16x4_v lo[TAPS], hi[TAPS];
                asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\tds_read_b128 %2, %4 offset:2048\n\t"
                             "ds_read_b128 %3, %4 offset:3072"
                             : "=&v"(fb[0]), "=&v"(fb[1]), "=&v"(fb[2]), "=&v"(fb[3]) : "v"(blk));
#pragma unroll
                for (int kb = 0; kb < 3; ++kb) {
                    const uint32_t r0 = x0 + (uint32_t)kb * row_step, r1 = x1 + (uint32_t)kb * row_step;
                    asm volatile("ds_read_b64_tr_b16 %0, %6\n\tds_read_b64_tr_b16 %1, %7\n\t"
                                 "ds_read_b64_tr_b16 %2, %6 offset:32\n\tds_read_b64_tr_b16 %3, %7 offset:32\n\t"
                                 "ds_read_b64_tr_b16 %4, %6 offset:64\n\tds_read_b64_tr_b16 %5, %7 offset:64"
                                 : "=&v"(lo[3 * kb]), "=&v"(hi[3 * kb]), "=&v"(lo[3 * kb + 1]), "=&v"(hi[3 * kb + 1]), "=&v"(lo[3 * kb + 2]),
                                   "=&v"(hi[3 * kb + 2])
                                 : "v"(r0), "v"(r1));
                }
                // tap t may start when at most 16 - 2 t of the reads behind its own are outstanding
#define WP_TAP(t, younger)                                                                                          \
                do {                                                                                                \
                    asm volatile("s_waitcnt lgkmcnt(" #younger ")"                                                  \
                                 : "+v"(lo[t]), "+v"(hi[t]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));   \
                    const s16x8_v both = {lo[t][0], lo[t][1], lo[t][2], lo[t][3], hi[t][0], hi[t][1], hi[t][2], hi[t][3]}; \
                    const bf16x8_v fa = __builtin_bit_cast(bf16x8_v, both);                                         \
                    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                   \
                        acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, __builtin_bit_cast(bf16x8_v, fb[j]), acc[t][j], 0, 0, 0); \
                } while (0)
                WP_TAP(0, 15); WP_TAP(1, 14); WP_TAP(2, 12); WP_TAP(3, 10); WP_TAP(4, 8);
                WP_TAP(5, 6); WP_TAP(6, 4); WP_TAP(7, 2); WP_TAP(8, 0);
#undef WP_TAP
            }
        }
    }

    // the next image of this lane: every wave has read the last fragments of this one before the buffers are refilled
    n += a.lanes;
    if (n >= a.N) break;
    src_img += (int64_t)a.lanes * a.Q * row_bytes;
    dz_row += (int64_t)a.lanes * a.Cout * a.PQ * 2;
    __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));
    __builtin_amdgcn_s_barrier();
    }

    // ---- the two waves of a channel block add their halves through LDS; the first stores
    __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4));
    __builtin_amdgcn_s_barrier();
    float* red = reinterpret_cast<float*>(lds) + (size_t)wa * (TAPS * 4 * 4 * 64);       // 36864 bytes per channel block
    if (ks == 1) {
#pragma unroll
        for (int t = 0; t < TAPS; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<f32x4_v*>(red + ((t * 4 + j) * 64 + l) * 4) = acc[t][j];
    }
    __syncthreads();
    if (ks == 0) {
        const int Mrows = TAPS * a.Cg;
        // acc[t][j][r]: input channel 64 h + 16 wa + 4 g + r, output channel 64 cb + 16 j + s
        float* out = a.partial + (size_t)lane * a.Ncols * Mrows + 64 * h + 16 * wa + 4 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = cb * 64 + 16 * j + s;
            if (col < a.Ncols) {
#pragma unroll
                for (int t = 0; t < TAPS; ++t) {
                    const f32x4_v o = *reinterpret_cast<const f32x4_v*>(red + ((t * 4 + j) * 64 + l) * 4);
                    f32x4_v v = acc[t][j];
                    v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
                    *reinterpret_cast<f32x4_v*>(out + (size_t)col * Mrows + t * a.Cg) = v;
                }
            }
        }
    }
}
#endif  // LUXHIP_CONV_WGRAD_PATCH_KERNEL

struct Problem {
    const bf16_t *src, *dz;
    float* partial;
    const void* zero;
    int Ctot, Cg, Cout, Ncols, P, Q, N, pad_w, pad_h;
};

// Workgroups per part (= partial sums that wgrad_reduce_kernel adds): one per image while the grid stays within two
// workgroups per compute unit, otherwise as many groups of eight as fit that bound (at least one).
inline int image_lanes(int N, int parts, int cus) {
    if ((int64_t)N * parts <= 2 * (int64_t)cus) return N;
    return std::min(N, std::max(8, (int)(2 * (int64_t)cus / parts) / 8 * 8));
}

// 3 x 3, unit stride and dilation, output as large as the input are the caller's to check.
inline bool applicable(const Problem& p, int cus) {
    const auto al = [](const void* q, uintptr_t n) { return (reinterpret_cast<uintptr_t>(q) & (n - 1)) == 0; };
    const int pitch = p.P + 2;
    const int64_t PQ = (int64_t)p.P * p.Q;
    if (p.Cg % 64 != 0 || p.Ctot % 8 != 0 || PQ % STEP_PX != 0 || p.N < 1) return false;
    const int rows = (p.P - 1 + TILE_PX - 1) / p.P + 1 + 2;               // image rows under a tile, plus halo
    if ((int64_t)rows * pitch > PATCH_PIX) return false;
    if ((int64_t)(rows + 1) * p.P * p.Ctot * 2 >= (int64_t(1) << 31)) return false;
    // enough workgroups to fill the device
    if ((int64_t)p.N * (p.Cg / 64) * ((p.Ncols + 63) / 64) < cus / 2) return false;
    return al(p.src, 16) && al(p.dz, 16) && al(p.partial, 16);
}

int launch(hipStream_t s, const Problem& p);    // conv_inst_wgrad_patch_bf16.hip

}  // namespace wpatch
}  // namespace luxhip
