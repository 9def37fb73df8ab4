// 3x3 / stride 1 / pad 1 convolution (NCHW data, OIHW weights, batch 1) as an implicit GEMM on
// the matrix cores with the image patch staged in LDS.
//
// Replaces the TVM-generated `conv2d` kernels of the reference
// (scripts/configure_kernels.py:28-38,60-68; e.g.
// legacy/tests/single_bgemm_conv2d/case-0_4/M_diff/case-2/cuda/kernels.cu:72-111).
//
// Convolution as GEMM:  out[co][p] = sum_k  Wt[co][k] * Xcol[k][p],  p = y*W + x, with the
// reduction index ordered tap-major, k = (kh*3+kw)*CI + ci, so that four consecutive k are four
// input channels under ONE filter tap and no im2col buffer is ever written.  One workgroup owns BM
// output channels x PB*16 pixels; its KS waves split the reduction by input channel: wave w takes
// the 16-channel groups w, w+KS, ... and walks all nine taps of a group before moving on.  The
// partial tiles meet in LDS once and are summed in wave order.
//
// Fetching the B operand (image values under a filter tap) from global memory tap by tap costs 16
// scalar loads with a border test and 4 weight loads per 16 MFMAs.  Measured on MI355X, every
// vector-ALU instruction a wave issues between its MFMAs costs ~20 clocks of MFMA issue and a
// global load with its address arithmetic 30-40, so such a loop spends most of its time not
// multiplying (8.0-8.2 us on the ResNet shape).  Here a wave
// first copies the 16 channels x (rows the tile touches + 2) x (W + 2) patch it needs into a
// zero-padded LDS tile of its own -- once, before the loop, where issue slots are free -- in the
// layout [channel quad kq][position][4 channels].  In the loop the B operand of a tap is then ONE
// 128-bit LDS read per 16-pixel block, at a compile-time offset from a per-block base register
// (the padding removes the border test, the tap is an immediate), and the A operand -- the
// lane's 4 channels x 9 taps of one filter row, 36 consecutive floats -- sits in registers for
// the whole group.  Loop body per tap: PB reads, 4*TM*PB MFMAs, no vector ALU.
//
// The tile is private to the wave, so the K loop has no barrier.  Consecutive pixels of a block
// are consecutive 16-byte slots of a plane; the planes start one slot apart (see PLANE), which a
// 128-bit read pays for with a second pass (measured 8 clocks per wave-level read instead of 5.3:
// the hardware pairs lanes of two neighbouring quarter-waves in one pass, so only planes a
// multiple of 256 bytes apart read conflict-free).  The loop needs a quarter of the LDS read rate
// even so, whereas the staging stores, which the shift makes conflict-free, are on the critical path.
//
// Measured on the ResNet shape (64 -> 64 channels, 56 x 56, 196 workgroups; in-kernel clocks): filter
// rows 1.5 us and patch 1.4 us (overlapping), loop 2.2 us (the MFMA pipe rate), reduction and stores
// 0.85 us, ~1.5 us launch: 6.3-6.9 us.  The lane order of
// the staging matters as much as the loop: with the chunk index fastest the scattered 4-byte LDS
// stores were 16-way bank conflicts and the patch alone took 2.9 us.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int CI_, int CO_, int H_, int W_, int BM_, int PB_, int KS_>
struct Conv3x3F32Lds {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr int CI = CI_, CO = CO_, H = H_, W = W_, BM = BM_, PB = PB_, KS = KS_;
    static constexpr int HW = H * W;
    static constexpr int TM = BM / 16;
    static constexpr int NGROUP = CI / 16;           // 16-channel groups
    static constexpr int GPW = NGROUP / KS;          // groups per wave
    static constexpr int TP = 16 * PB;               // pixels per tile (consecutive in row-major order)
    static constexpr int NPT = HW / TP;
    static constexpr int SPAN = (TP + W - 2) / W + 1;   // image rows TP consecutive pixels can touch
    static constexpr int R = SPAN + 2, WP = W + 2;      // staged rows / columns, one of padding on each side
    static constexpr int NPOS = R * WP;
    // bytes of one channel quad, [position][4 channels], padded to 16 (mod 256): the four planes then
    // start one 16-byte slot apart in the banks, which is what makes the staging writes below conflict-free
    // (and the tap reads two-way conflicted: the cheaper side of the trade, see the header)
    static constexpr int PLANE = (NPOS * 16 + 255) / 256 * 256 + 16;
    static constexpr int TILE_BYTES = 4 * PLANE;
    static constexpr int CPR = W / 4;                   // 16-byte chunks per image row
    static constexpr int NCH = R * CPR;                 // 16-byte chunks per channel of the patch (contiguous in memory)
    static constexpr int NLD = (NCH + 3) / 4;           // wave-level loads per group: 16 channels x 4 consecutive chunks each
    static constexpr int NZ = (TILE_BYTES + 1023) / 1024;
    static_assert(CI % 16 == 0 && CO % BM == 0 && BM % 16 == 0, "channel tiling");
    static_assert(HW % TP == 0 && NGROUP % KS == 0 && W % 4 == 0, "pixel / reduction tiling");
    static_assert((2 * WP + 2) * 16 + 3 * PLANE < 65536, "tap offsets are 16-bit immediates");

    static constexpr Dims3 GRID{NPT * (CO / BM), 1, 1};
    static constexpr Dims3 BLOCK{64 * KS, 1, 1};
    static constexpr int THREADS = 64 * KS;
    static constexpr bool HAS_BARRIERS = KS > 1;
    static constexpr int PART_BYTES = KS > 1 ? KS * TM * PB * 1024 : 0;

    struct Smem {
        __attribute__((aligned(16))) unsigned char t[KS * TILE_BYTES > PART_BYTES ? KS * TILE_BYTES : PART_BYTES];
    };

    // Workgroup id -> (pixel tile, output-channel tile).  Consecutive ids go to consecutive XCDs, each
    // with an L2 of its own, so id % 8 is taken as the XCD and id / 8 walks (pixel tile, channel tile)
    // within it: the CO / BM workgroups that share a pixel tile -- and with it an image patch -- run on
    // one XCD, and an XCD owns CONSECUTIVE pixel tiles, whose patches overlap in image rows.  Each L2
    // then fetches its eighth of the image (plus halo rows) once; with ids simply running over the
    // pixel tiles of one channel tile after the other, every L2 fetches most of the image.
    static constexpr int NCT = CO / BM;
    __device__ static __forceinline__ void tile_of(int vblock, int& pt, int& ct)
    {
        constexpr int PER_XCD = NPT / 8;                 // whole pixel tiles every XCD owns
        constexpr int FULL = 8 * PER_XCD * NCT;          // ids covered by them
        if (vblock < FULL) {
            const int xcd = vblock & 7, slot = vblock >> 3;
            pt = xcd * PER_XCD + slot / NCT;
            ct = slot % NCT;
        } else {                                         // the NPT % 8 pixel tiles left over
            const int rem = vblock - FULL;
            pt = 8 * PER_XCD + rem / NCT;
            ct = rem % NCT;
        }
    }

    // accumulator layout: lane (j = pixel, rg) owns output channels 4*rg+v of the block
    __device__ static __forceinline__ void store_block(float* __restrict__ Y, int co0, int p0, int tm, int pb,
                                                       const f32x4& blk, int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
#pragma unroll
        for (int v = 0; v < 4; ++v)
            Y[(size_t)(co0 + tm * 16 + 4 * rg + v) * HW + p0 + pb * 16 + j] = blk[v];
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        const float* __restrict__ X = static_cast<const float*>(I);
        const float* __restrict__ Wt = static_cast<const float*>(F);
        float* __restrict__ Y = static_cast<float*>(O);
        int pt, ct;
        tile_of(vblock, pt, ct);
        const int p0 = pt * TP, co0 = ct * BM;
        const int y_lo = p0 / W;                       // first image row of the tile; staged row 0 is y_lo - 1
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        const int li = lane & 15, kq = lane >> 4;
        unsigned char* const tile = sm.t + wave * TILE_BYTES;

        // padding (and rows outside the image) read as zero: 0 * w adds exactly 0, as a border
        // test would
#pragma unroll
        for (int z = 0; z < NZ; ++z) {
            const int off = z * 1024 + lane * 16;
            if (off < TILE_BYTES) *reinterpret_cast<f32x4*>(tile + off) = f32x4{0.f, 0.f, 0.f, 0.f};
        }

        // this lane's pixel of each block: the top-left tap of its window, plane kq
        const unsigned char* bbase[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            const int p = p0 + pb * 16 + li;
            bbase[pb] = tile + kq * PLANE + ((p / W - y_lo) * WP + p % W) * 16;
        }

        f32x4 acc[TM][PB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) acc[tm][pb] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 1
        for (int gi = 0; gi < GPW; ++gi) {
            const int ci0 = (wave + gi * KS) * 16;
            // A operand: Wt[co][ci0 + 4 kq + t][tap], t = 0..3, tap = 0..8 -- 36 consecutive floats
            f32x4 aw[TM][9];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const f32x4* src = reinterpret_cast<const f32x4*>(Wt + ((size_t)(co0 + tm * 16 + li) * CI + ci0 + 4 * kq) * 9);
#pragma unroll
                for (int j = 0; j < 9; ++j) aw[tm][j] = src[j];
            }
            // stage the patch: lane = 4 * channel + (chunk % 4), i.e. a wave-level load takes four
            // consecutive 16-byte chunks (64 bytes) of each of the 16 channels.  The four values of a chunk
            // go to four consecutive positions of the channel's plane; with this lane order the 64 lanes of
            // each of those stores fall in 64 different banks (channel % 4 -> word, channel / 4 -> plane,
            // one slot apart, chunk % 4 -> 64 bytes apart)
            const int cl = lane >> 2, c4 = lane & 3;
            f32x4 v[NLD];
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int cc = j * 4 + c4;                 // chunk within the channel's R x W patch
                const int r = cc / CPR, c = cc % CPR;
                const int yy = y_lo - 1 + r;
                const bool ok = cc < NCH && yy >= 0 && yy < H;
                v[j] = ok ? *reinterpret_cast<const f32x4*>(X + (size_t)(ci0 + cl) * HW + yy * W + 4 * c) : f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int cc = j * 4 + c4;
                const int r = cc / CPR, c = cc % CPR;
                const int yy = y_lo - 1 + r;
                if (cc < NCH && yy >= 0 && yy < H) {
                    float* dst = reinterpret_cast<float*>(tile + (cl / 4) * PLANE + (r * WP + 1 + 4 * c) * 16) + cl % 4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[4 * e] = v[j][e];
                }
            }

            // nine taps: read the next tap's operands while this one multiplies
            f32x4 b[2][PB];
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) b[0][pb] = *reinterpret_cast<const f32x4*>(bbase[pb]);
#pragma unroll
            for (int tap = 0; tap < 9; ++tap) {
                if (tap + 1 < 9) {
                    const int noff = (((tap + 1) / 3) * WP + (tap + 1) % 3) * 16;
#pragma unroll
                    for (int pb = 0; pb < PB; ++pb) b[(tap + 1) & 1][pb] = *reinterpret_cast<const f32x4*>(bbase[pb] + noff);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                        for (int pb = 0; pb < PB; ++pb)
                            acc[tm][pb] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[tm][(t * 9 + tap) / 4][(t * 9 + tap) % 4],
                                                                               b[tap & 1][pb][t], acc[tm][pb], 0, 0, 0);
            }
        }

        if constexpr (KS == 1) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) store_block(Y, co0, p0, tm, pb, acc[tm][pb], lane);
        } else {
            f32x4(*part)[TM * PB][64] = reinterpret_cast<f32x4(*)[TM * PB][64]>(sm.t);
            sync();  // the partial tiles overwrite the patches: every wave is done reading its own
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) part[wave][tm * PB + pb][lane] = acc[tm][pb];
            sync();
            // block u is finished by wave u mod KS, summing the partials of waves 0..KS-1 in order
#pragma unroll
            for (int u0 = 0; u0 < TM * PB; u0 += KS) {
                const int u = u0 + wave;
                if (u < TM * PB) {
                    f32x4 s = part[0][u][lane];
#pragma unroll
                    for (int w = 1; w < KS; ++w) s += part[w][u][lane];
                    store_block(Y, co0, p0, u / PB, u % PB, s, lane);
                }
            }
        }
    }
};

}  // namespace bfuse
