// 1 x 1 convolution (any stride, no padding; NCHW data, OIHW weights) of a batch of images as a stream: the
// layers of the reference's conv2d generator (scripts/configure_kernels.py:28-38, :60-68) with KH = KW = 1,
// which have no halo and nothing to reuse between filter taps.  Per image
//
//   Y[co][p] = sum_ci Wt[co][ci] * X[ci][p],   p = 0 .. H*W-1    (stride S: X[ci][S*oy][S*ox], p = oy*OW + ox),
//
// a matrix product whose B operand, X, is read exactly once: the layers with few channels (64 -> 64 on
// 56 x 56, 192 .. 288 -> 32 .. 64 on 35 x 35) compute 8 - 16 flops per byte and are bound by that read and the
// write of Y.  The general convolution stages every 16-channel patch in LDS and sums its waves' partial tiles
// there; here the image goes from memory straight into the registers of the MFMA that consumes it.
//
// One wave owns 64 consecutive pixels of one image (a tile) and BM output channels; the NW waves of a
// workgroup own NW consecutive tiles of the batch-wide tile sequence (image after image) and share the filter
// rows co0 .. co0+BM-1, which the
// workgroup stages in LDS in chunks of up to 64 input channels, double-buffered, one barrier per chunk.
//
// Lane (j = lane % 16, q = lane / 16) loads, for step s = 0..3 of a 16-channel group g, the 16 bytes
// X[16g + 4q + s][p0 + 4j .. p0 + 4j + 3]: sixteen lanes read 256 consecutive bytes of a channel row, one load
// instruction covers four rows.  Element i of that vector is the B operand (k = q, n = j) of pixel block i,
// the pixels p0 + 4n + i: the four blocks of a tile interleave, so that a lane ends up with four CONSECUTIVE
// pixels of four output channels and stores them as 16 bytes.  The A operand of step s is element s of the
// 16 bytes Wt[co0 + 16tm + j][16g + 4q .. + 3], as the filter lies in memory.
//
// Rows of H*W floats that are not whole 16-byte chunks (35 x 35, 73 x 73, 17 x 17) are read and written with
// 16-byte accesses on 4-byte boundaries.  The last tile of an image whose pixels are not a multiple of 64
// starts 64 pixels before the image's end: it overlaps its neighbour, and both write the same bits to the
// pixels they share (a pixel column of the product depends on that column of X alone, and both waves sum its
// channels in the same order).  Only an image of fewer than 64 pixels has a ragged tile, which goes element by
// element, every read clamped to the row and every write tested against it.  (Measured against ragged last
// tiles on every image: 0.81-0.87 of the time on the 35 x 35 and 17 x 17 layers, whose slow ragged wave held
// its workgroup's barriers up; 1.02-1.05 on 73 x 73.)  With a
// stride the pixels of a tile are not consecutive in the image: every element is read on its own, from an
// offset worked out once per lane (the same for every channel); the outputs are consecutive as before.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_conv_general.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));   // 16 bytes on a 4-byte boundary

template <int CI_, int CO_, int H_, int W_, int S_, int BM_, int NW_, int NIMG_ = 1, bool OVERLAP_ = true>
struct Conv1x1F32 {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr int CI = CI_, CO = CO_, H = H_, W = W_, S = S_, BM = BM_, NW = NW_, NIMG = NIMG_;
    static constexpr int KH = 1, KW = 1, P = 0, OH = (H - 1) / S + 1, OW = (W - 1) / S + 1;
    static constexpr int HW = H * W, OHW = OH * OW;
    static constexpr int TM = BM / 16;
    static constexpr int NG = CI / 16;                                   // 16-channel groups
    static constexpr int GPC = NG % 4 == 0 ? 4 : (NG % 3 == 0 ? 3 : (NG % 2 == 0 ? 2 : 1));   // groups per staged chunk of the filter
    static constexpr int NC = NG / GPC;                                  // chunks
    static constexpr int KC = 16 * GPC;                                  // input channels per chunk
    static constexpr int TPI = (OHW + 63) / 64;                          // 64-pixel tiles per image
    static constexpr bool RAGGED = OHW % 64 != 0;
    static constexpr bool ALIGNED = OHW % 4 == 0;                        // every output row and tile starts on a 16-byte boundary
    static constexpr bool GATHER = S > 1;                                // a tile's pixels are not consecutive in the image
    // the last tile of an image of 64 pixels or more starts 64 pixels before the image's end instead of running
    // past it: it overlaps its neighbour, both compute the shared pixels from the same operands in the same
    // order and write the same bits, and no tile needs the element-by-element path
    static constexpr bool OVERLAP = OVERLAP_ && RAGGED && OHW >= 64;
    static constexpr long long NTILE = (long long)TPI * NIMG;
    static constexpr int NPT = (int)((NTILE + NW - 1) / NW);            // groups of NW tiles
    static constexpr int NCT = CO / BM;
    static_assert(CI % 16 == 0 && CO % BM == 0 && BM % 16 == 0 && NW >= 1 && NW <= 16 && S >= 1, "channel tiling");
    static_assert(NTILE * NCT < (1LL << 31), "grid size");

    static constexpr Dims3 GRID{NPT * NCT, 1, 1};
    static constexpr Dims3 BLOCK{64 * NW, 1, 1};
    static constexpr int THREADS = 64 * NW;
    static constexpr bool HAS_BARRIERS = NW > 1;
    static constexpr bool LOOP_BARRIERS = NW > 1;      // the first barrier stands before the main loop, one more per chunk
    static constexpr int MIN_BARRIERS = NC;

    // staged chunk of the filter: [channel quad of the chunk][output channel][4 channels], one 16-byte slot of
    // padding per quad
    static constexpr int ROW = BM + 1;
    static constexpr int BUF = GPC * 4 * ROW * 16;
    static constexpr int NUNIT = BM * GPC * 4;                           // 16-byte units of a chunk
    static constexpr int NU = (NUNIT + THREADS - 1) / THREADS;           // per thread

    struct Smem {
        __attribute__((aligned(16))) unsigned char w[(NC > 1 ? 2 : 1) * BUF];
    };

    // Workgroup id -> (group of tiles, output-channel tile): id % 8 is taken as the XCD, which owns consecutive
    // tile groups and every channel tile of each, so that the workgroups reading the same pixels use one L2.
    __device__ static __forceinline__ void tile_of(int vblock, int& pt, int& ct)
    {
        constexpr int PER_XCD = NPT / 8;
        constexpr int FULL = 8 * PER_XCD * NCT;
        if (vblock < FULL) {
            const int xcd = vblock & 7, slot = vblock >> 3;
            pt = xcd * PER_XCD + slot / NCT;
            ct = slot % NCT;
        } else {
            const int rem = vblock - FULL;
            pt = 8 * PER_XCD + rem / NCT;
            ct = rem % NCT;
        }
    }

    // this lane's four pixels of channel row `row` (which starts at pixel 0 of the image): 16 bytes from its
    // first pixel p, or element by element from the offsets `off`
    __device__ static __forceinline__ f32x4 load_x(const float* __restrict__ row, int p, const int (&off)[4], bool each)
    {
        if (GATHER || (RAGGED && each)) {
            f32x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = row[off[i]];
            return v;
        }
        if constexpr (ALIGNED) return *reinterpret_cast<const f32x4*>(row + p);
        else {
            const f32x4u v = *reinterpret_cast<const f32x4u*>(row + p);
            return f32x4{v[0], v[1], v[2], v[3]};
        }
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
        const int co0 = ct * BM;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int j = lane & 15, q = lane >> 4;
        const int t = pt * NW + wave;
        const bool active = t < NTILE;                // the last workgroup may have waves without a tile
        const int img = active ? t / TPI : 0;
        int p0 = active ? (t - img * TPI) * 64 : 0;
        if (OVERLAP && p0 + 64 > OHW) p0 = OHW - 64;
        const bool tail = RAGGED && !OVERLAP && p0 + 64 > OHW;    // the same for the whole wave
        const int p = p0 + 4 * j;
        int off[4];                                   // where this lane's pixels lie in a channel row (past the image: its last pixel)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pi = p + i < OHW ? p + i : OHW - 1;
            off[i] = S == 1 ? pi : (pi / OW) * S * W + (pi % OW) * S;
        }
        // channel 4q of group 0 of this wave's image; step s is s rows further on, group g 16g rows
        const float* const xq = X + ((size_t)img * CI + 4 * q) * HW;

        // filter chunk c -> registers -> LDS
        f32x4 wreg[NU];
        auto fetch_w = [&](int c) {
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int unit = u * THREADS + tid;
                if (NUNIT % THREADS == 0 || unit < NUNIT) {
                    const int r = unit / (KC / 4), kq = unit % (KC / 4);
                    wreg[u] = *reinterpret_cast<const f32x4*>(Wt + (size_t)(co0 + r) * CI + c * KC + 4 * kq);
                }
            }
        };
        auto put_w = [&](int buf) {
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int unit = u * THREADS + tid;
                if (NUNIT % THREADS == 0 || unit < NUNIT) {
                    const int r = unit / (KC / 4), kq = unit % (KC / 4);
                    *reinterpret_cast<f32x4*>(sm.w + buf * BUF + (kq * ROW + r) * 16) = wreg[u];
                }
            }
        };

        f32x4 acc[TM][4];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[tm][i] = f32x4{0.f, 0.f, 0.f, 0.f};

        f32x4 xc[4], xn[4];
        fetch_w(0);
        if (active) {
#pragma unroll
            for (int s = 0; s < 4; ++s) xc[s] = load_x(xq + (size_t)s * HW, p, off, tail);
        }
        put_w(0);
        if constexpr (NW > 1) sync();     // (one wave orders its own LDS accesses)

#pragma unroll 1
        for (int c = 0; c < NC; ++c) {
            if (c + 1 < NC) fetch_w(c + 1);
            const unsigned char* const wb = sm.w + (NC > 1 ? (c & 1) * BUF : 0) + (q * ROW + j) * 16;
#pragma unroll
            for (int gg = 0; gg < GPC; ++gg) {
                const int g = c * GPC + gg;
                if (active) {
                    if (g + 1 < NG) {
#pragma unroll
                        for (int s = 0; s < 4; ++s) xn[s] = load_x(xq + (size_t)(16 * (g + 1) + s) * HW, p, off, tail);
                    }
                    f32x4 a[TM];
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm) a[tm] = *reinterpret_cast<const f32x4*>(wb + (gg * 4 * ROW + 16 * tm) * 16);
#pragma unroll
                    for (int s = 0; s < 4; ++s)
#pragma unroll
                        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                acc[tm][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[tm][s], xc[s][i], acc[tm][i], 0, 0, 0);
                    if (g + 1 < NG) {
#pragma unroll
                        for (int s = 0; s < 4; ++s) xc[s] = xn[s];
                    }
                }
            }
            if (c + 1 < NC) {
                put_w((c + 1) & 1);
                if constexpr (NW > 1) sync();     // everyone is done with this chunk's buffer, and the next chunk is in place
            }
        }

        if (!active) return;
        // acc[tm][i][r]: output channel co0 + 16tm + 4q + r, pixel p + i
        float* const yq = Y + ((size_t)img * CO + co0 + 4 * q) * OHW + p;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float* const y = yq + (size_t)(16 * tm + r) * OHW;
                const f32x4 v{acc[tm][0][r], acc[tm][1][r], acc[tm][2][r], acc[tm][3][r]};
                if (RAGGED && tail) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (p + i < OHW) y[i] = v[i];
                } else if constexpr (ALIGNED) {
                    *reinterpret_cast<f32x4*>(y) = v;
                } else {
                    *reinterpret_cast<f32x4u*>(y) = f32x4u{v[0], v[1], v[2], v[3]};
                }
            }
    }
};

}  // namespace bfuse
