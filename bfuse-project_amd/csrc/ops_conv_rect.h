// Convolution on rectangular pixel tiles: the implicit GEMM of ConvF32Lds (ops_conv_general.h: any filter size,
// stride, padding, image size and batch; channel groups of 16 -- or 4 -- under one filter tap; KS waves over the
// channel groups, each with a zero-padded LDS patch of its own; partial tiles summed in wave order) with the
// workgroup's pixels arranged as TH output rows x 16 output columns instead of 64 consecutive pixels.
//
// What that changes is the patch.  64 consecutive pixels of a wide image are part of one row, but the rows a
// wave stages are whole image rows: on a 147-wide image 4 x 149 positions for 64 outputs, of which 3 x 66 are
// read.  A TH x 16 tile needs ((TH-1) S + KH) x (15 S + KW) positions -- 6 x 18 for a 3 x 3 filter, 5.5 times
// fewer -- so the staging (global loads, scattered LDS writes) shrinks by that factor and so does the LDS a
// workgroup holds, which lets more workgroups share a CU.  The MFMA loop is ConvF32Lds's: per lane a base
// address in the patch plus a compile-time offset per tap.
//
// A patch row is a piece of an image row that starts anywhere, so it is fetched with ALIGNED 16-byte loads from
// the boundary below its start; each float of a vector knows its own column, and those outside the patch or
// the image are dropped (they stay zero in the tile, which is what padding reads as).  Output columns past
// the image (OW not a multiple of 16) and rows past it (OH not a multiple of TH) are computed on whatever the
// patch holds there and not stored.
//
// Replaces the same TVM-generated `conv2d` kernels of the reference as ConvF32Lds
// (scripts/configure_kernels.py:28-38,60-68); which of the two a shape gets is ConvTiling's choice.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "dispatch.h"
#include "ops_conv_1x1.h"
#include "ops_conv_general.h"
#include "wave.h"

namespace bfuse {

template <int CI_, int CO_, int H_, int W_, int KH_, int KW_, int S_, int P_, int BM_, int TH_, int KS_, int NIMG_ = 1>
struct ConvF32Rect {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr int CI = CI_, CO = CO_, H = H_, W = W_, KH = KH_, KW = KW_, S = S_, P = P_, BM = BM_, TH = TH_, KS = KS_, NIMG = NIMG_;
    static constexpr int OH = (H - KH + 2 * P) / S + 1, OW = (W - KW + 2 * P) / S + 1;
    static constexpr int HW = H * W, OHW = OH * OW, T = KH * KW;
    static constexpr int CG = CI >= 16 ? 16 : 4;        // channels per group
    static constexpr int NQ = CG / 4;                   // channel quads = planes of the tile = MFMAs per tap
    static constexpr int NGROUP = CG == 16 ? CI / 16 : 1;
    static constexpr int GPW = NGROUP / KS;             // groups per wave
    static constexpr int TM = BM / 16;
    static constexpr int PB = TH;                       // 16-pixel blocks of the tile: one per output row
    static constexpr int NTX = (OW + 15) / 16, NTY = (OH + TH - 1) / TH, NPT = NTX * NTY;
    static constexpr int PR = (TH - 1) * S + KH, PC = 15 * S + KW;   // patch rows / columns
    static constexpr int NPOS = PR * PC;
    // bytes of one channel quad, [position][4 channels], padded to 16 (mod 256): the planes then start one
    // 16-byte slot apart in the banks (see ops_conv.h)
    static constexpr int PLANE = (NPOS * 16 + 255) / 256 * 256 + 16;
    static constexpr int TILE_BYTES = NQ * PLANE;
    static constexpr int LPC = 64 / CG;                 // lanes that share a channel while staging
    static constexpr int NVR = (PC + 3) / 4 + 1;        // aligned 16-byte vectors that can overlap one patch row
    static constexpr int NU = PR * NVR;                 // staging units (row, vector) per channel
    static constexpr int NLD = (NU + LPC - 1) / LPC;    // wave-level loads per group
    static constexpr int NZ = (TILE_BYTES + 1023) / 1024;
    static_assert(CG == 16 ? CI % 16 == 0 : CI <= 4, "input channels: a multiple of 16, or at most 4");
    static_assert(CO % BM == 0 && BM % 16 == 0 && NGROUP % KS == 0, "channel tiling");
    static_assert(((KH - 1) * PC + KW - 1) * 16 + (NQ - 1) * PLANE + 16 < 65536, "tap offsets are 16-bit immediates");
    static_assert(S >= 1 && OH >= 1 && OW >= 1 && TH >= 1, "shape");

    static constexpr int NCT = CO / BM;
    static constexpr int WG_PER_IMAGE = NPT * NCT;
    static_assert(NIMG >= 1 && (long long)WG_PER_IMAGE * NIMG < (1LL << 31), "grid size");
    static constexpr Dims3 GRID{WG_PER_IMAGE * NIMG, 1, 1};
    static constexpr Dims3 BLOCK{64 * KS, 1, 1};
    static constexpr int THREADS = 64 * KS;
    static constexpr bool HAS_BARRIERS = KS > 1;
    static constexpr int PART_BYTES = KS > 1 ? KS * TM * PB * 1024 : 0;

    struct Smem {
        __attribute__((aligned(16))) unsigned char t[KS * TILE_BYTES > PART_BYTES ? KS * TILE_BYTES : PART_BYTES];
    };

    // Workgroup id -> (pixel tile, output-channel tile): id % 8 is taken as the XCD, which owns consecutive
    // pixel tiles and every channel tile of each, so that the workgroups sharing a patch use one L2.
    __device__ static __forceinline__ void tile_of(int vblock, int& pt, int& ct)
    {
        // over the pixel tiles of the WHOLE batch (image-major): with few tiles per image (an 8 x 8 image is one)
        // the channel tiles of one image would otherwise be consecutive ids, one per XCD, and each XCD would
        // fetch the image for itself (measured on the 1 x 1 layers of 8 x 8 images: 7.8 times the operands)
        constexpr int NPTB = NPT * NIMG;
        constexpr int PER_XCD = NPTB / 8;
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

    // accumulator layout: lane (j = column of the tile row, rg) owns output channels 4*rg+v of the block
    __device__ static __forceinline__ void store_block(float* __restrict__ Y, int co0, int oy, int ox0, int tm,
                                                       const f32x4& blk, int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
        const int ox = ox0 + j;
        if (oy < OH && ox < OW) {
#pragma unroll
            for (int v = 0; v < 4; ++v) Y[(size_t)(co0 + tm * 16 + 4 * rg + v) * OHW + oy * OW + ox] = blk[v];
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
        if constexpr (NIMG > 1) {
            const int img = pt / NPT;
            pt -= img * NPT;
            X += (size_t)img * CI * HW;
            Y += (size_t)img * CO * OHW;
        }
        const int co0 = ct * BM;
        const int oy0 = (pt / NTX) * TH, ox0 = (pt % NTX) * 16;   // first output row / column of the tile
        const int iy0 = oy0 * S - P, ix0 = ox0 * S - P;           // image row / column of patch position (0, 0)
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int li = lane & 15, kq = lane >> 4;
        unsigned char* const tile = sm.t + wave * TILE_BYTES;

#pragma unroll
        for (int z = 0; z < NZ; ++z) {
            const int off = z * 1024 + lane * 16;
            if (off < TILE_BYTES) *reinterpret_cast<f32x4*>(tile + off) = f32x4{0.f, 0.f, 0.f, 0.f};
        }

        // this lane's pixel of each block: the top-left tap of its window; channel quad kq (CG = 16) or
        // channel kq of the only quad (CG = 4)
        const unsigned char* bbase[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) bbase[pb] = tile + ((pb * S) * PC + li * S) * 16 + (CG == 16 ? kq * PLANE : kq * 4);

        f32x4 acc[TM][PB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) acc[tm][pb] = f32x4{0.f, 0.f, 0.f, 0.f};

        // columns of the patch that lie inside the image
        const int c_lo = ix0 < 0 ? -ix0 : 0;
        const int c_hi = W - ix0 < PC ? W - ix0 : PC;

#pragma unroll 1
        for (int gi = 0; gi < GPW; ++gi) {
            const int ci0 = (wave + gi * KS) * CG;
            // A operand.  CG = 16: Wt[co][ci0 + 4 kq + t][tap], t = 0..3: 4*T consecutive floats on a 16-byte
            // boundary.  CG = 4: Wt[co][kq][tap], T consecutive floats (zero for a channel the layer does not have).
            constexpr int NA = CG == 16 ? T : (T + 3) / 4;
            f32x4 aw[TM][NA];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                if constexpr (CG == 16) {
                    const f32x4* src = reinterpret_cast<const f32x4*>(Wt + ((size_t)(co0 + tm * 16 + li) * CI + ci0 + 4 * kq) * T);
#pragma unroll
                    for (int j = 0; j < T; ++j) aw[tm][j] = src[j];
                } else {
                    const float* src = Wt + ((size_t)(co0 + tm * 16 + li) * CI + (kq < CI ? kq : 0)) * T;
#pragma unroll
                    for (int j = 0; j < 4 * NA; ++j) aw[tm][j / 4][j % 4] = (j < T && kq < CI) ? src[j] : 0.f;
                }
            }

            // stage the patch: LPC lanes share a channel and take the (row, vector) units of its PR patch rows in turn
            const int cl = lane / LPC;
            int cu = lane % LPC;
            // which positions a lane stages does not change from one channel group to the next, and the compiler would
            // work out every address ahead of the loop and keep them all in registers: hidden from it
            asm volatile("" : "+v"(cu));
            const bool chan = ci0 + cl < CI;
            // element index, within the image tensor, of patch position (0, 0) of this lane's channel (32-bit: an image
            // tensor has fewer than 2^31 elements), and how far the tensor itself starts off a 16-byte boundary
            const int chan0 = (ci0 + cl) * HW + iy0 * W + ix0;
            const int xmis = (int)((reinterpret_cast<size_t>(X) >> 2) & 3);
            // No branches and no lane masks in here: validity is the sign bit of an OR of differences (negative = outside),
            // spread over the word by an arithmetic shift and used to pick between two addresses.  A vector that lies
            // outside the image is fetched from the tensor's first 16 bytes instead, and a float that is not part of the
            // patch is written to the 16 bytes of padding behind the plane.  (With compares, the sixteen loads and
            // sixty-four stores of a batch each held a 64-bit mask in scalar registers, more than there are.)
            unsigned char* const plane = tile + (cl / 4) * PLANE + (cl % 4) * 4;
            constexpr int DUMMY = PLANE - 16;
            const int chan_out = chan ? 0 : -1;
            constexpr int JB = NLD < 16 ? NLD : 16;
            constexpr int NBATCH = (NLD + JB - 1) / JB, UNROLL = (NIMG == 1 && NBATCH <= 4) ? NBATCH : 1;
#pragma unroll UNROLL
            for (int j0 = 0; j0 < NLD; j0 += JB) {
                f32x4 v[JB];
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const int u = (j0 + jj) * LPC + cu;
                    const int r = u / NVR, vi = u % NVR;
                    const int iy = iy0 + r;
                    const int e0 = chan0 + r * W;                            // element index of patch position (r, 0)
                    const int c0 = 4 * vi - ((e0 + xmis) & 3);               // patch column of the vector's first float
                    const int out = (chan_out | (NU - 1 - u) | iy | (H - 1 - iy) | (c0 + 3 - c_lo) | (c_hi - 1 - c0)) >> 31;
                    v[jj] = *reinterpret_cast<const f32x4*>(X + (((e0 + c0) & ~out) | (-xmis & out)));
                }
                asm volatile("" : "+v"(cu));   // likewise: the stores work their addresses out again, one vector at a time
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const int u = (j0 + jj) * LPC + cu;
                    const int r = u / NVR, vi = u % NVR;
                    const int iy = iy0 + r;
                    const int c0 = 4 * vi - ((chan0 + r * W + xmis) & 3);
                    const int row_out = chan_out | (NU - 1 - u) | iy | (H - 1 - iy);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int c = c0 + e;
                        const int out = (row_out | (c - c_lo) | (c_hi - 1 - c)) >> 31;
                        *reinterpret_cast<float*>(plane + ((((r * PC + c) * 16) & ~out) | (DUMMY & out))) = v[jj][e];
                    }
                }
            }

            // the taps: read the next tap's operands while this one multiplies
            if constexpr (CG == 16) {
                f32x4 b[2][PB];
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) b[0][pb] = *reinterpret_cast<const f32x4*>(bbase[pb]);
#pragma unroll
                for (int tap = 0; tap < T; ++tap) {
                    if (tap + 1 < T) {
                        const int noff = (((tap + 1) / KW) * PC + (tap + 1) % KW) * 16;
#pragma unroll
                        for (int pb = 0; pb < PB; ++pb) b[(tap + 1) & 1][pb] = *reinterpret_cast<const f32x4*>(bbase[pb] + noff);
                    }
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                            for (int pb = 0; pb < PB; ++pb)
                                acc[tm][pb] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[tm][(t * T + tap) / 4][(t * T + tap) % 4],
                                                                                   b[tap & 1][pb][t], acc[tm][pb], 0, 0, 0);
                }
            } else {
                float b[2][PB];
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) b[0][pb] = *reinterpret_cast<const float*>(bbase[pb]);
#pragma unroll
                for (int tap = 0; tap < T; ++tap) {
                    if (tap + 1 < T) {
                        const int noff = (((tap + 1) / KW) * PC + (tap + 1) % KW) * 16;
#pragma unroll
                        for (int pb = 0; pb < PB; ++pb) b[(tap + 1) & 1][pb] = *reinterpret_cast<const float*>(bbase[pb] + noff);
                    }
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                        for (int pb = 0; pb < PB; ++pb)
                            acc[tm][pb] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[tm][tap / 4][tap % 4], b[tap & 1][pb], acc[tm][pb], 0, 0, 0);
                }
            }
        }

        if constexpr (KS == 1) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) store_block(Y, co0, oy0 + pb, ox0, tm, acc[tm][pb], lane);
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
                    store_block(Y, co0, oy0 + u % PB, ox0, u / PB, s, lane);
                }
            }
        }
    }
};

// The tiling the library gives a convolution it has no hand-picked one for: as many output channels per
// workgroup as keep the filter fragments of a wave within ~72 registers (the staged patch is shared by all
// of them), 64 pixels (or the whole image when it has fewer), and as many waves over the channel groups as
// leave room for two workgroups' patches in a CU's LDS.
//
// The pixels are a rectangle of 16 columns (ConvF32Rect) for filters larger than 1 x 1 on wide images whose
// rows fill their 16-column tiles well -- at least 64 outputs wide, or at least 44 (any width at a stride: 64
// consecutive outputs of a strided layer need twice the image rows) with five sixths of the tile columns in
// use -- else 64 consecutive pixels (ConvF32Lds).  Measured at batch 1024, rectangle against
// consecutive pixels: 2.3-2.5x on 147-, 149- and 299-wide images, 2.2x on 55 outputs at stride 2, 1.6x for the
// 7 x 7 on 224, 1.3x on 73 and on 48, 1.1x on 56, 54 and 44; 1.0x on 50 (14 of its 64 tile columns idle);
// 0.8-0.9x on 35- and 28-wide images and 0.45-0.55x on 17-, 8- and 7-wide ones, whose rows fill half of a
// tile or less; at stride 2 1.14x on 28 and 1.23x on 14 outputs, 0.72x on 17, 0.55x on 8, 0.41x on 7; 1 x 1
// filters have no halo to save.
//
// The rectangle has 4 rows while a wave's patch of 16 channels stays within 12.5 KB, else 2, else 1: a stride
// widens the patch (9 x 33 pixels for 4 rows of a 3 x 3 filter at stride 2, 7 x 63 for 2 rows at stride 4), and
// the smaller patch lets more workgroups share a CU and hide the staging of each other's patches: 2 rows against
// 4 at stride 2, 1.20x (112-wide, 64 channels) and 1.12x (147-wide, 32 channels); 1 row against 2 at stride 4,
// 1.4x (227-wide).
//
// A strided layer with so few output channels that it computes less per byte of image than the chip can
// (CO x taps / (2 x stride^2) flops per byte against ~20) is bound by reading the image: one workgroup then
// computes all output channels (up to 64), so that the image is read once (1.14x on the 227-wide layer).
template <int CI, int CO, int H, int W, int KH, int KW, int S, int P, int NIMG>
struct ConvTiling {
    static constexpr int T = KH * KW;
    static constexpr int OH = (H - KH + 2 * P) / S + 1, OW = (W - KW + 2 * P) / S + 1;
    static constexpr int OHW = OH * OW;
    static constexpr bool RECT = T > 1 && (OW >= 64 || ((OW >= 44 || S > 1) && 6 * OW >= 5 * ((OW + 15) / 16 * 16)));
    static constexpr int patch_bytes(int th) { return ((th - 1) * S + KH) * (15 * S + KW) * (CI >= 16 ? 64 : 16); }
    static constexpr int TH = patch_bytes(4) <= 12800 ? 4 : patch_bytes(2) <= 12800 ? 2 : 1;
    static constexpr int pick_bm()
    {
        if (CI < 16) return 16;
        if (T == 1)      // a 1x1 filter is one register per row block: as many output channels as divide CO, up to 80
            for (int bm = 80; bm > 16; bm -= 16)     // (96 measured slower than 64 on the 8x8 and 17x17 layers)
                if (CO % bm == 0) return bm;
        if (RECT && CO * T < 40 * S * S)             // bound by reading the image
            for (int bm = 64; bm > 16; bm -= 16)
                if (CO % bm == 0) return bm;
        if (CO % 64 == 0 && 4 * T <= 18) return 64;
        if (CO % 48 == 0 && 3 * T <= 18) return 48;
        if (CO % 32 == 0 && 2 * T <= 18) return 32;
        return 16;
    }
    static constexpr int BM = pick_bm();
    static constexpr int PB = OHW >= 64 ? 4 : (OHW + 15) / 16;
    static constexpr int NGROUP = CI >= 16 ? CI / 16 : 1;
    // (only the chosen form is instantiated: the other may not fit this shape at all)
    static constexpr int TILE = std::conditional_t<RECT, ConvF32Rect<CI, CO, H, W, KH, KW, S, P, BM, TH, 1, NIMG>,
                                                   ConvF32Lds<CI, CO, H, W, KH, KW, S, P, BM, PB, 1, NIMG>>::TILE_BYTES;
    static constexpr int pick_ks()
    {
        // a rectangle gets no more waves than it has rows: the sum of the waves' partial tiles costs the same
        // whatever the rows' arithmetic (4 waves on 2 rows: 0.92x of 2 waves on the 112-wide stride-2 layer)
        const int most = RECT ? TH : 4;
        if (most >= 4 && NGROUP % 4 == 0 && 4 * TILE <= 80 * 1024) return 4;
        if (most >= 2 && NGROUP % 2 == 0 && 2 * TILE <= 80 * 1024) return 2;
        return 1;
    }
    static constexpr int KS = pick_ks();
    // A 1 x 1 filter on enough pixels to give every SIMD of the chip a 64-pixel tile is streamed (Conv1x1F32:
    // no LDS patch, no partial sums), with as many output channels per workgroup as divide CO, up to 80.
    // Measured at batch 1024 against the staged form: 2.1x on 64 -> 64 channels at 56 x 56 (5.2 TB/s of image and
    // output), 1.3-1.7x on the 35 x 35 layers, 1.8x on 73 x 73, 1.2-1.3x on 17 x 17 and 8 x 8 with 768-2048 channels
    // (120 TFLOP/s), 1.7x on 256 -> 256 at 56 x 56 (117 TFLOP/s).
    static constexpr bool STREAM = T == 1 && P == 0 && CI % 16 == 0 && CO % 16 == 0 && (long long)((OHW + 63) / 64) * NIMG >= 1024;
    static constexpr int stream_bm()
    {
        for (int bm = 80; bm > 16; bm -= 16)
            if (CO % bm == 0) return bm;
        return 16;
    }
    using staged = std::conditional_t<RECT, ConvF32Rect<CI, CO, H, W, KH, KW, S, P, BM, TH, KS, NIMG>,
                                      ConvF32Lds<CI, CO, H, W, KH, KW, S, P, BM, PB, KS, NIMG>>;
    // A rectangle on at most four input channels (one wave, a patch of a few KB) is held to twelve workgroups per
    // CU, three waves per SIMD: the sixteen its registers allow run the 7 x 7 on RGB 1.25x slower (LdsReserve).
    static constexpr int RESERVE = RECT && CI < 16 && (int)sizeof(typename staged::Smem) < 163840 / 12 - 1024
                                       ? 163840 / 12 - (int)sizeof(typename staged::Smem) : 0;
    using held = std::conditional_t<(RESERVE > 0), LdsReserve<staged, (RESERVE > 0 ? RESERVE : 1)>, staged>;
    using type = std::conditional_t<STREAM, Conv1x1F32<CI, CO, H, W, S, stream_bm(), 4, NIMG>, held>;
};
template <int CI, int CO, int H, int W, int KH, int KW, int S, int P, int NIMG = 1>
using ConvF32Auto = typename ConvTiling<CI, CO, H, W, KH, KW, S, P, NIMG>::type;

}  // namespace bfuse
