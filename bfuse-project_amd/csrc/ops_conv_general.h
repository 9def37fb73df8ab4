// Convolution of any filter size, stride, padding and batch (NCHW data, OIHW weights, dilation 1)
// as an implicit GEMM on the matrix cores with the image patch staged in LDS: the general form of
// Conv3x3F32Lds (ops_conv.h), which stays the tuned kernel for 3x3 / stride 1 / padding 1 on images
// whose rows are whole 16-byte chunks.
//
// Replaces the TVM-generated `conv2d` kernels of the reference for every argument list its
// generator takes (scripts/configure_kernels.py:28-38 shapes, :60-68 topi.nn.conv2d with strides,
// padding, dilation 1): the ResNet-18 layers of test-utils/examples/resnet-18.yaml -- 7x7 stride 2
// padding 3 on three input channels, 1x1 with stride 1 and 2, 3x3 with stride 2, and 3x3 on 14x14
// and 7x7 images.
//
//   out[co][p] = sum_k Wt[co][k] * Xcol[k][p],   p = oy*OW + ox,   k = (kh*KW + kw)*CG + c
//
// The input channels are taken in groups of CG (16, or 4 when the layer has at most 4): four
// consecutive k are four channels under ONE filter tap, so no im2col buffer is written.  One
// workgroup owns BM output channels x PB*16 consecutive output pixels; its KS waves split the channel
// groups, each wave stages the patch of its group in a zero-padded LDS tile of its own (no barrier in
// the loop) and walks the KH*KW taps; the partial tiles meet in LDS once and are summed in wave order.
//
// Staged tile of a group: the input rows iy_lo .. iy_lo+R-1 that the tile's output rows touch
// (iy_lo = oy_lo*S - P, R = (rows-1)*S + KH), every column -P .. W+P-1, layout
// [channel quad][row][column][4 channels].  The B operand of tap (kh, kw) for output pixel (oy, ox)
// then sits at position ((oy-oy_lo)*S + kh)*WP + ox*S + kw: a per-lane base plus a compile-time
// offset per tap, for any stride; padding and rows outside the image read as zero, as a border test
// would give.  Image rows that are not whole 16-byte chunks (W = 14, 7, 35, 299 ...) are staged with 8- or 4-byte
// loads (one image) or from aligned 16-byte loads over the contiguous span of rows (a batch).  A last pixel block that runs past the image (14x14 and 7x7 outputs are not multiples of 16
// pixels) computes on the last pixel again and is not stored.
//
// A batch of NIMG images is NIMG times the workgroups of one image; every image is tiled alike.  The pixel tiles
// of the whole batch, image after image, are what is dealt over the XCDs (tile_of): each XCD owns consecutive
// tiles and every channel tile of each.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <int CI_, int CO_, int H_, int W_, int KH_, int KW_, int S_, int P_, int BM_, int PB_, int KS_, int NIMG_ = 1>
struct ConvF32Lds {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr int CI = CI_, CO = CO_, H = H_, W = W_, KH = KH_, KW = KW_, S = S_, P = P_, BM = BM_, PB = PB_, KS = KS_, NIMG = NIMG_;
    static constexpr int OH = (H - KH + 2 * P) / S + 1, OW = (W - KW + 2 * P) / S + 1;
    static constexpr int HW = H * W, OHW = OH * OW, T = KH * KW;
    static constexpr int CG = CI >= 16 ? 16 : 4;        // channels per group
    static constexpr int NQ = CG / 4;                   // channel quads = planes of the tile = MFMAs per tap
    static constexpr int NGROUP = CG == 16 ? CI / 16 : 1;
    static constexpr int GPW = NGROUP / KS;             // groups per wave
    static constexpr int TM = BM / 16;
    static constexpr int TP = 16 * PB;                  // output pixels per tile (consecutive in row-major order)
    static constexpr int NPT = (OHW + TP - 1) / TP;
    static constexpr int SPAN0 = (TP + OW - 2) / OW + 1;         // output rows TP consecutive pixels can touch
    static constexpr int SPAN = SPAN0 < OH ? SPAN0 : OH;
    static constexpr int R = (SPAN - 1) * S + KH, WP = W + 2 * P;   // staged rows / columns
    static constexpr int NPOS = R * WP;
    // bytes of one channel quad, [position][4 channels], padded to 16 (mod 256): the planes then start one
    // 16-byte slot apart in the banks (see ops_conv.h)
    static constexpr int PLANE = (NPOS * 16 + 255) / 256 * 256 + 16;
    static constexpr int TILE_BYTES = NQ * PLANE;
    static constexpr int VW = W % 4 == 0 ? 4 : (W % 2 == 0 ? 2 : 1);   // floats per staging load: image rows start on VW*4-byte boundaries
    static constexpr int LPC = 64 / CG;                 // lanes that share a channel while staging
    static constexpr int NU = R * W / VW;               // staging units per channel
    static constexpr int NLD = (NU + LPC - 1) / LPC;    // wave-level loads per group
    static constexpr int NZ = (TILE_BYTES + 1023) / 1024;
    static_assert(CG == 16 ? CI % 16 == 0 : CI <= 4, "input channels: a multiple of 16, or at most 4");
    static_assert(CO % BM == 0 && BM % 16 == 0 && NGROUP % KS == 0, "channel tiling");
    static_assert(((KH - 1) * WP + KW - 1) * 16 + (NQ - 1) * PLANE + 16 < 65536, "tap offsets are 16-bit immediates");
    static_assert(S >= 1 && OH >= 1 && OW >= 1, "shape");

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
    // pixel tiles and every channel tile of each, so that the workgroups sharing an image patch use one L2
    // (as in Conv3x3F32Lds).
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

    // accumulator layout: lane (j = pixel, rg) owns output channels 4*rg+v of the block
    __device__ static __forceinline__ void store_block(float* __restrict__ Y, int co0, int p0, int tm, int pb,
                                                       const f32x4& blk, int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
        const int p = p0 + pb * 16 + j;
        if (p < OHW) {
#pragma unroll
            for (int v = 0; v < 4; ++v) Y[(size_t)(co0 + tm * 16 + 4 * rg + v) * OHW + p] = blk[v];
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
        const int p0 = pt * TP, co0 = ct * BM;
        const int oy_lo = p0 / OW;                     // first output row of the tile
        const int iy_lo = oy_lo * S - P;               // image row of staged row 0
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
        for (int pb = 0; pb < PB; ++pb) {
            int p = p0 + pb * 16 + li;
            if (p > OHW - 1) p = OHW - 1;              // past the image: a valid address, the result is not stored
            const int pos = ((p / OW - oy_lo) * S) * WP + (p % OW) * S;
            bbase[pb] = tile + pos * 16 + (CG == 16 ? kq * PLANE : kq * 4);
        }

        f32x4 acc[TM][PB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) acc[tm][pb] = f32x4{0.f, 0.f, 0.f, 0.f};

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
            // stage the patch: LPC lanes share a channel and take consecutive units (VW floats) of its R x W
            // rows, which are contiguous in memory
            const int cl = lane / LPC, cu = lane % LPC;
            // in batches of JB loads, so that a large patch (7x7 filters on 224-wide rows) does not need a
            // register per element
            // Rows that are not whole 16-byte chunks: a single image (latency regime) takes them with 8- or 4-byte
            // loads straight from their rows (9.9 / 11.4 / 17.0 us against 12.2 / 14.6 / 19.2 for the 14x14 and 7x7
            // layers of ResNet-18); a batch of images (throughput) from aligned 16-byte loads, a quarter of the load
            // instructions (1024 images: 20-45 % faster on 35-, 73-, 147- and 299-wide images, 8-11 % on 14 and 7).
            if constexpr (VW == 4 || W < 4 || NIMG == 1) {
                constexpr int JB = NLD < 16 ? NLD : 16;
                // a single image is in the latency regime: its few batches are unrolled (the next batch's loads go out
                // under this one's LDS writes); a batch of images keeps the registers for wider tiles and loops
                constexpr int NBATCH = (NLD + JB - 1) / JB, UNROLL = (NIMG == 1 && NBATCH <= 4) ? NBATCH : 1;
#pragma unroll UNROLL
                for (int j0 = 0; j0 < NLD; j0 += JB) {
                    float v[JB][VW];
#pragma unroll
                    for (int jj = 0; jj < JB; ++jj) {
                        const int u = (j0 + jj) * LPC + cu;
                        const int r = (u * VW) / W, x = (u * VW) % W;
                        const int iy = iy_lo + r;
                        const bool ok = j0 + jj < NLD && u < NU && iy >= 0 && iy < H && ci0 + cl < CI;
                        const float* src = X + (size_t)(ci0 + cl) * HW + iy * W + x;
                        if constexpr (VW == 4) {
                            const f32x4 q = ok ? *reinterpret_cast<const f32x4*>(src) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[jj][e] = q[e];
                        } else if constexpr (VW == 2) {
                            const f32x2 q = ok ? *reinterpret_cast<const f32x2*>(src) : f32x2{0.f, 0.f};
                            v[jj][0] = q[0];
                            v[jj][1] = q[1];
                        } else {
                            v[jj][0] = ok ? *src : 0.f;
                        }
                    }
#pragma unroll
                    for (int jj = 0; jj < JB; ++jj) {
                        const int u = (j0 + jj) * LPC + cu;
                        const int r = (u * VW) / W, x = (u * VW) % W;
                        const int iy = iy_lo + r;
                        if (j0 + jj < NLD && u < NU && iy >= 0 && iy < H && ci0 + cl < CI) {
                            float* dst = reinterpret_cast<float*>(tile + (cl / 4) * PLANE + (r * WP + P + x) * 16) + cl % 4;
#pragma unroll
                            for (int e = 0; e < VW; ++e) dst[4 * e] = v[jj][e];
                        }
                    }
                }
            } else {
                // Image rows that do not start on 16-byte boundaries (odd widths; any width when the image itself
                // starts off one): the rows of a channel that lie inside the image are one contiguous span, which
                // is fetched with ALIGNED 16-byte loads from the boundary below its start; each of a vector's
                // four floats then finds its own (row, column), and those before and behind the span are dropped.
                const int r_lo = iy_lo < 0 ? -iy_lo : 0;
                const int r_hi = H - iy_lo < R ? H - iy_lo : R;
                const int len = (r_hi - r_lo) * W;
                const float* span = X + (size_t)(ci0 + cl) * HW + (iy_lo + r_lo) * W;
                const int mis = (int)((reinterpret_cast<size_t>(span) >> 2) & 3);
                const f32x4* vec = reinterpret_cast<const f32x4*>(span - mis);
                const bool chan = ci0 + cl < CI;
                constexpr int NV = (R * W + 3) / 4 + 1;          // aligned vectors that can overlap a span
                constexpr int NLA = (NV + LPC - 1) / LPC;
                constexpr int JA = NLA < 16 ? NLA : 16;
                constexpr int NBATCH = (NLA + JA - 1) / JA, UNROLL = (NIMG == 1 && NBATCH <= 4) ? NBATCH : 1;
#pragma unroll UNROLL
                for (int j0 = 0; j0 < NLA; j0 += JA) {
                    f32x4 v[JA];
#pragma unroll
                    for (int jj = 0; jj < JA; ++jj) {
                        const int u = (j0 + jj) * LPC + cu;
                        const int i0 = 4 * u - mis;              // span index of the vector's first float
                        v[jj] = (chan && i0 + 3 >= 0 && i0 < len) ? vec[u] : f32x4{0.f, 0.f, 0.f, 0.f};
                    }
#pragma unroll
                    for (int jj = 0; jj < JA; ++jj) {
                        const int u = (j0 + jj) * LPC + cu;
                        const int i0 = 4 * u - mis;
                        int r = (i0 + W) / W - 1 + r_lo, x = (i0 + W) % W;   // i0 >= -3 and W >= 4
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (chan && i0 + e >= 0 && i0 + e < len)
                                reinterpret_cast<float*>(tile + (cl / 4) * PLANE + (r * WP + P + x) * 16)[cl % 4] = v[jj][e];
                            if (++x == W) {
                                x = 0;
                                ++r;
                            }
                        }
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
                        const int noff = (((tap + 1) / KW) * WP + (tap + 1) % KW) * 16;
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
                        const int noff = (((tap + 1) / KW) * WP + (tap + 1) % KW) * 16;
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

// An operator with its first two operands exchanged: a 1x1 / stride 1 convolution is the product
// Wt[CO, CI] . X[CI, H*W], i.e. a GEMM whose first operand is the convolution's SECOND (the weights).
template <class Op>
struct SwapOperands : Op {
    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, typename Op::Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        Op::run(vblock, tid, sm, F, I, O, sync);
    }
};

}  // namespace bfuse
