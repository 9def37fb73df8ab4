// 3x3 / stride 1 / pad 1 convolution (NCHW data, OIHW weights, batch 1) as an implicit GEMM
// on the matrix cores, and 3x3 / stride 2 / pad 1 max-pooling.
//
// Replaces the TVM-generated `conv2d` kernels of the reference
// (scripts/configure_kernels.py:28-38,60-68; e.g.
// legacy/tests/single_bgemm_conv2d/case-0_4/M_diff/case-2/cuda/kernels.cu:72-111); the
// max-pool side follows files/resnet-18.txt:8 (pool 3x3, stride 2, padding 1).
//
// Convolution as GEMM:  out[co][p] = sum_k  Wt[co][k] * Xcol[k][p],  p = y*W + x,
// with the reduction index ordered tap-major, k = (kh*3+kw)*CI + ci, so that four
// consecutive k are four input channels under ONE filter tap: the B operand of an MFMA
// step is then four loads at channel stride with one shared border test, and no im2col
// buffer is ever written.  One workgroup owns BM output channels x PB*16 pixels; its KS
// waves split the reduction by input channel: wave w takes the 16-channel groups w, w+KS, ...
// and walks all nine taps of a group before moving on, so the 16 x 576-byte weight rows and
// the 16 image channels it touches stay in the CU's vector L1 for nine stages.  The partial
// tiles meet in LDS once and are summed in wave order.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int CI_, int CO_, int H_, int W_, int BM_, int PB_, int KS_>
struct Conv3x3F32 {
    static constexpr int CI = CI_, CO = CO_, H = H_, W = W_, BM = BM_, PB = PB_, KS = KS_;
    static constexpr int HW = H * W;
    static constexpr int TM = BM / 16;
    static constexpr int NGROUP = CI / 16;           // 16-channel groups
    static constexpr int NST = 9 * NGROUP / KS;      // stages per wave: 16 channels of one tap each
    static constexpr int NPT = HW / (16 * PB);       // pixel tiles
    static constexpr int NBUF = 3;                   // register stages in flight
    static_assert(CI % 16 == 0 && CO % BM == 0 && BM % 16 == 0, "channel tiling");
    static_assert(HW % (16 * PB) == 0 && NGROUP % KS == 0, "pixel / reduction tiling");

    static constexpr Dims3 GRID{NPT, CO / BM, 1};
    static constexpr Dims3 BLOCK{64 * KS, 1, 1};
    static constexpr int THREADS = 64 * KS;
    static constexpr bool HAS_BARRIERS = KS > 1;

    struct Smem {
        f32x4 part[KS > 1 ? KS : 1][KS > 1 ? TM * PB : 1][64];
    };

    struct Frag {
        float a[TM][4];
        float b[PB][4];
    };

    // stage s of wave `wave`: channel group wave + (s/9)*KS, tap s%9
    __device__ static __forceinline__ void load_stage(Frag& f, const float* __restrict__ X,
                                                      const float* __restrict__ Wt, int co0, int wave, int s,
                                                      const int (&py)[PB], const int (&px)[PB], int lane)
    {
        const int i = lane & 15, kq = lane >> 4;
        const int tap = s % 9, ci0 = (wave + (s / 9) * KS) * 16 + 4 * kq;
        const int dy = tap / 3 - 1, dx = tap % 3 - 1;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                f.a[tm][t] = Wt[((size_t)(co0 + tm * 16 + i) * CI + ci0 + t) * 9 + tap];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            const int yy = py[pb] + dy, xx = px[pb] + dx;
            const bool in = (unsigned)yy < (unsigned)H && (unsigned)xx < (unsigned)W;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                f.b[pb][t] = in ? X[(size_t)(ci0 + t) * HW + yy * W + xx] : 0.f;
        }
    }

    __device__ static __forceinline__ void mma_stage(f32x4 (&acc)[TM][PB], const Frag& f)
    {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb)
                    acc[tm][pb] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[tm][t], f.b[pb][t], acc[tm][pb], 0, 0, 0);
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
        const Dims3 vb = delinearize(vblock, GRID);
        const int p0 = vb.x * (16 * PB), co0 = vb.y * BM;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        int py[PB], px[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            const int p = p0 + pb * 16 + (lane & 15);
            py[pb] = p / W;
            px[pb] = p % W;
        }

        f32x4 acc[TM][PB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) acc[tm][pb] = f32x4{0.f, 0.f, 0.f, 0.f};

        Frag buf[NBUF];
#pragma unroll
        for (int s = 0; s < NBUF - 1; ++s)
            if (s < NST) load_stage(buf[s], X, Wt, co0, wave, s, py, px, lane);
        for (int s0 = 0; s0 < NST; s0 += NBUF) {
#pragma unroll
            for (int u = 0; u < NBUF; ++u) {
                const int s = s0 + u;
                if (s < NST) {
                    if (s + NBUF - 1 < NST)
                        load_stage(buf[(u + NBUF - 1) % NBUF], X, Wt, co0, wave, s + NBUF - 1, py, px, lane);
                    mma_stage(acc, buf[u]);
                }
            }
        }

        if constexpr (KS == 1) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) store_block(Y, co0, p0, tm, pb, acc[tm][pb], lane);
        } else {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) sm.part[wave][tm * PB + pb][lane] = acc[tm][pb];
            sync();
            // block u is finished by wave u mod KS, summing the partials of waves 0..KS-1 in order
#pragma unroll
            for (int u0 = 0; u0 < TM * PB; u0 += KS) {
                const int u = u0 + wave;
                if (u < TM * PB) {
                    f32x4 s = sm.part[0][u][lane];
#pragma unroll
                    for (int w = 1; w < KS; ++w) s += sm.part[w][u][lane];
                    store_block(Y, co0, p0, u / PB, u % PB, s, lane);
                }
            }
        }
    }
};

// max over 3x3 windows, stride 2, padding 1 (padding never wins), x[C,H,W] -> y[C,H/2,W/2].
// One thread produces four consecutive outputs of a row from three input rows
// (two 128-bit loads + one scalar per row) and stores them with one 128-bit store.
template <int C_, int H_, int W_, int THREADS_>
struct MaxPool3x3S2 {
    static constexpr int C = C_, H = H_, W = W_, THREADS = THREADS_;
    static constexpr int OH = H / 2, OW = W / 2;
    static constexpr int QUADS = OW / 4;                 // 4-output groups per output row
    static constexpr int TOTAL = C * OH * QUADS;
    static_assert(H % 2 == 0 && W % 8 == 0, "even extent, rows of whole 8-float groups");
    static_assert(TOTAL % THREADS == 0, "whole workgroups");
    static constexpr Dims3 GRID{TOTAL / THREADS, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    struct Smem {};

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void*,
                                               void* O, Sync)
    {
        const float* __restrict__ x = static_cast<const float*>(I);
        float* __restrict__ y = static_cast<float*>(O);
        const int g = vblock * THREADS + tid;
        const int q = g % QUADS, oy = g / QUADS % OH, c = g / (QUADS * OH);
        const int ix0 = 8 * q;  // input columns ix0-1 .. ix0+7 feed outputs 4q .. 4q+3
        const float ninf = -__builtin_inff();
        float m0 = ninf, m1 = ninf, m2 = ninf, m3 = ninf;
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const int iy = 2 * oy - 1 + r;
            if (iy < 0 || iy >= H) continue;
            const float* row = x + ((size_t)c * H + iy) * W;
            const f32x4 a = *reinterpret_cast<const f32x4*>(row + ix0);
            const f32x4 b = *reinterpret_cast<const f32x4*>(row + ix0 + 4);
            const float l = ix0 > 0 ? row[ix0 - 1] : ninf;
            m0 = fmaxf(m0, fmaxf(fmaxf(l, a[0]), a[1]));
            m1 = fmaxf(m1, fmaxf(fmaxf(a[1], a[2]), a[3]));
            m2 = fmaxf(m2, fmaxf(fmaxf(a[3], b[0]), b[1]));
            m3 = fmaxf(m3, fmaxf(fmaxf(b[1], b[2]), b[3]));
        }
        *reinterpret_cast<f32x4*>(y + ((size_t)c * OH + oy) * OW + 4 * q) = f32x4{m0, m1, m2, m3};
    }
};

}  // namespace bfuse
