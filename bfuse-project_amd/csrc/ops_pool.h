// 3x3 / stride 2 / pad 1 max-pooling (NCHW, batch 1).
//
// The reference fuses only GEMM-like operators; this side follows files/resnet-18.txt:8
// (`nn.max_pool2d`, pool 3x3, stride 2, padding 1, (1,64,112,112) -> (1,64,56,56)).
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));

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
