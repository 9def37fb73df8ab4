// Memory-bound sides: elementwise bias+ReLU, LayerNorm, causal softmax, RMSNorm+RoPE.
// All use 128-bit coalesced loads/stores and wave64 DPP reductions; none needs LDS or a
// barrier, so they can sit on either side of a horizontal or block fusion.
//
// The reference generates none of these (it only fuses GEMM-like TVM kernels); their
// arithmetic follows the reference's Relay dumps, cited per operator.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));

struct NoSmem {
    // empty: the operator uses no LDS
};

// y = max(x + b, 0) over COUNT floats, b a full-length vector.
// Workgroup v owns a contiguous slice of COUNT / GRID floats; consecutive lanes read
// consecutive 16-byte vectors.
template <int COUNT_, int THREADS_, int NBLOCKS_>
struct BiasRelu {
    static constexpr int COUNT = COUNT_, THREADS = THREADS_;
    static constexpr Dims3 GRID{NBLOCKS_, 1, 1};
    static constexpr Dims3 BLOCK{THREADS_, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int PER_BLOCK = COUNT / NBLOCKS_;
    static constexpr int ITERS = PER_BLOCK / (4 * THREADS);
    static_assert(COUNT % NBLOCKS_ == 0 && PER_BLOCK % (4 * THREADS) == 0, "slice must be whole vectors");
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void* F,
                                               void* O, Sync)
    {
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)vblock * (PER_BLOCK / 4);
        const f32x4* __restrict__ b = static_cast<const f32x4*>(F) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4 xv[ITERS], bv[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            xv[it] = x[it * THREADS + tid];
            bv[it] = b[it * THREADS + tid];
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            f32x4 s = xv[it] + bv[it];
            f32x4 r;
            r[0] = fmaxf(s[0], 0.f);
            r[1] = fmaxf(s[1], 0.f);
            r[2] = fmaxf(s[2], 0.f);
            r[3] = fmaxf(s[3], 0.f);
            y[it * THREADS + tid] = r;
        }
    }
};

// LayerNorm over the last axis of x[ROWS, D]; F holds gamma[D] then beta[D].
//   y = (x - mean) * (1 / sqrt(var + eps)) * gamma + beta, biased variance
// (files/bert-base-uncased.txt:8-16).  One wave per row, the row lives in registers
// (D/256 128-bit vectors per lane), mean and variance are two DPP reductions.
template <int ROWS_, int D_, int WAVES_, int EPS_E12_ = 1>
struct LayerNorm {
    static constexpr int ROWS = ROWS_, D = D_, WAVES = WAVES_;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr Dims3 GRID{ROWS / WAVES, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int VEC = D / 256;  // 128-bit vectors per lane
    static_assert(ROWS % WAVES == 0 && D % 256 == 0, "one wave per row, whole vectors per lane");
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void* F,
                                               void* O, Sync)
    {
        const int wave = tid >> 6, lane = tid & 63;
        const int row = vblock * WAVES + wave;
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)row * (D / 4);
        const f32x4* __restrict__ gamma = static_cast<const f32x4*>(F);
        const f32x4* __restrict__ beta = gamma + D / 4;
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)row * (D / 4);
        const float eps = 1e-12f * (float)EPS_E12_;

        f32x4 v[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = x[i * 64 + lane];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
        const float mean = wave_sum(s) / (float)D;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            v[i] -= mean;
            q += (v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3]);
        }
        const float var = wave_sum(q) / (float)D;
        const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const f32x4 g = gamma[i * 64 + lane], b = beta[i * 64 + lane];
            y[i * 64 + lane] = (v[i] * rstd) * g + b;
        }
    }
};

// softmax over the last axis of x[HEADS, S, S] with the causal mask: column j > row i is
// masked to -inf before the softmax, so its probability is exactly 0
// (files/gpt2.txt:35-36).  One wave per row; only the visible prefix is read.
template <int HEADS_, int S_, int WAVES_>
struct SoftmaxCausal {
    static constexpr int HEADS = HEADS_, S = S_, WAVES = WAVES_;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int ROWS = HEADS * S;
    static constexpr Dims3 GRID{ROWS / WAVES, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int VEC = S / 256;
    static_assert(ROWS % WAVES == 0 && S % 256 == 0, "one wave per row, whole vectors per lane");
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void*,
                                               void* O, Sync)
    {
        const int wave = tid >> 6, lane = tid & 63;
        const int row = vblock * WAVES + wave;
        const int i = row % S;  // query position: columns 0..i are visible
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)row * (S / 4);
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)row * (S / 4);
        const float ninf = -__builtin_inff();

        f32x4 v[VEC];
        float m = ninf;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const int col = (c * 64 + lane) * 4;
            v[c] = f32x4{ninf, ninf, ninf, ninf};
            if (col <= i) {
                const f32x4 t = x[c * 64 + lane];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[c][e] = (col + e <= i) ? t[e] : ninf;
            }
            m = fmaxf(m, fmaxf(fmaxf(v[c][0], v[c][1]), fmaxf(v[c][2], v[c][3])));
        }
        m = wave_max(m);
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[c][e] = expf(v[c][e] - m);  // exp(-inf) == 0 for masked columns
            s += (v[c][0] + v[c][1]) + (v[c][2] + v[c][3]);
        }
        s = wave_sum(s);
#pragma unroll
        for (int c = 0; c < VEC; ++c) y[c * 64 + lane] = v[c] / s;
    }
};

}  // namespace bfuse
