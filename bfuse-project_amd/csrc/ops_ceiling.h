// Measured ceilings: kernels that do nothing but the one thing a roofline is drawn from, so that a
// benchmark run can state what THIS chip sustains next to the published peak it divides by.
//   MfmaStream   a dense stream of independent MFMAs with operands that toggle bits, no memory
//                traffic in the loop: what the matrix cores deliver at the clock the power
//                management grants them (the published peaks assume the boost clock)
// (the memory ceiling is CopyF32 in ops_rowwise.h).
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_rowwise.h"

namespace bfuse {

typedef short bf16x8_bits __attribute__((ext_vector_type(8)));

// 256 workgroups x eight waves (two per SIMD), every wave ITERS rounds of 2 x 7 independent
// accumulator tiles (the register shape of the bf16 GEMM's compute waves).  BF16: v_mfma_f32_16x16x32_bf16,
// else v_mfma_f32_16x16x4_f32.  Operands are made in registers from a hash of the thread's position
// (random sign, mantissa and low exponent bits; nothing overflows in ITERS rounds); I and F
// are not read.  O[workgroup * 512 + thread] receives the sum of the thread's accumulator elements:
// the same bytes on every launch.
template <bool BF16_, int ITERS_, int UNROLL_ = 8>
struct MfmaStream {
    static constexpr bool BF16 = BF16_;
    static constexpr int ITERS = ITERS_, THREADS = 512, WORKGROUPS = 256;
    static constexpr Dims3 GRID{WORKGROUPS, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    using Smem = NoSmem;
    // flops one launch performs
    static constexpr double FLOPS = (double)WORKGROUPS * (THREADS / 64) * 14.0 * ITERS * (BF16 ? 16384.0 : 2048.0);

    __device__ static __forceinline__ unsigned mix(unsigned x)
    {
        x ^= x >> 16;
        x *= 0x7feb352dU;
        x ^= x >> 15;
        x *= 0x846ca68bU;
        x ^= x >> 16;
        return x;
    }
    // a bf16 bit pattern: random sign, mantissa and low exponent bits, magnitudes 1/128 .. 2 (sums of
    // 32-term products over ITERS rounds stay far inside fp32's range)
    __device__ static __forceinline__ short random_bf16(unsigned h) { return (short)((h & 0x80ff) | 0x3c00 | ((h >> 20) & 0x300)); }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void*, const void*, void* O, Sync)
    {
        f32x4 acc[2][7];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 7; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        bf16x8_bits a[2], b[7];
        float fa[2], fb[7];
        const unsigned t = (unsigned)vblock * 1024u + (unsigned)tid;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int e = 0; e < 8; ++e) a[i][e] = random_bf16(mix(t * 64u + i * 8u + e));
            fa[i] = ((float)(mix(t * 7u + i) & 0xffffu) / 65536.f - 0.5f) * 0.0625f;
        }
#pragma unroll
        for (int j = 0; j < 7; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) b[j][e] = random_bf16(mix(t * 64u + 32u + j * 8u + e));
            fb[j] = ((float)(mix(t * 11u + j) & 0xffffu) / 65536.f - 0.5f) * 0.0625f;
        }
#pragma unroll UNROLL_
        for (int it = 0; it < ITERS; ++it) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 7; ++j) {
                    if constexpr (BF16)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
                }
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 7; ++j) s += (acc[i][j][0] + acc[i][j][1]) + (acc[i][j][2] + acc[i][j][3]);
        static_cast<float*>(O)[(size_t)vblock * THREADS + tid] = s;
    }
};

}  // namespace bfuse
