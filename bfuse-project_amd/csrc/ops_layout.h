// Weight layout: W[ROWS, COLS] -> W^T[COLS, ROWS] for 16-bit elements.
//
// The bf16 GEMM side takes its weight as [N, K] -- the reference's `dense` layout (out, in),
// scripts/configure_kernels.py:21-26 -- because both operands of a bf16 MFMA are contiguous along K.
// A weight that is held as [K, N] is brought into that layout ONCE, when it is loaded (weights do not
// change between launches), by this kernel; the GEMM itself is unchanged.  Memory-bound: every element
// is read once and written once, through a 64 x 64 tile in LDS so that both sides move whole 128-byte
// lines.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef unsigned short u16x8_t __attribute__((ext_vector_type(8)));

template <int ROWS_, int COLS_>
struct Transpose16 {
    static constexpr int ROWS = ROWS_, COLS = COLS_, TILE = 64, THREADS = 256;
    static_assert(ROWS % TILE == 0 && COLS % TILE == 0, "whole 64 x 64 tiles");
    static constexpr int TR = ROWS / TILE, TC = COLS / TILE;
    static constexpr Dims3 GRID{TR * TC, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    // rows 132 bytes apart: the eight rows a lane gathers from and the eight lanes that gather from one
    // row fall into different banks
    static constexpr int PITCH = TILE + 2;
    struct Smem {
        unsigned short t[TILE][PITCH];
    };

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void*, void* O, Sync sync)
    {
        const unsigned short* __restrict__ in = static_cast<const unsigned short*>(I);
        unsigned short* __restrict__ out = static_cast<unsigned short*>(O);
        // consecutive tiles walk down a column of tiles: their output rows are contiguous in memory
        const int r0 = (vblock % TR) * TILE, c0 = (vblock / TR) * TILE;
        u16x8_t v[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * THREADS, r = c >> 3, c8 = c & 7;
            v[i] = *reinterpret_cast<const u16x8_t*>(in + (size_t)(r0 + r) * COLS + c0 + c8 * 8);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * THREADS, r = c >> 3, c8 = c & 7;
#pragma unroll
            for (int e = 0; e < 8; e += 2)   // 32-bit stores: a row starts on a 4-byte, not a 16-byte, boundary
                *reinterpret_cast<unsigned int*>(&sm.t[r][c8 * 8 + e]) = (unsigned int)v[i][e] | ((unsigned int)v[i][e + 1] << 16);
        }
        sync();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * THREADS, n = c >> 3, k8 = c & 7;
            u16x8_t w;
#pragma unroll
            for (int e = 0; e < 8; ++e) w[e] = sm.t[k8 * 8 + e][n];
            *reinterpret_cast<u16x8_t*>(out + (size_t)(c0 + n) * ROWS + r0 + k8 * 8) = w;
        }
    }
};

// The same for 32-bit elements: the fp32 GEMM sides take their weight as [K, N]; the reference's `dense`
// weight is (out, in) = [N, K] (scripts/configure_kernels.py:21-26).  A weight held in the reference's
// layout is transposed once, when it is loaded.  64 x 64 tiles through LDS, 128-bit loads and stores.
template <int ROWS_, int COLS_>
struct Transpose32 {
    static constexpr int ROWS = ROWS_, COLS = COLS_, TILE = 64, THREADS = 256;
    static_assert(ROWS % TILE == 0 && COLS % TILE == 0, "whole 64 x 64 tiles");
    static constexpr int TR = ROWS / TILE, TC = COLS / TILE;
    static constexpr Dims3 GRID{TR * TC, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    static constexpr int PITCH = TILE + 1;   // rows 65 words apart: a column of the tile falls into 64 different banks
    struct Smem {
        float t[TILE][PITCH];
    };

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void*, void* O, Sync sync)
    {
        typedef float f32x4_t __attribute__((ext_vector_type(4)));
        const float* __restrict__ in = static_cast<const float*>(I);
        float* __restrict__ out = static_cast<float*>(O);
        const int r0 = (vblock % TR) * TILE, c0 = (vblock / TR) * TILE;
        f32x4_t v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * THREADS, r = c >> 4, c4 = c & 15;
            v[i] = *reinterpret_cast<const f32x4_t*>(in + (size_t)(r0 + r) * COLS + c0 + c4 * 4);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * THREADS, r = c >> 4, c4 = c & 15;
#pragma unroll
            for (int e = 0; e < 4; ++e) sm.t[r][c4 * 4 + e] = v[i][e];
        }
        sync();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * THREADS, n = c >> 4, k4 = c & 15;
            f32x4_t w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = sm.t[k4 * 4 + e][n];
            *reinterpret_cast<f32x4_t*>(out + (size_t)(c0 + n) * ROWS + r0 + k4 * 4) = w;
        }
    }
};

}  // namespace bfuse
