// bf16 GEMM side with fp32 accumulation on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16):  C[M,N] = A[M,K] . W[N,K]^T, bf16 in, bf16 out (one rounding,
// to nearest even, of the fp32 accumulator).
//
// W is stored [N,K] -- the reference's `dense` weight layout (out,in)
// (scripts/configure_kernels.py:21-26,50-58) -- so both operands are contiguous along K,
// which is what the bf16 MFMA wants: every lane supplies eight consecutive k of one row.
//
// One workgroup (four waves, 2 x 2) owns a BM x BN tile and walks K in steps of 64:
//   global -> VGPR (128-bit, coalesced: 8 lanes cover one 128-byte row segment)
//          -> LDS, rows padded to 144 bytes so the 128-bit operand reads of 16 lanes fall
//             in 16 disjoint bank groups
//          -> MFMA operands (ds_read_b128).
// LDS is double buffered and the next K-step's global loads are issued before the current
// step's MFMAs, so one barrier per step suffices.  The epilogue rounds to bf16, transposes
// the tile through LDS and writes 128-bit row segments.
//
// Workgroup ids map to tiles so that the BM-tiles sharing one slab of W run on the same XCD
// at the same time (consecutive workgroup ids go to consecutive XCDs): the slab is fetched
// from HBM once and hit in that XCD's L2 by the other M-tiles.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// fp32 -> bf16 bits, round to nearest even (finite inputs)
__device__ __forceinline__ unsigned int f32_to_bf16_bits(float f)
{
    unsigned int u = __builtin_bit_cast(unsigned int, f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float bf16_bits_to_f32(unsigned int h) { return __builtin_bit_cast(float, h << 16); }

template <int M_, int N_, int K_, int BM_, int BN_>
struct GemmBf16NT {
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_;
    static constexpr int BK = 64;
    static constexpr int THREADS = 256;
    static constexpr int WM = BM / 2, WN = BN / 2;      // wave tile (2 x 2 waves)
    static constexpr int TM = WM / 16, TN = WN / 16;    // 16x16 blocks per wave
    static constexpr int PITCH = BK + 8;                // bf16 elements per LDS row (144 bytes)
    static constexpr int NKT = K / BK;
    static constexpr int CHUNKS = (BM + BN) * (BK / 8); // 16-byte chunks per stage
    static constexpr int CPT = CHUNKS / THREADS;        // chunks per thread
    static constexpr int CPITCH = BN + 8;               // epilogue tile row pitch (bf16)
    static constexpr int OCHUNKS = BM * (BN / 8);
    static_assert(M % BM == 0 && N % BN == 0 && K % BK == 0, "tile must divide the problem");
    static_assert(WM % 16 == 0 && WN % 16 == 0 && BN % 8 == 0, "wave tile must be whole 16x16 blocks");
    static_assert(CHUNKS % THREADS == 0 && OCHUNKS % THREADS == 0, "whole chunks per thread");
    static constexpr int MT = M / BM, NT = N / BN;
    static_assert((MT * NT) % 8 == 0 && NT % 8 == 0, "tiles are dealt to 8 XCDs");

    static constexpr Dims3 GRID{MT * NT, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;

    static constexpr int STAGE_ELEMS = (BM + BN) * PITCH;
    static constexpr int EPI_ELEMS = BM * CPITCH;
    struct Smem {
        __attribute__((aligned(16))) unsigned short t[(2 * STAGE_ELEMS > EPI_ELEMS) ? 2 * STAGE_ELEMS : EPI_ELEMS];
    };

    // chunk c of a stage: rows 0..BM-1 are A rows, BM.. are W rows; 8 chunks per row
    __device__ static __forceinline__ void load_tile(u32x4 (&r)[CPT], const unsigned short* __restrict__ A,
                                                     const unsigned short* __restrict__ Wt, int m0, int n0, int k0,
                                                     int tid)
    {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * THREADS;
            const int row = c >> 3, col = (c & 7) * 8;
            const unsigned short* src = row < BM ? A + (size_t)(m0 + row) * K + k0 + col
                                                 : Wt + (size_t)(n0 + row - BM) * K + k0 + col;
            r[i] = *reinterpret_cast<const u32x4*>(src);
        }
    }
    __device__ static __forceinline__ void store_tile(const u32x4 (&r)[CPT], unsigned short* stage, int tid)
    {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * THREADS;
            const int row = c >> 3, col = (c & 7) * 8;
            *reinterpret_cast<u32x4*>(stage + row * PITCH + col) = r[i];
        }
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        const unsigned short* __restrict__ A = static_cast<const unsigned short*>(I);
        const unsigned short* __restrict__ Wt = static_cast<const unsigned short*>(F);
        unsigned short* __restrict__ C = static_cast<unsigned short*>(O);
        // XCD x = vblock % 8 owns N-tiles x*NT/8 .. ; the MT tiles of one N-tile are adjacent slots
        const int xcd = vblock & 7, slot = vblock >> 3;
        const int nt = xcd * (NT / 8) + slot / MT, mt = slot % MT;
        const int m0 = mt * BM, n0 = nt * BN;
        const int wave = tid >> 6, lane = tid & 63;
        const int wm = wave >> 1, wn = wave & 1;
        const int li = lane & 15, kq = lane >> 4;

        f32x4 acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

        u32x4 regs[CPT];
        load_tile(regs, A, Wt, m0, n0, 0, tid);
        store_tile(regs, sm.t, tid);
        sync();

        for (int kt = 0; kt < NKT; ++kt) {
            const unsigned short* cur = sm.t + (kt & 1) * STAGE_ELEMS;
            if (kt + 1 < NKT) load_tile(regs, A, Wt, m0, n0, (kt + 1) * BK, tid);
            const unsigned short* a_base = cur + (wm * WM + li) * PITCH + 8 * kq;
            const unsigned short* b_base = cur + (BM + wn * WN + li) * PITCH + 8 * kq;
#pragma unroll 1
            for (int ks = 0; ks < BK / 32; ++ks) {
                bf16x8 af[TM];
#pragma unroll
                for (int a = 0; a < TM; ++a)
                    af[a] = *reinterpret_cast<const bf16x8*>(a_base + a * 16 * PITCH + ks * 32);
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    const bf16x8 bfr = *reinterpret_cast<const bf16x8*>(b_base + b * 16 * PITCH + ks * 32);
#pragma unroll
                    for (int a = 0; a < TM; ++a)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[a], bfr, acc[a][b], 0, 0, 0);
                }
            }
            if (kt + 1 < NKT) store_tile(regs, sm.t + ((kt + 1) & 1) * STAGE_ELEMS, tid);
            sync();
        }

        // epilogue: accumulator layout (lane (j, rg): rows 4*rg+v, column j) -> bf16 tile in LDS
        unsigned short* ct = sm.t;
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    ct[(wm * WM + a * 16 + 4 * kq + v) * CPITCH + wn * WN + b * 16 + li] =
                        (unsigned short)f32_to_bf16_bits(acc[a][b][v]);
        sync();
#pragma unroll
        for (int i = 0; i < OCHUNKS / THREADS; ++i) {
            const int c = tid + i * THREADS;
            const int row = c / (BN / 8), col = (c % (BN / 8)) * 8;
            *reinterpret_cast<u32x4*>(C + (size_t)(m0 + row) * N + n0 + col) =
                *reinterpret_cast<const u32x4*>(ct + row * CPITCH + col);
        }
    }
};

}  // namespace bfuse
