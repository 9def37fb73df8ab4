// fp32 GEMM side: C[M,N] = A[M,K] . B[K,N] (+ optional tanh-GELU), row-major, on the
// gfx950 matrix cores (v_mfma_f32_16x16x4_f32).
//
// Replaces the TVM-generated `dense` kernels of the reference
// (scripts/configure_kernels.py:50-58; body e.g. tests/benchmark/cuda/dense1_0_dense2_0_bfuse.cu:82+).
// Shapes are compile-time, as in the reference's generated kernels.  B is [K,N] (the
// reference's dense weight is (out,in) = [N,K]; values and results do not depend on it).
//
// Decomposition, chosen for problems that are only a few 16x16 blocks per SIMD:
//   * one workgroup = one BM x BN tile of C; its KS waves split K (wave w owns
//     k in [w*K/KS, (w+1)*K/KS)) and each accumulates the WHOLE tile over its k-range.
//     No operand is shared between waves, so operands go global -> VGPR directly in MFMA
//     layout with 128-bit loads and the main loop has no barrier at all;
//   * at the end the KS partial tiles meet in LDS (one barrier) and are summed in wave
//     order 0..KS-1, so the result does not depend on timing;
//   * columns are handled in groups of 64: lane (j = lane%16, kq = lane/16) loads
//     B[k+4kq+t][n0+4j .. n0+4j+3] (t = 0..3) with one 128-bit load each.  Component e of
//     those vectors feeds 16x16 block e of the group, whose column j therefore is global
//     column n0+4j+e: after the MFMAs a lane holds four consecutive columns of a row and
//     stores them with one 128-bit store.  A trailing group of 32 columns works the same way
//     with 64-bit loads and two blocks (lane j: columns 2j, 2j+1), a trailing group of 16
//     columns uses 32-bit loads/stores.
//   * lane (i = lane%16, kq) loads A[m0+i][k+4kq .. k+4kq+3]; component t is the A operand of
//     MFMA step t, matching B row k+4kq+t above (the instruction sums over kq).
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

enum Epilogue : int { kEpiNone = 0, kEpiGeluTanh = 1 };

// 0.5*x*(1+tanh(0.797885*(x+0.044715*x^3))) with the constants of the reference's GPT-2 dump
// (files/gpt2.txt:67-74), evaluated as x / (1 + exp(-2u)): 0.5*(1 + tanh u) is the logistic
// function of 2u, which has no cancellation for negative x and needs one v_exp_f32 and one
// v_rcp_f32 (both ~1 ulp) instead of the library tanh's several dozen instructions -- the
// epilogue runs on SIMDs whose issue slots other workgroups' MFMAs are competing for.
// exp2 overflows to +inf for very negative x (result -0, the limit) and flushes to 0 for very
// positive x (result x).
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float x3 = x * x * x;
    const float u = 0.797885f * (x + 0.044715f * x3);
    const float e = __builtin_amdgcn_exp2f(u * -2.885390081777927f);   // exp(-2u) = 2^(-2u log2 e)
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// B_NK_: the second operand is stored [N, K] (the reference's `dense` / `batch_matmul` layout, both operands
// contiguous along K): a lane then loads, for each of its four columns 4j+e, the four k it needs with ONE
// 128-bit load (component t is MFMA step t) where the [K, N] layout gives it, for each k-step t, four columns
// with one load -- the same number of loads and registers, indexed the other way round.
// BATCH_ > 1: BATCH_ independent products A[b] . B[b] of the same shape (the reference's bgemm,
// scripts/configure_kernels.py:14-19,40-48); workgroup v works on batch v / tiles, tile v % tiles.
template <int M_, int N_, int K_, int BM_, int BN_, int KS_, int EPI_ = kEpiNone, int NBUF_ = 2, int SCHED_ = 1, bool B_NK_ = false, int BATCH_ = 1>
struct GemmF32 {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr bool B_NK = B_NK_;
    static constexpr int BATCH = BATCH_;
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, KS = KS_, EPI = EPI_;
    static constexpr int TM = BM / 16;          // 16-row blocks per tile
    static constexpr int G4 = BN / 64;          // 64-column groups
    static constexpr int G2 = (BN % 64) / 32;   // trailing 32-column group
    static constexpr int G1 = (BN % 32) / 16;   // trailing 16-column group
    static constexpr int NB = 4 * G4 + 2 * G2 + G1;   // 16 x 16 accumulator blocks per row block
    static constexpr int KW = K / KS;           // k-range of one wave
    static constexpr int STAGE = 16;            // k per stage (one 128-bit A load)
    static constexpr int NSTAGE = KW / STAGE;
    static constexpr int NBUF = NBUF_;          // register stages in flight (>= 2)
    // A tile that does not divide the problem: the last row (column) tile starts BM rows (BN columns) before the
    // end instead of running past it.  It overlaps its neighbour, and both write the same bits to what they
    // share: an element of the product is the same sequence of multiply-adds over k in every tile.
    static constexpr int MT = (M + BM - 1) / BM, NT = (N + BN - 1) / BN;   // row and column tiles
    static_assert(M >= BM && N >= BN, "a tile is not larger than the problem");
    static_assert(BM % 16 == 0 && BN % 16 == 0 && K % (KS * STAGE) == 0, "shape/tile mismatch");
    static_assert(N % 4 == 0 && K % 4 == 0, "rows must be 16-byte aligned");
    static_assert(NSTAGE >= NBUF - 1, "k-range shorter than the prefetch depth");

    static constexpr int TILES = NT * MT;
    static constexpr Dims3 GRID{NT, MT, BATCH};
    static constexpr Dims3 BLOCK{64 * KS, 1, 1};
    static constexpr int THREADS = 64 * KS;
    static constexpr bool HAS_BARRIERS = KS > 1;
    static constexpr int NUNIT = TM * (G4 + G2 + G1);  // reduction / store units (one column group of one row block)
    // 32 accumulator blocks (a 128 x 64 tile) and their operand stages do not fit the 256 registers of two waves per SIMD
    static constexpr int MIN_WAVES_PER_EU = TM * NB >= 32 ? 1 : 2;

    // partial tiles of every wave, in accumulator layout
    struct Smem {
        f32x4 part[KS > 1 ? KS : 1][KS > 1 ? TM * NB : 1][64];
    };

    struct Frag {
        f32x4 a[TM];
        f32x4 b4[G4 > 0 ? G4 : 1][4];  // [group][t] -> 4 columns
        f32x2 b2[G2 > 0 ? G2 : 1][4];  // [group][t] -> 2 columns
        float b1[G1 > 0 ? G1 : 1][4];  // [group][t]
        // B_NK: b4[group][e] holds the four k of column 4j+e; the narrower groups likewise
        f32x4 n2[(B_NK && G2 > 0) ? G2 : 1][2];  // [group][e] -> 4 k of column 2j+e
        f32x4 n1[(B_NK && G1 > 0) ? G1 : 1];     // [group]    -> 4 k of column j
    };

    // Every address is a wave-uniform part (tile origin, k, the row block, the k-step t: scalar
    // registers) plus this lane's constant 32-bit offset: the loads then take the scalar-base form and
    // no vector instruction is spent on addresses between the MFMAs.
    __device__ static __forceinline__ void load_stage(Frag& f, const float* __restrict__ A,
                                                      const float* __restrict__ B, int m0, int n0,
                                                      int k, int lane)
    {
        const int i = lane & 15, kq = lane >> 4;
        const unsigned a_off = (unsigned)(i * K + 4 * kq) * 4u;            // bytes
        const unsigned b_off = (unsigned)(4 * kq * N + 4 * i) * 4u;
        const unsigned b2_off = (unsigned)(4 * kq * N + 2 * i) * 4u;
        const unsigned b1_off = (unsigned)(4 * kq * N + i) * 4u;
        const char* a_ub = reinterpret_cast<const char*>(A + (size_t)m0 * K + k);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            f.a[tm] = *reinterpret_cast<const f32x4*>(a_ub + (size_t)tm * 16 * K * 4 + a_off);
        if constexpr (B_NK) {
            // rows of B are columns of the product: lane (j = i, kq) reads B[n][k + 4kq .. + 3]
            const char* n_ub = reinterpret_cast<const char*>(B + (size_t)n0 * K + k);
            const unsigned n4_off = (unsigned)(4 * i * K + 4 * kq) * 4u;
            const unsigned n2_off = (unsigned)(2 * i * K + 4 * kq) * 4u;
            const unsigned n1_off = (unsigned)(i * K + 4 * kq) * 4u;
#pragma unroll
            for (int g = 0; g < G4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    f.b4[g][e] = *reinterpret_cast<const f32x4*>(n_ub + ((size_t)(g * 64 + e) * K) * 4 + n4_off);
#pragma unroll
            for (int g = 0; g < G2; ++g)
#pragma unroll
                for (int e = 0; e < 2; ++e)
                    f.n2[g][e] = *reinterpret_cast<const f32x4*>(n_ub + ((size_t)(G4 * 64 + g * 32 + e) * K) * 4 + n2_off);
#pragma unroll
            for (int g = 0; g < G1; ++g)
                f.n1[g] = *reinterpret_cast<const f32x4*>(n_ub + ((size_t)(G4 * 64 + G2 * 32 + g * 16) * K) * 4 + n1_off);
            return;
        }
        const char* b_ub = reinterpret_cast<const char*>(B + (size_t)k * N + n0);
#pragma unroll
        for (int g = 0; g < G4; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                f.b4[g][t] = *reinterpret_cast<const f32x4*>(b_ub + ((size_t)t * N + g * 64) * 4 + b_off);
#pragma unroll
        for (int g = 0; g < G2; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                f.b2[g][t] = *reinterpret_cast<const f32x2*>(b_ub + ((size_t)t * N + G4 * 64 + g * 32) * 4 + b2_off);
#pragma unroll
        for (int g = 0; g < G1; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                f.b1[g][t] = *reinterpret_cast<const float*>(b_ub + ((size_t)t * N + G4 * 64 + G2 * 32 + g * 16) * 4 + b1_off);
    }

    __device__ static __forceinline__ void mma_stage(f32x4 (&acc)[TM][NB], const Frag& f)
    {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
                for (int g = 0; g < G4; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[tm][4 * g + e] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            f.a[tm][t], B_NK ? f.b4[g][e][t] : f.b4[g][t][e], acc[tm][4 * g + e], 0, 0, 0);
#pragma unroll
                for (int g = 0; g < G2; ++g)
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        acc[tm][4 * G4 + 2 * g + e] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            f.a[tm][t], B_NK ? f.n2[g][e][t] : f.b2[g][t][e], acc[tm][4 * G4 + 2 * g + e], 0, 0, 0);
#pragma unroll
                for (int g = 0; g < G1; ++g)
                    acc[tm][4 * G4 + 2 * G2 + g] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        f.a[tm][t], B_NK ? f.n1[g][t] : f.b1[g][t], acc[tm][4 * G4 + 2 * G2 + g], 0, 0, 0);
            }
        }
    }

    __device__ static __forceinline__ float epilogue(float v)
    {
        if constexpr (EPI == kEpiGeluTanh) return gelu_tanh(v);
        return v;
    }

    // Store one unit (row block tm, column group u) held in accumulator layout:
    // lane (j, rg) owns rows 4*rg+v (v = 0..3).
    __device__ static __forceinline__ void store_group4(float* __restrict__ C, int m0, int n0, int tm,
                                                        int g, const f32x4 (&blk)[4], int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            f32x4 o;
            o[0] = epilogue(blk[0][v]);
            o[1] = epilogue(blk[1][v]);
            o[2] = epilogue(blk[2][v]);
            o[3] = epilogue(blk[3][v]);
            *reinterpret_cast<f32x4*>(C + (size_t)(m0 + tm * 16 + 4 * rg + v) * N + n0 + g * 64 + 4 * j) = o;
        }
    }
    __device__ static __forceinline__ void store_group2(float* __restrict__ C, int m0, int n0, int tm,
                                                        int g, const f32x4 (&blk)[2], int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            f32x2 o;
            o[0] = epilogue(blk[0][v]);
            o[1] = epilogue(blk[1][v]);
            *reinterpret_cast<f32x2*>(C + (size_t)(m0 + tm * 16 + 4 * rg + v) * N + n0 + G4 * 64 + g * 32 + 2 * j) = o;
        }
    }
    __device__ static __forceinline__ void store_group1(float* __restrict__ C, int m0, int n0, int tm,
                                                        int g, const f32x4& blk, int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
#pragma unroll
        for (int v = 0; v < 4; ++v)
            C[(size_t)(m0 + tm * 16 + 4 * rg + v) * N + n0 + G4 * 64 + G2 * 32 + g * 16 + j] = epilogue(blk[v]);
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        // Many products: whole products are dealt to the XCDs (id % 8 is taken as the XCD, as in XcdTiles), so that the
        // tiles of one product share one L2 and its operands are fetched once -- with 8 x 8 tiles per product a
        // rectangle per XCD fetches three times as much (measured at 1024 products: 3-7 % on the K = 512 products,
        // nothing on the others, which are not bound there).  Few products keep the rectangles (every XCD works on each).
        constexpr bool PRODUCT_PER_XCD = BATCH >= 64 && BATCH % 8 == 0;
        int batch = BATCH > 1 ? vblock / TILES : 0;
        if constexpr (PRODUCT_PER_XCD) {
            const int xcd = vblock & 7, slot = vblock >> 3;
            batch = (slot / TILES) * 8 + xcd;
            vblock = slot % TILES;
        }
        const float* __restrict__ A = static_cast<const float*>(I) + (size_t)batch * M * K;
        const float* __restrict__ B = static_cast<const float*>(F) + (size_t)batch * K * N;
        float* __restrict__ C = static_cast<float*>(O) + (size_t)batch * M * N;
        const Dims3 vb = PRODUCT_PER_XCD ? Dims3{vblock % NT, vblock / NT, 0}
                                         : XcdTiles<NT, MT, BM, BN>::tile(BATCH > 1 ? vblock % TILES : vblock);   // tiles dealt so that each XCD's L2 fetches as little as possible
        const int m0 = (M % BM != 0 && (int)vb.y == MT - 1) ? M - BM : vb.y * BM;
        const int n0 = (N % BN != 0 && (int)vb.x == NT - 1) ? N - BN : vb.x * BN;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        const int kbeg = wave * KW;

        f32x4 acc[TM][NB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int c = 0; c < NB; ++c) acc[tm][c] = f32x4{0.f, 0.f, 0.f, 0.f};

        Frag buf[NBUF];
#pragma unroll
        for (int s = 0; s < NBUF - 1; ++s) load_stage(buf[s], A, B, m0, n0, kbeg + s * STAGE, lane);

        // NSTAGE stages, NBUF-1 loads in flight; the loop is unrolled by NBUF so every buffer
        // index is a compile-time constant.
        for (int s0 = 0; s0 < NSTAGE; s0 += NBUF) {
#pragma unroll
            for (int u = 0; u < NBUF; ++u) {
                const int s = s0 + u;
                if (s < NSTAGE) {
                    if (s + NBUF - 1 < NSTAGE)
                        load_stage(buf[(u + NBUF - 1) % NBUF], A, B, m0, n0, kbeg + (s + NBUF - 1) * STAGE, lane);
                    // keep the loads ahead of this stage's MFMAs: the scheduler otherwise sinks
                    // them to the end of the stage and the next stage waits on them at once
                    if constexpr (SCHED_ == 1) __builtin_amdgcn_sched_barrier(0);
                    mma_stage(acc, buf[u]);
                }
            }
        }

        if constexpr (KS == 1) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
                for (int g = 0; g < G4; ++g) {
                    const f32x4 blk[4] = {acc[tm][4 * g], acc[tm][4 * g + 1], acc[tm][4 * g + 2], acc[tm][4 * g + 3]};
                    store_group4(C, m0, n0, tm, g, blk, lane);
                }
#pragma unroll
                for (int g = 0; g < G2; ++g) {
                    const f32x4 blk[2] = {acc[tm][4 * G4 + 2 * g], acc[tm][4 * G4 + 2 * g + 1]};
                    store_group2(C, m0, n0, tm, g, blk, lane);
                }
#pragma unroll
                for (int g = 0; g < G1; ++g) store_group1(C, m0, n0, tm, g, acc[tm][4 * G4 + 2 * G2 + g], lane);
            }
        } else {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int c = 0; c < NB; ++c) sm.part[wave][tm * NB + c][lane] = acc[tm][c];
            sync();
            // unit u = (tm, group); wave w finishes units u == w (mod KS), summing waves 0..KS-1 in order
#pragma unroll
            for (int u0 = 0; u0 < NUNIT; u0 += KS) {
                const int u = u0 + wave;
                if (u < NUNIT) {
                    const int tm = u / (G4 + G2 + G1), g = u % (G4 + G2 + G1);
                    if (g < G4) {
                        f32x4 blk[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            f32x4 s = sm.part[0][tm * NB + 4 * g + e][lane];
#pragma unroll
                            for (int w = 1; w < KS; ++w) s += sm.part[w][tm * NB + 4 * g + e][lane];
                            blk[e] = s;
                        }
                        store_group4(C, m0, n0, tm, g, blk, lane);
                    } else if (g < G4 + G2) {
                        f32x4 blk[2];
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            f32x4 s = sm.part[0][tm * NB + 4 * G4 + 2 * (g - G4) + e][lane];
#pragma unroll
                            for (int w = 1; w < KS; ++w) s += sm.part[w][tm * NB + 4 * G4 + 2 * (g - G4) + e][lane];
                            blk[e] = s;
                        }
                        store_group2(C, m0, n0, tm, g - G4, blk, lane);
                    } else {
                        const int b = 4 * G4 + 2 * G2 + (g - G4 - G2);
                        f32x4 s = sm.part[0][tm * NB + b][lane];
#pragma unroll
                        for (int w = 1; w < KS; ++w) s += sm.part[w][tm * NB + b][lane];
                        store_group1(C, m0, n0, tm, g - G4 - G2, s, lane);
                    }
                }
            }
        }
    }
};

// (LdsReserve, the adaptor that bounds how many workgroups of an operator are resident on a CU, is in wave.h)

}  // namespace bfuse
