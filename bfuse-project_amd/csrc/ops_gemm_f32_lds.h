// fp32 GEMM side, LDS-staged variant:  C[M,N] = A[M,K] . B[K,N] (+ optional tanh-GELU).
//
// Same arithmetic as GemmF32 (v_mfma_f32_16x16x4_f32), different decomposition, for tiles
// that divide evenly over waves WITHOUT splitting K: the workgroup's waves form a
// (BM/16) x (BN/WN) grid, each owning a 16 x WN strip of the tile over the whole K, so a wave
// holds only WN/16 accumulator blocks (12 VGPRs for WN = 48) and the kernel stays far below
// the 128-VGPR line -- four or more waves per SIMD, which is what lets a memory-bound
// operator's waves live next to it in a fused kernel.
//
// Operands are shared through LDS and arrive by direct global->LDS loads
// (global_load_lds_dwordx4) into a ring of NSTG stages of BK = 32 k; NSTG-1 stages are in
// flight; one fence-free barrier per stage, taken one K-substep BEFORE the stage is needed so
// that its first operand reads overlap the previous stage's last MFMAs.  A wave-level load
// writes 64 x 16 contiguous bytes, so rows cannot be padded; bank conflicts are avoided by
// permuting which global chunk each lane fetches:
//   A stage [BM][32] : 16-byte chunk c of row r sits at chunk position c ^ ((r >> 1) & 7)
//   B stage [32][BN] : row k is rotated right by 4*((k/4)%4) chunks (16 floats each), so the four
//                      k-quads a wave reads at once fall in four different bank ranges.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_gemm_f32.h"
#include "wave.h"

namespace bfuse {

template <int M_, int N_, int K_, int BM_, int BN_, int WN_, int EPI_ = kEpiNone, int NSTG_ = 4>
struct GemmF32Lds {
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, WN = WN_, EPI = EPI_, NSTG = NSTG_;
    static constexpr int BK = 32;
    static constexpr int WAVES_M = BM / 16, WAVES_N = BN / WN, WAVES = WAVES_M * WAVES_N;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int TN = WN / 16;                    // accumulator blocks per wave
    static constexpr int NKT = K / BK;
    static constexpr int A_CHUNKS = BM * (BK / 4);        // 16-byte chunks of the A stage
    static constexpr int B_ROWCH = BN / 4;                // chunks per B row
    static constexpr int B_CHUNKS = BK * B_ROWCH;
    static constexpr int A_BYTES = A_CHUNKS * 16, B_BYTES = B_CHUNKS * 16;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int A_INSTR = A_CHUNKS / 64, B_INSTR = B_CHUNKS / 64, INSTR = A_INSTR + B_INSTR;
    static constexpr int IPW_HI = (INSTR + WAVES - 1) / WAVES;   // wave-level loads per stage: waves < N_HI issue IPW_HI,
    static constexpr int N_HI = INSTR - (IPW_HI - 1) * WAVES;    // the others IPW_HI - 1
    static_assert(M % BM == 0 && N % BN == 0 && K % BK == 0 && BM % 16 == 0 && BN % WN == 0 && WN % 16 == 0, "tiling");
    static_assert(A_CHUNKS % 64 == 0 && B_CHUNKS % 64 == 0 && BN % 16 == 0, "whole wave-level loads per stage");
    static_assert(NSTG >= 3 && NSTG <= 6 && NKT >= NSTG - 1 && NSTG * STAGE_BYTES <= 160 * 1024, "ring shape");
    static_assert((B_ROWCH % 4) == 0 && BN >= 64, "row rotation works on groups of four chunks");

    static constexpr Dims3 GRID{N / BN, M / BM, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    static constexpr bool LOOP_BARRIERS = true;   // one workgroup barrier per K-stage, not only in the epilogue

    struct Smem {
        __attribute__((aligned(1024))) unsigned char t[NSTG * STAGE_BYTES];
    };
    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    template <int N_OUT>
    __device__ static __forceinline__ void wait_vm()
    {
        __builtin_amdgcn_s_waitcnt((N_OUT & 0xF) | ((N_OUT >> 4) << 14) | 0x0F70);
    }

    // global source of this lane for wave-level load j of a stage at k = 0
    __device__ static __forceinline__ const float* source(int j, int lane, const float* A, const float* B, int m0, int n0)
    {
        const int c = (j < A_INSTR ? j : j - A_INSTR) * 64 + lane;
        if (j < A_INSTR) {
            const int row = c >> 3, pc = c & 7;
            return A + (size_t)(m0 + row) * K + ((pc ^ ((row >> 1) & 7)) << 2);
        }
        const int row = c / B_ROWCH, pc = c % B_ROWCH;
        const int gc = (pc + B_ROWCH - 4 * ((row >> 2) & 3)) % B_ROWCH;   // undo the rotation
        return B + (size_t)row * N + n0 + 4 * gc;
    }

    __device__ static __forceinline__ void issue(const float* const (&src)[IPW_HI], const int (&kstride)[IPW_HI],
                                                 lds_u8* stage_base, const int (&lds_off)[IPW_HI], int n_mine, int kt)
    {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int i = 0; i < IPW_HI; ++i)
            if (i < n_mine)
                __builtin_amdgcn_global_load_lds(src[i] + (size_t)kt * kstride[i], stage_base + lds_off[i], 16, 0, 0);
#endif
    }

    // ---- operand fragments of one K-substep (16 k): read and waited for by hand, so that the
    // next substep's reads stay in flight under this substep's MFMAs (the compiler would wait
    // for all outstanding LDS reads before the first MFMA)
    struct Frag {
        f32x4 a;          // A[row][4kq .. 4kq+3]
        float b[TN][4];   // B[4kq + t][column] per accumulator block
    };
    static constexpr int READS = 1 + 4 * TN;
    static_assert(TN == 3, "the dependency list in wait_set names three accumulator blocks");

    __device__ static __forceinline__ void read_set(Frag& f, int a_addr, const int (&b_addr)[TN], int stage_off)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read_b128 %0, %1" : "=v"(f.a) : "v"(a_addr + stage_off));
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int ad = b_addr[b] + stage_off;
            asm volatile("ds_read_b32 %0, %1" : "=v"(f.b[b][0]) : "v"(ad));
            asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(f.b[b][1]) : "v"(ad), "n"(BN * 4));
            asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(f.b[b][2]) : "v"(ad), "n"(BN * 8));
            asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(f.b[b][3]) : "v"(ad), "n"(BN * 12));
        }
#endif
    }
    // wait until at most N_OUT of this wave's LDS reads are outstanding; LDS reads return in
    // order, so everything issued before the newest N_OUT has landed
    template <int N_OUT>
    __device__ static __forceinline__ void wait_set(Frag& f)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%13)"
                     : "+v"(f.a), "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[0][2]), "+v"(f.b[0][3]), "+v"(f.b[1][0]),
                       "+v"(f.b[1][1]), "+v"(f.b[1][2]), "+v"(f.b[1][3]), "+v"(f.b[2][0]), "+v"(f.b[2][1]),
                       "+v"(f.b[2][2]), "+v"(f.b[2][3])
                     : "n"(N_OUT));
#endif
    }

    // this wave's loads of a K-step have landed once only `newer` later steps' loads are outstanding
    __device__ static __forceinline__ void wait_stage(int wave, int newer)
    {
        if (wave < N_HI) {
            if (newer >= 3) wait_vm<IPW_HI * 3>();
            else if (newer == 2) wait_vm<IPW_HI * 2>();
            else if (newer == 1) wait_vm<IPW_HI>();
            else wait_vm<0>();
        } else {
            if (newer >= 3) wait_vm<(IPW_HI - 1) * 3>();
            else if (newer == 2) wait_vm<(IPW_HI - 1) * 2>();
            else if (newer == 1) wait_vm<IPW_HI - 1>();
            else wait_vm<0>();
        }
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        const float* __restrict__ A = static_cast<const float*>(I);
        const float* __restrict__ B = static_cast<const float*>(F);
        float* __restrict__ C = static_cast<float*>(O);
        const Dims3 vb = delinearize(vblock, GRID);
        const int m0 = vb.y * BM, n0 = vb.x * BN;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int wm = wave / WAVES_N, wn = wave % WAVES_N;
        const int li = lane & 15, kq = lane >> 4;

        // this wave's share of the stage's wave-level loads: j = wave, wave + WAVES, ...
        const int n_mine = wave < N_HI ? IPW_HI : IPW_HI - 1;
        const float* src[IPW_HI];
        int kstride[IPW_HI], lds_off[IPW_HI];
#pragma unroll
        for (int i = 0; i < IPW_HI; ++i) {
            const int j = wave + i * WAVES;
            const int jj = j < INSTR ? j : INSTR - 1;
            src[i] = source(jj, lane, A, B, m0, n0);
            kstride[i] = jj < A_INSTR ? BK : BK * N;              // floats per K-step
            lds_off[i] = jj < A_INSTR ? jj * 1024 : A_BYTES + (jj - A_INSTR) * 1024;
        }
        lds_u8* const lds = (lds_u8*)sm.t;

        f32x4 acc[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (int s = 0; s < NSTG - 1; ++s) issue(src, kstride, lds + s * STAGE_BYTES, lds_off, n_mine, s);

        // operand read addresses (absolute LDS byte addresses in stage 0)
        const int lds_base = (int)(unsigned)(unsigned long long)lds;
        const int arow = wm * 16 + li;
        int a_rd[BK / 16];
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks)
            a_rd[ks] = lds_base + arow * 128 + (((ks * 4 + kq) ^ ((arow >> 1) & 7)) << 4);
        // B element (k, n) of the stage sits at float index k*BN + (n + 16*((k/4)%4)) % BN
        int b_rd[BK / 16][TN];
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks)
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                const int k = ks * 16 + 4 * kq;   // + t below: same k/4 group for t = 0..3
                const int n = wn * WN + b * 16 + li;
                b_rd[ks][b] = lds_base + A_BYTES + 4 * (k * BN + (n + 16 * ((k >> 2) & 3)) % BN);
            }

        // K-step 0 has landed
        wait_stage(wave, NKT - 1 < NSTG - 2 ? NKT - 1 : NSTG - 2);
        sync.raw();
        Frag f[2];
        read_set(f[0], a_rd[0], b_rd[0], 0);
        int stage_off = 0;
#pragma unroll 1   // stays rolled: registers with reads in flight must never be spilled
        for (int kt = 0; kt < NKT; ++kt) {
#pragma unroll
            for (int ks = 0; ks < BK / 16; ++ks) {
                Frag& cur = f[ks & 1];
                Frag& nxt = f[(ks + 1) & 1];
                if (ks + 1 < BK / 16) {
                    read_set(nxt, a_rd[ks + 1], b_rd[ks + 1], stage_off);
                    wait_set<READS>(cur);
                } else if (kt + 1 < NKT) {
                    // last K-substep of this stage: the next stage must have landed; everyone is
                    // then past stage kt-1, whose buffer the load issued here overwrites
                    const int left = NKT - 2 - kt;
                    wait_stage(wave, left < NSTG - 3 ? left : NSTG - 3);
                    sync.raw();
                    if (kt + NSTG - 1 < NKT) {
                        int so = stage_off - STAGE_BYTES;
                        if (so < 0) so += NSTG * STAGE_BYTES;
                        issue(src, kstride, lds + so, lds_off, n_mine, kt + NSTG - 1);
                    }
                    stage_off = stage_off + STAGE_BYTES == NSTG * STAGE_BYTES ? 0 : stage_off + STAGE_BYTES;
                    read_set(nxt, a_rd[0], b_rd[0], stage_off);
                    wait_set<READS>(cur);
                } else {
                    wait_set<0>(cur);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int b = 0; b < TN; ++b)
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.a[t], cur.b[b][t], acc[b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // accumulator layout: lane (j, rg) owns rows 4*rg+v, column j of each block
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float o = acc[b][v];
                if constexpr (EPI == kEpiGeluTanh) o = gelu_tanh(o);
                C[(size_t)(m0 + wm * 16 + 4 * kq + v) * N + n0 + wn * WN + b * 16 + li] = o;
            }
    }
};

}  // namespace bfuse
