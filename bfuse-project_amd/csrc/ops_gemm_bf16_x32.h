// bf16 GEMM side on the 32x32x16 matrix instruction (v_mfma_f32_32x32x16_bf16):
// C[M,N] = A[M,K] . W[N,K]^T, bf16 in, fp32 accumulate, bf16 out.  Loads, LDS ring, swizzle,
// barriers, producer waves, tile -> XCD mapping and the epilogue's transposition are those of
// GemmBf16NTDma (ops_gemm_bf16.h); what differs is the instruction the compute waves multiply
// with, and with it the shape of their tiles.
//
// Why it was tried, and what came of it: a bf16 MFMA stream on MI355X is bound by power, not by
// the pipe.  With random operands and no memory traffic, 16x16x32 is accepted every ~20 clocks
// instead of 16 (at 1.83-1.99 GHz), 32x32x16 every 16.9 (at 1.71-1.77 GHz): 6-8 % more flops.
// Inside this GEMM the same trade goes the other way.  Read inside the kernels on one box, a
// 64-k stage takes 1042-1052 clocks here against 1124 with 16x16x32 -- the stalls do go -- but
// the shader clock the chip grants falls from 1.51 GHz to 1.26-1.36 GHz, and the kernel is 3-4 %
// slower (48.9 against 47.2 us).  It stays as a tested alternative; the 16x16x32 kernel is the
// headline.  Reading ahead further costs more than it hides (RD = 3: 48.9 us, 6: 49.4, 10: 50.4).
//
// Wave tiles: a 32x32 block needs whole multiples of 32 columns, and the 224-column workgroup
// tile that gives 256 workgroups (one per CU) is seven blocks wide.  The 2 * BM/32 compute waves
// are therefore NOT equal: the waves with wn = 0 own 32 rows x TN0 = 4 column blocks, those with
// wn = 1 own 32 x TN1 = 3.  wave = wn * WGM + wm, so that waves w and w + 4 -- which share a SIMD
// -- are one of each kind and every SIMD multiplies seven blocks per 16-k step (measured: 49.4 us
// against 51.0 with wave = 2 * wm + wn, where a SIMD hosts two waves of one kind).
//
// Operand reads: per 64-k stage a wave needs, in this order, A[ks], B[ks][0..TNW-1] for
// ks = 0..3 (16 k each): one 128-bit LDS read per fragment (lane = (row % 32, half): eight
// consecutive k of one row).  They are issued by hand RD reads ahead of the MFMA that consumes
// them and waited for with s_waitcnt lgkmcnt(n): LDS reads of a wave return in order, so "at
// most n outstanding" names exactly the fragments that have landed.  Addresses: one base
// register per (16-k step, operand, stage pair) -- the XOR swizzle is not additive in the k
// step -- with the column block and the stage as immediate offsets.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_gemm_bf16.h"
#include "wave.h"

namespace bfuse {

typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int M_, int N_, int K_, int BM_, int BN_, int NSTG_ = 3, int RD_ = 3, int PW_ = 4>
struct GemmBf16NT32 {
    static constexpr int WGM = BM_ / 32;
    using Base = GemmBf16NTDma<M_, N_, K_, BM_, BN_, NSTG_, 4, WGM, 2, PW_>;   // loads, ring and barriers
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, NSTG = NSTG_, PW = PW_;
    static constexpr int BK = Base::BK, NKT = Base::NKT, STAGE_BYTES = Base::STAGE_BYTES;
    static constexpr int NCOMP = 2 * WGM;
    static constexpr int THREADS = Base::THREADS, CTHREADS = Base::CTHREADS;
    static constexpr int KSTEPS = BK / 16;                 // 16-k steps per stage
    static constexpr int NBLK = BN / 32;                   // 32-column blocks of the workgroup tile
    static constexpr int TN0 = (NBLK + 1) / 2, TN1 = NBLK / 2;
    static constexpr int RD = RD_;                         // reads in flight ahead of the consuming MFMA
    static constexpr int RB = RD + 1;                      // B fragment registers (a ring)
    static constexpr int CPITCH = Base::CPITCH, OCHUNKS = Base::OCHUNKS;
    static_assert(BM % 32 == 0 && BN % 32 == 0 && TN1 >= 1, "32 x 32 blocks");
    static_assert(RD >= 1 && RD <= 14, "lgkmcnt is a 4-bit count");
    static_assert(STAGE_BYTES + (TN0 - 1) * 4096 + 4096 <= 65536, "stage + block offsets are 16-bit immediates");
    static constexpr int MT = Base::MT, NT = Base::NT;

    static constexpr Dims3 GRID = Base::GRID;
    static constexpr Dims3 BLOCK = Base::BLOCK;
    static constexpr bool HAS_BARRIERS = true;
    static constexpr bool LOOP_BARRIERS = true;   // one workgroup barrier per K-stage, not only in the epilogue
    using Smem = typename Base::Smem;
    using Src = typename Base::Src;
    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    struct Addr {
        int a[KSTEPS][(NSTG + 1) / 2], b[KSTEPS][(NSTG + 1) / 2];   // [..][h]: base of stage 2h
    };

    // ---- the read sequence of one stage for a wave with TNW column blocks -----------------------
    // read i: step ks = i / (1 + TNW); j = i % (1 + TNW): j == 0 -> A[ks], else B[ks][j - 1]
    template <int TNW> static constexpr int nreads() { return KSTEPS * (1 + TNW); }
    template <int TNW> static constexpr int need(int st) { return (st / TNW) * (1 + TNW) + 1 + st % TNW; }   // read MFMA group st waits for
    template <int TNW> static constexpr int issued(int st)   // reads issued before MFMA group st starts
    {
        if (st >= KSTEPS * TNW) return nreads<TNW>();
        const int n = need<TNW>(st) + RD + 1;
        return n < nreads<TNW>() ? n : nreads<TNW>();
    }

    template <int IMM>
    __device__ static __forceinline__ bf16x8 lds_read(int addr)
    {
        bf16x8 r;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
#else
        r = bf16x8{};
#endif
        return r;
    }
    template <int U, int TNW, int I, int END>
    __device__ static __forceinline__ void issue_reads(bf16x8 (&af)[KSTEPS], bf16x8 (&bq)[RB], const Addr& ad)
    {
        if constexpr (I < END) {
            constexpr int ks = I / (1 + TNW), j = I % (1 + TNW);
            if constexpr (j == 0) af[ks] = lds_read<(U % 2) * STAGE_BYTES>(ad.a[ks][U / 2]);
            else bq[(ks * TNW + j - 1) % RB] = lds_read<(U % 2) * STAGE_BYTES + (j - 1) * 4096>(ad.b[ks][U / 2]);
            issue_reads<U, TNW, I + 1, END>(af, bq, ad);
        }
    }
    template <int N_OUT>
    __device__ static __forceinline__ void wait_lds(bf16x8& b, bf16x8& a)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(b), "+v"(a) : "n"(N_OUT));
#endif
    }
    template <int U, int TNW, int ST>
    __device__ static __forceinline__ void step_chain(f32x16 (&acc)[TNW], bf16x8 (&af)[KSTEPS], bf16x8 (&bq)[RB], const Addr& ad)
    {
        if constexpr (ST < KSTEPS * TNW) {
            constexpr int ks = ST / TNW, b = ST % TNW;
            wait_lds<issued<TNW>(ST) - need<TNW>(ST) - 1>(bq[ST % RB], af[ks]);
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks], bq[ST % RB], acc[b], 0, 0, 0);
            issue_reads<U, TNW, issued<TNW>(ST), issued<TNW>(ST + 1)>(af, bq, ad);
            __builtin_amdgcn_sched_barrier(0);
            step_chain<U, TNW, ST + 1>(acc, af, bq, ad);
        }
    }

    // one K-step out of LDS stage U
    template <int U, int TNW, class Sync>
    __device__ static __forceinline__ void k_step(int kt, f32x16 (&acc)[TNW], const Addr& ad, const Src& src, unsigned lds,
                                                  bool full, Sync& sync)
    {
        if (kt >= NKT) return;
        if constexpr (PW == 0) Base::template load_step<U>(kt, src, lds, full, sync);
        else sync.raw();
        bf16x8 af[KSTEPS], bq[RB];
        issue_reads<U, TNW, 0, issued<TNW>(0)>(af, bq, ad);
        __builtin_amdgcn_sched_barrier(0);
        step_chain<U, TNW, 0>(acc, af, bq, ad);
    }

    // the K loop and the tile store of a compute wave that owns column blocks nb0 .. nb0 + TNW - 1
    template <int TNW, class Sync>
    __device__ static __forceinline__ void compute(int wm, int nb0, int lane, Smem& sm, const Src& src, unsigned lds, bool full,
                                                   Sync& sync)
    {
        const int r = lane & 31, g = lane >> 5;
        const unsigned lds_base = (unsigned)(unsigned long long)(lds_u8*)sm.t;
        Addr ad;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int c = ks * 2 + g;
            const int arow = wm * 32 + r, brow = BM + nb0 * 32 + r;
#pragma unroll
            for (int h = 0; h < (NSTG + 1) / 2; ++h) {
                ad.a[ks][h] = (int)lds_base + 2 * h * STAGE_BYTES + arow * 128 + ((c ^ ((arow >> 1) & 7)) << 4);
                ad.b[ks][h] = (int)lds_base + 2 * h * STAGE_BYTES + brow * 128 + ((c ^ ((brow >> 1) & 7)) << 4);
            }
        }
        f32x16 acc[TNW];
#pragma unroll
        for (int b = 0; b < TNW; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[b][e] = 0.f;

#pragma unroll 1
        for (int kt0 = 0; kt0 < NKT; kt0 += NSTG) {
            k_step<0, TNW>(kt0, acc, ad, src, lds, full, sync);
            if constexpr (NSTG > 1) k_step<1, TNW>(kt0 + 1, acc, ad, src, lds, full, sync);
            if constexpr (NSTG > 2) k_step<2, TNW>(kt0 + 2, acc, ad, src, lds, full, sync);
            if constexpr (NSTG > 3) k_step<3, TNW>(kt0 + 3, acc, ad, src, lds, full, sync);
        }
        sync();  // all waves are done reading the last stage before the tile buffer overwrites it

        // accumulator layout of the 32x32 instruction: lane (column r, half g) holds rows
        // 8 * (e / 4) + 4 * g + e % 4, e = 0..15
        unsigned short* ct = reinterpret_cast<unsigned short*>(sm.t);
#pragma unroll
        for (int b = 0; b < TNW; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                ct[(wm * 32 + 8 * (e / 4) + 4 * g + e % 4) * CPITCH + (nb0 + b) * 32 + r] = (unsigned short)f32_to_bf16_bits(acc[b][e]);
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F, void* O, Sync sync)
    {
        const unsigned short* __restrict__ A = static_cast<const unsigned short*>(I);
        const unsigned short* __restrict__ Wt = static_cast<const unsigned short*>(F);
        unsigned short* __restrict__ C = static_cast<unsigned short*>(O);
        const int xcd = vblock & 7, slot = vblock >> 3;
        const int nt = xcd * (NT / 8) + slot / MT, mt = slot % MT;
        const int m0 = mt * BM, n0 = nt * BN;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: scalar branches
        const bool compute_wave = wave < NCOMP;
        const bool loader = PW == 0 || !compute_wave;
        const int lw = PW == 0 ? wave : (compute_wave ? 0 : wave - NCOMP);   // index among the loading waves
        const bool full = lw < Base::GEXTRA;

        Src src;
        src.a_ub = reinterpret_cast<const char*>(A + (size_t)m0 * K);
        src.w_ub = reinterpret_cast<const char*>(Wt + (size_t)n0 * K);
        src.lw = lw;
#pragma unroll
        for (int i = 0; i < Base::GPW; ++i) {
            int row = 8 * (lw + i * Base::NWAVES) + (lane >> 3);
            if (row >= Base::ROWS) row = Base::ROWS - 1;  // slot not issued (see `full`)
            const int gc = (lane & 7) ^ ((row >> 1) & 7);
            src.voff[i] = (unsigned)((row < BM ? row : row - BM) * K + gc * 8) * 2u;
        }
        const unsigned lds = (unsigned)(unsigned long long)(lds_u8*)sm.t + (unsigned)lw * 1024u;

        if (loader) {
#pragma unroll
            for (int s = 0; s < NSTG - 1; ++s) Base::issue(src, lds, s, s, full);
        }
        if (PW > 0 && !compute_wave) {
            // a producer wave's whole K loop: the barriers of the compute waves, in the same order
#pragma unroll 1
            for (int kt0 = 0; kt0 < NKT; kt0 += NSTG) {
                Base::template load_step<0>(kt0, src, lds, full, sync);
                if constexpr (NSTG > 1) Base::template load_step<1>(kt0 + 1, src, lds, full, sync);
                if constexpr (NSTG > 2) Base::template load_step<2>(kt0 + 2, src, lds, full, sync);
                if constexpr (NSTG > 3) Base::template load_step<3>(kt0 + 3, src, lds, full, sync);
            }
            sync();  // the two barriers of the epilogue
            sync();
            return;
        }

        const int wm = wave % WGM, wn = wave / WGM;
        if (wn == 0) compute<TN0>(wm, 0, lane, sm, src, lds, full, sync);
        else compute<TN1>(wm, TN0, lane, sm, src, lds, full, sync);
        sync();
        const unsigned short* ct = reinterpret_cast<const unsigned short*>(sm.t);
#pragma unroll
        for (int i = 0; i < OCHUNKS / CTHREADS; ++i) {
            const int c = tid + i * CTHREADS;
            const int row = c / (BN / 8), col = (c % (BN / 8)) * 8;
            *reinterpret_cast<u32x4*>(C + (size_t)(m0 + row) * N + n0 + col) = *reinterpret_cast<const u32x4*>(ct + row * CPITCH + col);
        }
    }
};

}  // namespace bfuse
