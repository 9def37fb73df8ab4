// fp32 GEMM side, split-K with private LDS staging:  C[M,N] = A[M,K] . B[K,N] (+ optional
// tanh-GELU).  Same arithmetic and the same decomposition as GemmF32 -- one workgroup per
// BM x BN tile, its KS waves split K and each accumulates the whole tile over its own k-range,
// partial tiles summed through LDS in wave order -- but the operands take another road:
//
//   GemmF32     global -> VGPR (global_load_dwordx4 in MFMA layout)
//   GemmF32Dma  global -> LDS  (global_load_lds_dwordx4 into a ring PRIVATE to the wave)
//                      -> VGPR (ds_read_b128 / b64 in MFMA layout)
//
// Measured on MI355X, the global->VGPR path delivers ~30 B/clk per CU and the direct-to-LDS
// path ~52 B/clk; a 32 x 144 tile over K = 768 needs 540 KB per CU, which keeps the first path
// busy enough that the single in-order wave per SIMD stalls at load issue.  Staging through
// LDS costs LDS reads instead (250 B/clk per CU available) and takes the look-ahead out of
// the register file.  Because no operand is shared between waves the ring needs NO barrier:
// a wave waits for its own loads with s_waitcnt vmcnt(n) and for its own LDS reads with
// s_waitcnt lgkmcnt(0); both are written by hand because the compiler would order every LDS
// read after every outstanding direct-to-LDS load.
//
// Stage = 8 k.  Per wave and stage the ring slot holds A[BM][8] (rows of 32 bytes) followed by
// B[8][BN].  Lane (i = lane % 16, kq = lane / 16) reads A[i][2kq], A[i][2kq+1] with one 64-bit
// read and B[2kq+t][4i .. 4i+3] (t = 0, 1) with 128-bit reads; component e of a B vector feeds
// accumulator block e of its 64-column group, so that block's column i is tile column 4i+e
// and a lane ends up with four consecutive columns of a row (128-bit stores), as in GemmF32.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_gemm_f32.h"
#include "wave.h"

namespace bfuse {

typedef float f32x2 __attribute__((ext_vector_type(2)));

//
// PW_ = 1 adds one producer wave per k-range: it issues that range's direct-to-LDS loads and the
// compute wave issues only LDS reads and MFMAs (a global load costs the issuing wave ~110 clocks
// in which it cannot issue an MFMA; a wave that only loads does not disturb an MFMA wave on the
// same SIMD).  Producer and compute waves meet at one workgroup barrier per K-stage.
template <int M_, int N_, int K_, int BM_, int BN_, int KS_, int EPI_ = kEpiNone, int NSTG_ = 3, int PW_ = 0>
struct GemmF32Dma {
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, KS = KS_, EPI = EPI_, NSTG = NSTG_;
    static constexpr int TM = BM / 16;
    static constexpr int G4 = BN / 64;          // 64-column groups
    static constexpr int G1 = (BN % 64) / 16;   // trailing 16-column groups
    static constexpr int NB = 4 * G4 + G1;      // accumulator blocks per row block
    static constexpr int KW = K / KS;           // k-range of one wave
    static constexpr int STAGE = 8;
    static constexpr int NSTAGE = KW / STAGE;
    static constexpr int A_BYTES = BM * STAGE * 4;
    static constexpr int B_BYTES = STAGE * BN * 4;
    static constexpr int A_LOADS = A_BYTES / 1024;                  // wave-level loads (64 lanes x 16 bytes)
    static constexpr int B_LOADS = (B_BYTES + 1023) / 1024;         // the last one may be partial
    static constexpr int B_CHUNKS = B_BYTES / 16;
    static constexpr int LPS = A_LOADS + B_LOADS;                   // loads per stage
    static constexpr int STAGE_BYTES = A_BYTES + B_LOADS * 1024;    // slot size (B rounded up to whole loads)
    static constexpr int WAVE_BYTES = NSTG * STAGE_BYTES;
    static_assert(M % BM == 0 && N % BN == 0 && K % (KS * STAGE) == 0, "tile must divide the problem");
    static_assert(BM % 32 == 0 && BN % 16 == 0 && N % 4 == 0 && K % 4 == 0, "shape/tile mismatch");   // A stage = whole loads
    static_assert(NSTG >= 2 && NSTAGE >= NSTG && NSTAGE % 2 == 0, "pipeline shape");
    static_assert((NSTG - 1) * LPS <= 63, "vmcnt range");
    static_assert(!(PW_ && KS_ == 1), "producer waves go with a K split");

    static constexpr Dims3 GRID{N / BN, M / BM, 1};
    static constexpr int PW = PW_;
    static constexpr int NW = KS * (1 + PW_);   // waves in the workgroup
    static constexpr Dims3 BLOCK{64 * NW, 1, 1};
    static constexpr int THREADS = 64 * NW;
    static constexpr bool HAS_BARRIERS = NW > 1;
    static constexpr int NUNIT = TM * (G4 + G1);
    static constexpr int RING_BYTES = KS * WAVE_BYTES;
    static constexpr int PART_BYTES = KS > 1 ? KS * TM * NB * 64 * 16 : 16;

    struct Smem {
        __attribute__((aligned(1024))) unsigned char t[RING_BYTES > PART_BYTES ? RING_BYTES : PART_BYTES];
    };
    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    template <int N_OUT>
    __device__ static __forceinline__ void wait_vm()
    {
        __builtin_amdgcn_s_waitcnt((N_OUT & 0xF) | ((N_OUT >> 4) << 14) | 0x0F70);
    }

    struct Frag {
        f32x2 a[TM];
        f32x4 b4[G4 > 0 ? G4 : 1][2];
        float b1[G1 > 0 ? G1 : 1][2];
    };
    struct Ctx {
        const float* a_src[A_LOADS];   // this lane's source of every A load of stage 0
        const float* b_src[B_LOADS];
        lds_u8* ring;                  // this wave's ring
        int a_rd[TM], b4_rd[G4 > 0 ? G4 : 1][2], b1_rd[G1 > 0 ? G1 : 1][2];   // LDS byte addresses in slot 0
    };

    // ---- one memory operation at a time, so that they can be dealt between the MFMAs ----------
    static constexpr int NREADS = TM + 2 * (G4 + G1);     // LDS reads per stage
    static constexpr int NOPS = LPS + 1 + NREADS;         // loads, the wait for the next stage, its reads
    static constexpr int NGROUPS = 2 * TM * (G4 + G1);    // MFMA groups per stage (4 MFMAs or 1)
    static constexpr int OPS_PER_GROUP = (NOPS + NGROUPS - 3) / (NGROUPS - 2);   // leave the last two groups free

    template <int I>
    __device__ static __forceinline__ void issue_one(const Ctx& c, int slot, int s)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        lds_u8* dst = c.ring + slot * STAGE_BYTES;
        if constexpr (I < A_LOADS) {
            __builtin_amdgcn_global_load_lds(c.a_src[I] + s * STAGE, dst + I * 1024, 16, 0, 0);
        } else {
            constexpr int J = I - A_LOADS;
            __builtin_amdgcn_global_load_lds(c.b_src[J] + (size_t)s * STAGE * N, dst + A_BYTES + J * 1024, 16, 0, 0);
        }
#endif
    }
    template <int I>
    __device__ static __forceinline__ void issue_all(const Ctx& c, int slot, int s)
    {
        if constexpr (I < LPS) {
            issue_one<I>(c, slot, s);
            issue_all<I + 1>(c, slot, s);
        }
    }
    template <int J>
    __device__ static __forceinline__ void read_one(Frag& f, const Ctx& c, int off)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (J < TM) {
            asm volatile("ds_read_b64 %0, %1" : "=v"(f.a[J]) : "v"(c.a_rd[J] + off));
        } else if constexpr (J < TM + 2 * G4) {
            constexpr int g = (J - TM) / 2, t = (J - TM) % 2;
            asm volatile("ds_read_b128 %0, %1" : "=v"(f.b4[g][t]) : "v"(c.b4_rd[g][t] + off));
        } else {
            constexpr int g = (J - TM - 2 * G4) / 2, t = (J - TM - 2 * G4) % 2;
            asm volatile("ds_read_b32 %0, %1" : "=v"(f.b1[g][t]) : "v"(c.b1_rd[g][t] + off));
        }
#endif
    }
    __device__ static __forceinline__ void read_stage(Frag& f, const Ctx& c, int off)
    {
        read_all<0>(f, c, off);
    }
    template <int J>
    __device__ static __forceinline__ void read_all(Frag& f, const Ctx& c, int off)
    {
        if constexpr (J < NREADS) {
            read_one<J>(f, c, off);
            read_all<J + 1>(f, c, off);
        }
    }
    // all LDS reads of this wave have landed; every fragment register is named so that the
    // compiler neither moves its uses above the wait nor reuses it while the read is in flight
    __device__ static __forceinline__ void wait_reads(Frag& f)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) asm volatile("" : "+v"(f.a[tm]));
#pragma unroll
        for (int g = 0; g < G4; ++g)
#pragma unroll
            for (int t = 0; t < 2; ++t) asm volatile("" : "+v"(f.b4[g][t]));
#pragma unroll
        for (int g = 0; g < G1; ++g)
#pragma unroll
            for (int t = 0; t < 2; ++t) asm volatile("" : "+v"(f.b1[g][t]));
#endif
    }

    // memory operation OP of step s: first the refill of the slot stage s came from (its
    // reads were waited for at the end of the previous step), then the wait that certifies
    // stage s+1 (stages up to s+NSTG-1 were issued before this step, the refill adds s+NSTG),
    // then the reads of stage s+1
    // REFILL: stage s+NSTG exists; NEXT: stage s+1 exists.  Compile-time, so that a step's body
    // has no branch in it.
    template <int OP, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void mem_op(int s, int slot, int next_off, Frag& nxt, const Ctx& c)
    {
        if constexpr (OP < LPS) {
            if constexpr (REFILL && !PW) issue_one<OP>(c, slot, s + NSTG);
        } else if constexpr (OP == LPS) {
            if constexpr (NEXT && !PW) {
                if constexpr (REFILL) wait_vm<(NSTG - 1) * LPS>();
                else wait_vm<0>();
            }
        } else if constexpr (OP < NOPS) {
            if constexpr (NEXT) read_one<OP - LPS - 1>(nxt, c, next_off);
        }
    }
    template <int G, int K0, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void mem_ops(int s, int slot, int next_off, Frag& nxt, const Ctx& c)
    {
        if constexpr (K0 < OPS_PER_GROUP) {
            mem_op<G * OPS_PER_GROUP + K0, REFILL, NEXT>(s, slot, next_off, nxt, c);
            mem_ops<G, K0 + 1, REFILL, NEXT>(s, slot, next_off, nxt, c);
        }
    }

    // MFMA group G of a stage, then its share of the memory operations
    template <int G, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void groups(int s, int slot, int next_off, f32x4 (&acc)[TM][NB], const Frag& cur, Frag& nxt, const Ctx& c)
    {
        if constexpr (G < NGROUPS) {
            constexpr int t = G / (TM * (G4 + G1)), tm = (G / (G4 + G1)) % TM, g = G % (G4 + G1);
            if constexpr (g < G4) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[tm][4 * g + e] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.a[tm][t], cur.b4[g][t][e], acc[tm][4 * g + e], 0, 0, 0);
            } else {
                acc[tm][4 * G4 + g - G4] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.a[tm][t], cur.b1[g - G4][t], acc[tm][4 * G4 + g - G4], 0, 0, 0);
            }
            mem_ops<G, 0, REFILL, NEXT>(s, slot, next_off, nxt, c);
            __builtin_amdgcn_sched_barrier(0);
            groups<G + 1, REFILL, NEXT>(s, slot, next_off, acc, cur, nxt, c);
        }
    }

    // one K-stage: fragments of stage s are in `cur`; refill its slot with stage s+NSTG, read
    // stage s+1 into `nxt`, multiply -- the memory operations dealt between the MFMA groups
    template <class Sync>
    __device__ static __forceinline__ void step(int s, int& slot, f32x4 (&acc)[TM][NB], Frag& cur, Frag& nxt, const Ctx& c, Sync& sync)
    {
        int next_slot = slot + 1;
        if (next_slot == NSTG) next_slot = 0;
        const int next_off = next_slot * STAGE_BYTES;
        // barrier of stage s (producer mode): stage s+1 is in LDS (the producers waited for it)
        // and every compute wave holds stage s in registers, so its slot can be refilled
        if constexpr (PW) sync.raw();
        if (s + NSTG < NSTAGE) groups<0, true, true>(s, slot, next_off, acc, cur, nxt, c);
        else if (s + 1 < NSTAGE) groups<0, false, true>(s, slot, next_off, acc, cur, nxt, c);
        else groups<0, false, false>(s, slot, next_off, acc, cur, nxt, c);
        wait_reads(nxt);
        slot = next_slot;
    }

    __device__ static __forceinline__ float epilogue(float v)
    {
        if constexpr (EPI == kEpiGeluTanh) return gelu_tanh(v);
        return v;
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
        const int li = lane & 15, kq = lane >> 4;
        const bool producer = PW && wave >= KS;
        const int part = wave < KS ? wave : wave - KS;        // k-range this wave computes or loads
        const int kbeg = part * KW;

        Ctx c;
        c.ring = (lds_u8*)sm.t + part * WAVE_BYTES;
        // A slot: [BM][8] floats; a wave-level load covers 32 rows (two lanes per 32-byte row)
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            c.a_src[i] = A + (size_t)(m0 + i * 32 + (lane >> 1)) * K + kbeg + (lane & 1) * 4;
        // B slot: [8][BN] floats, 16-byte chunk ch = (row, ch % (BN/4))
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            // lanes past the end of a partial last load fetch the last chunk again; it lands in
            // the slot's padding (the slot reserves whole loads)
            int ch = i * 64 + lane;
            if (ch >= B_CHUNKS) ch = B_CHUNKS - 1;
            c.b_src[i] = B + (size_t)(kbeg + ch / (BN / 4)) * N + n0 + (ch % (BN / 4)) * 4;
        }
        const int base = (int)(unsigned)(unsigned long long)c.ring;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) c.a_rd[tm] = base + (tm * 16 + li) * 32 + kq * 8;
#pragma unroll
        for (int g = 0; g < G4; ++g)
#pragma unroll
            for (int t = 0; t < 2; ++t) c.b4_rd[g][t] = base + A_BYTES + ((2 * kq + t) * BN + g * 64 + 4 * li) * 4;
#pragma unroll
        for (int g = 0; g < G1; ++g)
#pragma unroll
            for (int t = 0; t < 2; ++t) c.b1_rd[g][t] = base + A_BYTES + ((2 * kq + t) * BN + G4 * 64 + g * 16 + li) * 4;

        f32x4 acc[TM][NB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[tm][b] = f32x4{0.f, 0.f, 0.f, 0.f};

        // stages 0 .. NSTG-1 go out; stage 0's fragments are read before the loop
        if (producer) {
            // the producer's whole K loop: same barriers as the compute waves, in the same order
#pragma unroll
            for (int s = 0; s < NSTG; ++s) issue_all<0>(c, s, s);
            wait_vm<(NSTG - 1) * LPS>();
            sync.raw();   // stage 0 is in LDS
            int slot = 0;
#pragma unroll 1
            for (int s = 0; s < NSTAGE; ++s) {
                if (s + 1 < NSTAGE) {
                    if (s + NSTG - 1 < NSTAGE) wait_vm<(NSTG - 2) * LPS>();
                    else wait_vm<0>();
                }
                sync.raw();
                if (s + NSTG < NSTAGE) issue_all<0>(c, slot, s + NSTG);
                slot = slot + 1 == NSTG ? 0 : slot + 1;
            }
        } else {
            Frag f0, f1;
            if constexpr (!PW) {
#pragma unroll
                for (int s = 0; s < NSTG; ++s) issue_all<0>(c, s, s);
                wait_vm<(NSTG - 1) * LPS>();
            } else {
                sync.raw();   // stage 0 is in LDS
            }
            read_stage(f0, c, 0);
            wait_reads(f0);
            int slot = 0;
#pragma unroll 1
            for (int s = 0; s < NSTAGE; s += 2) {
                step(s, slot, acc, f0, f1, c, sync);
                step(s + 1, slot, acc, f1, f0, c, sync);
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
                for (int g = 0; g < G1; ++g) store_group1(C, m0, n0, tm, g, acc[tm][4 * G4 + g], lane);
            }
        } else {
            // the rings are dead (every wave has consumed its last stage before it gets here, and
            // the barrier below orders the other waves' ring reads before this wave's writes)
            sync();
            f32x4(*part)[TM * NB][64] = reinterpret_cast<f32x4(*)[TM * NB][64]>(sm.t);
            if (!producer) {
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int b = 0; b < NB; ++b) part[wave][tm * NB + b][lane] = acc[tm][b];
            }
            sync();
            // every wave of the workgroup, producers included, finishes units
#pragma unroll
            for (int u0 = 0; u0 < NUNIT; u0 += NW) {
                const int u = u0 + wave;
                if (u < NUNIT) {
                    const int tm = u / (G4 + G1), g = u % (G4 + G1);
                    if (g < G4) {
                        f32x4 blk[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            f32x4 s = part[0][tm * NB + 4 * g + e][lane];
#pragma unroll
                            for (int w = 1; w < KS; ++w) s += part[w][tm * NB + 4 * g + e][lane];
                            blk[e] = s;
                        }
                        store_group4(C, m0, n0, tm, g, blk, lane);
                    } else {
                        f32x4 s = part[0][tm * NB + 4 * G4 + (g - G4)][lane];
#pragma unroll
                        for (int w = 1; w < KS; ++w) s += part[w][tm * NB + 4 * G4 + (g - G4)][lane];
                        store_group1(C, m0, n0, tm, g - G4, s, lane);
                    }
                }
            }
        }
    }

    __device__ static __forceinline__ void store_group4(float* __restrict__ C, int m0, int n0, int tm, int g, const f32x4 (&blk)[4], int lane)
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
    __device__ static __forceinline__ void store_group1(float* __restrict__ C, int m0, int n0, int tm, int g, const f32x4& blk, int lane)
    {
        const int j = lane & 15, rg = lane >> 4;
#pragma unroll
        for (int v = 0; v < 4; ++v)
            C[(size_t)(m0 + tm * 16 + 4 * rg + v) * N + n0 + G4 * 64 + g * 16 + j] = epilogue(blk[v]);
    }
};

}  // namespace bfuse
