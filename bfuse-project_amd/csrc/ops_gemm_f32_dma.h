// fp32 GEMM side, split-K with private LDS staging:  C[M,N] = A[M,K] . B[K,N] (+ optional
// tanh-GELU).  Same arithmetic and the same decomposition as GemmF32 -- one workgroup per
// BM x BN tile, its KS waves split K and each accumulates the whole tile over its own k-range,
// partial tiles summed through LDS in wave order -- but the operands take another road:
//
//   GemmF32     global -> VGPR (global_load_dwordx4 in MFMA layout)
//   GemmF32Dma  global -> LDS  (global_load_lds_dwordx4 into a ring PRIVATE to the wave)
//                      -> VGPR (ds_read_b128 / b64 in MFMA layout)
//
// What the road buys is an inner loop made of MFMAs and almost nothing else.  Measured on
// MI355X with single instructions dealt between the MFMAs of the issuing wave: one vector-ALU
// instruction costs ~20 clocks of MFMA issue, an LDS read with an immediate offset ~12, an LDS
// read whose address needs a v_add ~37, a load with the 64-bit vector address arithmetic the
// compiler emits 30-40, a direct-to-LDS load with a scalar base 8-14.  So here
//   * the ring slot, the fragment and the stage are immediate offsets on three base registers
//     (the loop is unrolled over 2 fragment buffers x NSTG slots, the tail stages peeled with
//     compile-time flags: no branch, no address arithmetic in a stage);
//   * the loads are dma_load_lds_b128 (wave.h): a wave-uniform base in scalar registers, advanced
//     by scalar adds, plus a constant per-lane offset;
//   * the memory operations are dealt one or two per MFMA group.
// A 32 x 144 tile gives 36 MFMAs : 6 loads : 8 LDS reads per 8-k stage and the loop runs at the
// pipe rate (32.6 clocks per MFMA measured inside the kernel).  Because no operand is shared
// between waves the ring needs NO barrier: a wave waits for its own loads with
// s_waitcnt vmcnt(n) and for its own LDS reads with s_waitcnt lgkmcnt(0), both by hand (the
// loads are asm, the compiler does not count them).
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

// (One producer wave per k-range issuing the loads was tried: it has to meet its compute wave at a
// workgroup barrier per K-stage, which costs about what the six loads per stage did -- no faster.)
template <int M_, int N_, int K_, int BM_, int BN_, int KS_, int EPI_ = kEpiNone, int NSTG_ = 3>
struct GemmF32Dma {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
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
    static_assert(NSTG >= 2 && NSTAGE >= NSTG, "pipeline shape");
    static_assert((NSTG - 1) * LPS <= 63, "vmcnt range");
    static_assert(NSTG * STAGE_BYTES + BN * 8 + 1024 < 65536, "fragment offsets are 16-bit immediates");

    static constexpr Dims3 GRID{N / BN, M / BM, 1};
    static constexpr int NW = KS;   // waves in the workgroup
    static constexpr Dims3 BLOCK{64 * NW, 1, 1};
    static constexpr int THREADS = 64 * NW;
    static constexpr bool HAS_BARRIERS = NW > 1;
    static constexpr int RING_BYTES = KS * WAVE_BYTES;
    // The partial tiles meet in LDS.  Component v of every f32x4 accumulator (row 4*rg + v of its
    // 16-row block) is finished by wave v / OWN: a wave writes the components that other waves own,
    // reads the other waves' values of its own components and adds them in wave order 0 .. KS-1 with
    // its register value in its own place -- the order of the sum is fixed, the work (sums, epilogue,
    // stores) is the same for every wave whatever the tile's mix of 64- and 16-column groups, and a
    // quarter (KS = 4) of the partial values never leaves its registers.  It happens in ROUNDS rounds of
    // TMR row blocks each, so that the reduction buffer is no larger than the rings it reuses: the
    // static LDS size decides whether a second workgroup (of either side of a fused kernel) fits on
    // the CU.
    static_assert(KS == 1 || KS == 2 || KS == 4, "the reduction deals the four accumulator components to the waves");
    static constexpr int OWN = 4 / KS;          // accumulator components a wave finishes
    static constexpr int FOREIGN = 4 - OWN;     // components it hands to other waves
    static constexpr int FULL_PART_BYTES = KS * TM * NB * FOREIGN * 256;
    static constexpr int ROUNDS = (KS > 1 && FULL_PART_BYTES > RING_BYTES && TM % 2 == 0) ? 2 : 1;
    static constexpr int TMR = TM / ROUNDS;
    static constexpr int PART_BYTES = KS > 1 ? KS * TMR * NB * FOREIGN * 256 : 16;

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
        // sources: a wave-uniform base (scalar registers) plus this lane's constant byte offset
        const char* a_ub;              // A + m0 * K + kbeg
        const char* b_ub;              // B + kbeg * N + n0
        unsigned a_voff[A_LOADS], b_voff[B_LOADS];
        unsigned ring;                 // LDS byte address of this wave's ring (wave-uniform)
        // LDS byte address of this lane's part of each operand in slot 0; every fragment is a
        // compile-time offset from one of them (an address computed between MFMAs costs the
        // wave ~20 clocks of MFMA issue, an immediate offset nothing)
        int a_base, b4_base, b1_base;
    };

    // ---- one memory operation at a time, so that they can be dealt between the MFMAs ----------
    static constexpr int NREADS = TM + 2 * (G4 + G1);     // LDS reads per stage
    static constexpr int NOPS = LPS + 1 + NREADS;         // loads, the wait for the next stage, its reads
    static constexpr int NGROUPS = 2 * TM * (G4 + G1);    // MFMA groups per stage (4 MFMAs or 1)
    static constexpr int OPS_PER_GROUP = (NOPS + NGROUPS - 3) / (NGROUPS - 2);   // leave the last two groups free

    template <int I>
    __device__ static __forceinline__ void issue_one(const Ctx& c, int slot, int s)
    {
        const unsigned dst = c.ring + slot * STAGE_BYTES;   // `slot` is a compile-time constant at every call
        if constexpr (I < A_LOADS) {
            dma_load_lds_b128(c.a_voff[I], c.a_ub + (size_t)s * (STAGE * 4), dst + I * 1024);
        } else {
            constexpr int J = I - A_LOADS;
            dma_load_lds_b128(c.b_voff[J], c.b_ub + (size_t)s * (STAGE * N * 4), dst + A_BYTES + J * 1024);
        }
    }
    template <int I>
    __device__ static __forceinline__ void issue_all(const Ctx& c, int slot, int s)
    {
        if constexpr (I < LPS) {
            issue_one<I>(c, slot, s);
            issue_all<I + 1>(c, slot, s);
        }
    }
    template <int J, int SLOT>
    __device__ static __forceinline__ void read_one(Frag& f, const Ctx& c)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        constexpr int S0 = SLOT * STAGE_BYTES;
        if constexpr (J < TM) {
            asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(f.a[J]) : "v"(c.a_base), "n"(S0 + J * 16 * 32));
        } else if constexpr (J < TM + 2 * G4) {
            constexpr int g = (J - TM) / 2, t = (J - TM) % 2;
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.b4[g][t]) : "v"(c.b4_base), "n"(S0 + (t * BN + g * 64) * 4));
        } else {
            constexpr int g = (J - TM - 2 * G4) / 2, t = (J - TM - 2 * G4) % 2;
            asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(f.b1[g][t]) : "v"(c.b1_base), "n"(S0 + (t * BN + G4 * 64 + g * 16) * 4));
        }
#endif
    }
    template <int SLOT, int J = 0>
    __device__ static __forceinline__ void read_stage(Frag& f, const Ctx& c)
    {
        if constexpr (J < NREADS) {
            read_one<J, SLOT>(f, c);
            read_stage<SLOT, J + 1>(f, c);
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
    template <int OP, int SLOT, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void mem_op(int s, Frag& nxt, const Ctx& c)
    {
        if constexpr (OP < LPS) {
            if constexpr (REFILL) issue_one<OP>(c, SLOT, s + NSTG);
        } else if constexpr (OP == LPS) {
            if constexpr (NEXT) {
                if constexpr (REFILL) wait_vm<(NSTG - 1) * LPS>();
                else wait_vm<0>();
            }
        } else if constexpr (OP < NOPS) {
            if constexpr (NEXT) read_one<OP - LPS - 1, (SLOT + 1) % NSTG>(nxt, c);
        }
    }
    template <int G, int K0, int SLOT, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void mem_ops(int s, Frag& nxt, const Ctx& c)
    {
        if constexpr (K0 < OPS_PER_GROUP) {
            mem_op<G * OPS_PER_GROUP + K0, SLOT, REFILL, NEXT>(s, nxt, c);
            mem_ops<G, K0 + 1, SLOT, REFILL, NEXT>(s, nxt, c);
        }
    }

    // MFMA group G of a stage, then its share of the memory operations
    template <int G, int SLOT, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void groups(int s, f32x4 (&acc)[TM][NB], const Frag& cur, Frag& nxt, const Ctx& c)
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
            mem_ops<G, 0, SLOT, REFILL, NEXT>(s, nxt, c);
            __builtin_amdgcn_sched_barrier(0);
            groups<G + 1, SLOT, REFILL, NEXT>(s, acc, cur, nxt, c);
        }
    }

    // one K-stage out of ring slot SLOT: its fragments are in `cur`; refill the slot with stage
    // s+NSTG (REFILL: that stage exists), read stage s+1 into `nxt` (NEXT), multiply -- the
    // memory operations dealt between the MFMA groups.  Slot and both flags are compile-time: the
    // body has no branch and no address arithmetic in it.
    template <int SLOT, bool REFILL, bool NEXT>
    __device__ static __forceinline__ void step(int s, f32x4 (&acc)[TM][NB], Frag& cur, Frag& nxt, const Ctx& c)
    {
        groups<0, SLOT, REFILL, NEXT>(s, acc, cur, nxt, c);
        wait_reads(nxt);
    }

    // The fragment buffers alternate (period 2) and the ring slots rotate (period NSTG): UNR stages
    // bring both back to where they started.
    static constexpr int UNR = NSTG % 2 == 0 ? NSTG : 2 * NSTG;
    static constexpr int MAIN = NSTAGE > NSTG ? ((NSTAGE - NSTG) / UNR) * UNR : 0;   // stages in the rolled loop: all refill
    template <int J>
    __device__ static __forceinline__ void main_chain(int s0, f32x4 (&acc)[TM][NB], Frag& f0, Frag& f1, const Ctx& c)
    {
        if constexpr (J < UNR) {
            if constexpr (J % 2 == 0) step<J % NSTG, true, true>(s0 + J, acc, f0, f1, c);
            else step<J % NSTG, true, true>(s0 + J, acc, f1, f0, c);
            main_chain<J + 1>(s0, acc, f0, f1, c);
        }
    }
    template <int S>
    __device__ static __forceinline__ void tail_chain(f32x4 (&acc)[TM][NB], Frag& f0, Frag& f1, const Ctx& c)
    {
        if constexpr (S < NSTAGE) {
            if constexpr (S % 2 == 0) step<S % NSTG, (S + NSTG < NSTAGE), (S + 1 < NSTAGE)>(S, acc, f0, f1, c);
            else step<S % NSTG, (S + NSTG < NSTAGE), (S + 1 < NSTAGE)>(S, acc, f1, f0, c);
            tail_chain<S + 1>(acc, f0, f1, c);
        }
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
        const Dims3 vb = XcdTiles<N / BN, M / BM, BM, BN>::tile(vblock);   // tiles dealt so that each XCD's L2 fetches as little as possible
        const int m0 = vb.y * BM, n0 = vb.x * BN;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int li = lane & 15, kq = lane >> 4;
        const int kbeg = wave * KW;        // k-range this wave accumulates

        Ctx c;
        c.ring = (unsigned)(unsigned long long)(lds_u8*)sm.t + (unsigned)wave * WAVE_BYTES;
        c.a_ub = reinterpret_cast<const char*>(A + (size_t)m0 * K + kbeg);
        c.b_ub = reinterpret_cast<const char*>(B + (size_t)kbeg * N + n0);
        // A slot: [BM][8] floats; a wave-level load covers 32 rows (two lanes per 32-byte row)
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            c.a_voff[i] = (unsigned)((i * 32 + (lane >> 1)) * K + (lane & 1) * 4) * 4u;
        // B slot: [8][BN] floats, 16-byte chunk ch = (row, ch % (BN/4))
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            // lanes past the end of a partial last load fetch the last chunk again; it lands in
            // the slot's padding (the slot reserves whole loads)
            int ch = i * 64 + lane;
            if (ch >= B_CHUNKS) ch = B_CHUNKS - 1;
            c.b_voff[i] = (unsigned)((ch / (BN / 4)) * N + (ch % (BN / 4)) * 4) * 4u;
        }
        const int base = (int)c.ring;
        c.a_base = base + li * 32 + kq * 8;
        c.b4_base = base + A_BYTES + (2 * kq * BN + 4 * li) * 4;
        c.b1_base = base + A_BYTES + (2 * kq * BN + li) * 4;

        f32x4 acc[TM][NB];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[tm][b] = f32x4{0.f, 0.f, 0.f, 0.f};

        // stages 0 .. NSTG-1 go out; stage 0's fragments are read before the loop
        {
            Frag f0, f1;
#pragma unroll
            for (int s = 0; s < NSTG; ++s) issue_all<0>(c, s, s);
            wait_vm<(NSTG - 1) * LPS>();
            read_stage<0>(f0, c);
            wait_reads(f0);
#pragma unroll 1
            for (int s0 = 0; s0 < MAIN; s0 += UNR) main_chain<0>(s0, acc, f0, f1, c);
            tail_chain<MAIN>(acc, f0, f1, c);
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
            float* part = reinterpret_cast<float*>(sm.t) + lane;
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r) {
                sync();   // first pass: the rings are dead; later passes: the previous sums have been read
                if (wave == 0) hand_over<0>(acc, r, part);
                else if (wave == 1) hand_over<1>(acc, r, part);
                else if (wave == 2) hand_over<(KS > 2 ? 2 : 0)>(acc, r, part);
                else hand_over<(KS > 2 ? 3 : 0)>(acc, r, part);
                sync();
                if (wave == 0) finish<0>(acc, r, part, C, m0, n0, lane);
                else if (wave == 1) finish<1>(acc, r, part, C, m0, n0, lane);
                else if (wave == 2) finish<(KS > 2 ? 2 : 0)>(acc, r, part, C, m0, n0, lane);
                else finish<(KS > 2 ? 3 : 0)>(acc, r, part, C, m0, n0, lane);
            }
        }
    }

    // word index (before the lane) of component V of block `blk` in the area wave X writes
    template <int X, int V>
    static constexpr int part_index(int blk)
    {
        static_assert(V / OWN != X, "a wave keeps its own components in registers");
        return ((X * (TMR * NB) + blk) * FOREIGN + (V < X * OWN ? V : V - OWN)) * 64;
    }
    template <int W, int V>
    __device__ static __forceinline__ void hand_over_one(const f32x4 (&acc)[TM][NB], int r, float* part)
    {
        if constexpr (V < 4) {
            if constexpr (V / OWN != W) {
#pragma unroll
                for (int tm = 0; tm < TMR; ++tm)
#pragma unroll
                    for (int b = 0; b < NB; ++b) part[part_index<W, V>(tm * NB + b)] = acc[r * TMR + tm][b][V];
            }
            hand_over_one<W, V + 1>(acc, r, part);
        }
    }
    template <int W>
    __device__ static __forceinline__ void hand_over(const f32x4 (&acc)[TM][NB], int r, float* part)
    {
        hand_over_one<W, 0>(acc, r, part);
    }
    // sum over the waves in wave order, wave W's own value taken from its register
    template <int W, int V>
    __device__ static __forceinline__ float total(float own, const float* part, int blk)
    {
        float s;
        if constexpr (W == 0) s = own;
        else s = part[part_index<0, V>(blk)];
        return total_rest<W, V, 1>(s, own, part, blk);
    }
    template <int W, int V, int X>
    __device__ static __forceinline__ float total_rest(float s, float own, const float* part, int blk)
    {
        if constexpr (X < KS) {
            if constexpr (X == W) s += own;
            else s += part[part_index<X, V>(blk)];
            return total_rest<W, V, X + 1>(s, own, part, blk);
        } else {
            return s;
        }
    }
    template <int W, int T = 0>
    __device__ static __forceinline__ void finish(const f32x4 (&acc)[TM][NB], int r, const float* part, float* __restrict__ C,
                                                  int m0, int n0, int lane)
    {
        if constexpr (T < OWN) {
            constexpr int V = W * OWN + T;
            const int j = lane & 15, rg = lane >> 4;
#pragma unroll
            for (int tm = 0; tm < TMR; ++tm) {
                float* __restrict__ row = C + (size_t)(m0 + (r * TMR + tm) * 16 + 4 * rg + V) * N + n0;
#pragma unroll
                for (int g = 0; g < G4; ++g) {
                    f32x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o[e] = epilogue(total<W, V>(acc[r * TMR + tm][4 * g + e][V], part, tm * NB + 4 * g + e));
                    *reinterpret_cast<f32x4*>(row + g * 64 + 4 * j) = o;
                }
#pragma unroll
                for (int g = 0; g < G1; ++g)
                    row[G4 * 64 + g * 16 + j] = epilogue(total<W, V>(acc[r * TMR + tm][4 * G4 + g][V], part, tm * NB + 4 * G4 + g));
            }
            finish<W, T + 1>(acc, r, part, C, m0, n0, lane);
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
