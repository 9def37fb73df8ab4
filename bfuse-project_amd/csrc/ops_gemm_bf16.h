// bf16 GEMM side with fp32 accumulation on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16):  C[M,N] = A[M,K] . W[N,K]^T, bf16 in, bf16 out (one rounding,
// to nearest even, of the fp32 accumulator).
//
// W is stored [N,K] -- the reference's `dense` weight layout (out,in)
// (scripts/configure_kernels.py:21-26,50-58) -- so both operands are contiguous along K,
// which is what the bf16 MFMA wants: every lane supplies eight consecutive k of one row.
//
// One workgroup owns a BM x BN tile and walks K in steps of 64; the epilogue rounds to bf16,
// transposes the tile through LDS and writes 128-bit row segments.
//
// Workgroup ids map to tiles so that the BM-tiles sharing one slab of W run on the same XCD
// at the same time (consecutive workgroup ids go to consecutive XCDs): the slab is fetched
// from HBM once and hit in that XCD's L2 by the other M-tiles.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// The K-pipeline is built around direct global->LDS loads
// (global_load_lds_dwordx4): no staging registers, NSTG LDS stages in a ring, NSTG-1
// K-steps of loads in flight while one is multiplied.  A wave-level load writes 64 lanes x
// 16 bytes contiguously (8 rows of 128 bytes), so rows cannot be padded; instead the
// 16-byte chunk c of row r is stored at chunk position c ^ ((r >> 1) & 7), which makes the
// 128-bit operand reads of 16 consecutive rows hit 16 different bank groups.
//
// Waves: WGM_ x WGN_ of them tile the workgroup's BM x BN block.  One wave per SIMD (2 x 2)
// cannot keep the matrix core busy with 16x16x32 MFMAs: measured on MI355X, a lone wave
// issues one every ~28 clocks where the pipe takes 16, and two waves per SIMD reach ~18.
// The 4 x 2 layout (eight waves of 32 x BN/2) therefore trades 40 % more LDS operand reads
// (still under 60 % of the ~250 B/clk the LDS delivers to eight waves) for a 1.5x higher
// MFMA issue ceiling.
//
// Producer waves (PW_ > 0): measured on MI355X, a load issued between two MFMAs of the same wave
// takes 8-14 clocks out of its MFMA stream when its base is in scalar registers (30-40 with the
// 64-bit vector address arithmetic the compiler emits), an LDS read ~12; the same loads issued by
// another wave of the SIMD cost the MFMA wave nothing.  With PW_ extra waves the direct-to-LDS
// loads are issued by them and the WGM_ x WGN_ compute waves issue only LDS reads and MFMAs.  All
// waves take part in every barrier.
// EARLY_ > 0 (with producer waves): the barrier that certifies K-step kt+1 is taken inside step kt,
// before MFMA group EARLY_ of its STEPS groups, and the first operand fragments of step kt+1 are
// requested right after it, so that they arrive while the last groups of step kt multiply.  With the
// barrier at the top of the step every wave of the workgroup waits for its first LDS reads at the
// same moment and the matrix cores idle for that long once per step.  The fragments of two
// consecutive steps live in two register sets, so the rolled loop holds 2 * NSTG_ steps.  Measured
// on MI355X on the 512 x 4096 x 14336 instance, both forms in one run: 46.8 against 48.2 us, and
// 47.8 against 49.4-49.8 us with the norm waves fused in.
// CLK_ (instrumentation, off in every product kernel): wave 0 of each workgroup reads the shader-clock
// counter and the 100 MHz wall clock before its K loop, after it, and when its last store has been
// acknowledged, and writes them with the XCD it ran on behind the output matrix (STAMP_WORDS 64-bit words per
// workgroup at byte offset M * N * 2 of O; the kernel is then registered with an output that much larger).
// The counters are scalar memory reads; each is waited for at once, so none is in flight when the
// hand-counted LDS waits of the loop run.
template <int M_, int N_, int K_, int BM_, int BN_, int NSTG_ = 3, int PD_ = 4, int WGM_ = 2, int WGN_ = 2, int PW_ = 0, int EARLY_ = 0,
          bool CLK_ = false>
struct GemmBf16NTDma {
    static constexpr bool MATRIX_CORES = true;   // the inner loop is a stream of MFMAs (what the fusion chooser asks)
    static constexpr bool CLK = CLK_;
    static constexpr int STAMP_WORDS = 8;   // clock x 3, wall x 3, XCC_ID, HW_ID
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, NSTG = NSTG_;
    static constexpr int BK = 64;
    static constexpr int WGM = WGM_, WGN = WGN_, NCOMP = WGM_ * WGN_, PW = PW_;
    static constexpr int NWAVES = PW_ > 0 ? PW_ : NCOMP;   // waves that issue the global loads
    static constexpr int THREADS = 64 * (NCOMP + PW_);
    static constexpr int CTHREADS = 64 * NCOMP;           // compute threads (they also store the tile)
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 16, TN = WN / 16;
    static constexpr int NKT = K / BK;
    static constexpr int ROWS = BM + BN;
    static constexpr int GROUPS = ROWS / 8;             // wave-level loads per stage
    static constexpr int GPW = (GROUPS + NWAVES - 1) / NWAVES;   // per wave: waves < GEXTRA issue GPW, the others GPW - 1
    static constexpr int GEXTRA = GROUPS % NWAVES == 0 ? NWAVES : GROUPS % NWAVES;
    static constexpr int STAGE_BYTES = ROWS * 128;
    static constexpr int CPITCH = BN + 8;
    static constexpr int OCHUNKS = BM * (BN / 8);
    static_assert(M % BM == 0 && N % BN == 0 && K % BK == 0, "tile must divide the problem");
    static_assert(BM % WGM == 0 && BN % WGN == 0 && WM % 16 == 0 && WN % 16 == 0 && BM % 8 == 0 && BN % 8 == 0, "tile shape");
    static_assert(TM == 2 || TM == 4, "the hand-written LDS wait lists two or four A fragments");
    static_assert(OCHUNKS % CTHREADS == 0 && NSTG >= 2 && NSTG <= 4 && NKT >= NSTG - 1, "pipeline shape");
    static_assert(PD_ >= 1 && PD_ < (BK / 32) * (BN / WGN_ / 16), "read-ahead distance");
    // the hand-written wait counts (allowed()) count the next substep's A fragments, requested after group
    // ks*TN+1, as reads that may still be in flight for the PD groups that follow: the substep must be
    // longer than that, or its successor's first group would use them unwaited (the build's check of the
    // assembly finds such MFMAs: seen with TN = 2 and with TN = PD = 4)
    static_assert(BN / WGN_ / 16 > PD_ + 1, "column blocks per wave must exceed the read-ahead distance + 1");
    static constexpr int MT = M / BM, NT = N / BN;
    static_assert((MT * NT) % 8 == 0 && NT % 8 == 0, "tiles are dealt to 8 XCDs");

    static constexpr Dims3 GRID{MT * NT, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    static constexpr bool LOOP_BARRIERS = true;   // one workgroup barrier per K-stage, not only in the epilogue
    static constexpr int MIN_BARRIERS = K_ / 64 + 2;   // what every wave executes: one per K-step, two in the epilogue
    static constexpr int EPI_BYTES = BM * CPITCH * 2;
    struct Smem {
        __attribute__((aligned(1024))) unsigned char t[((NSTG * STAGE_BYTES > EPI_BYTES) ? NSTG * STAGE_BYTES : EPI_BYTES)];
    };

    // s_waitcnt vmcnt(n), other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
    template <int N_OUT>
    __device__ static __forceinline__ void wait_vm()
    {
        __builtin_amdgcn_s_waitcnt((N_OUT & 0xF) | ((N_OUT >> 4) << 14) | 0x0F70);
    }

    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    // this wave's wave-level loads of K-step kt into LDS stage `stage`: group wave + i * NWAVES
    // (8 rows each); `full` says whether this wave owns a group in the last, partial round
    // Addresses are a wave-uniform base (scalar registers, advanced per K-step by scalar adds) plus a
    // per-lane 32-bit offset that never changes: a 64-bit vector add per load would cost the SIMD's
    // MFMA stream ~20 clocks each, whichever wave issues it.
    struct Src {
        const char* a_ub;      // A + m0 * K           (bytes)
        const char* w_ub;      // W + n0 * K
        unsigned voff[GPW];    // (row within its operand) * K * 2 + swizzled chunk * 16
        int lw;                // index among the loading waves
    };
    __device__ static __forceinline__ void issue(const Src& src, unsigned wave_base, int stage, int kt, bool full)
    {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int i = 0; i < GPW; ++i)
            if (i + 1 < GPW || full) {
                const bool is_a = 8 * (src.lw + i * NWAVES) < BM;   // wave-uniform: a group of 8 rows is all A or all W
                const char* ub = (is_a ? src.a_ub : src.w_ub) + (size_t)kt * (BK * 2);
                dma_load_lds_b128(src.voff[i], ub, wave_base + stage * STAGE_BYTES + i * NWAVES * 1024);
            }
#endif
    }
    // "the loads of the K-step that is due have landed": at most `newer` K-steps' loads outstanding
    template <int NEWER>
    __device__ static __forceinline__ void wait_stage(bool full)
    {
        if constexpr (GEXTRA == NWAVES) {
            wait_vm<GPW * NEWER>();
        } else {
            if (full) wait_vm<GPW * NEWER>();
            else wait_vm<(GPW - 1) * NEWER>();
        }
    }

    // ---- operand reads are issued and waited for by hand ------------------------------------
    // The compiler waits for ALL outstanding LDS reads (lgkmcnt(0)) before the first MFMA
    // that needs one of them, which throws away the read-ahead; written as asm it cannot see
    // them, and each MFMA group waits only for the fragments it uses (LDS reads of a wave
    // return in order, so "at most n outstanding" identifies which have landed).
    // Operand addresses: one base register per (32-k substep, operand) and stage pair; the 16-row
    // block and the stage are immediate offsets (+16 rows = +2048 bytes leaves the swizzle key alone)
    struct Addr {
        int a[BK / 32][(NSTG + 1) / 2], b[BK / 32][(NSTG + 1) / 2];   // [..][h]: base of stage 2h
    };
    static_assert(STAGE_BYTES + ((TM > TN ? TM : TN) - 1) * 2048 + 2048 <= 65536, "stage + block offsets are 16-bit immediates");
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
    template <int U, int KS, int BLK>
    __device__ static __forceinline__ bf16x8 read_a(const Addr& ad) { return lds_read<(U % 2) * STAGE_BYTES + BLK * 2048>(ad.a[KS][U / 2]); }
    template <int U, int KS, int BLK>
    __device__ static __forceinline__ bf16x8 read_b(const Addr& ad) { return lds_read<(U % 2) * STAGE_BYTES + BLK * 2048>(ad.b[KS][U / 2]); }
    template <int N_OUT>
    __device__ static __forceinline__ void wait_lds(bf16x8& b, bf16x8 (&a)[TM])
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (TM == 4) {
            asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(b), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]) : "n"(N_OUT));
        } else {
            asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(b), "+v"(a[0]), "+v"(a[1]) : "n"(N_OUT));
        }
#endif
    }

    static constexpr int STEPS = BK / 32 * TN;
    static constexpr int PD = PD_;      // B fragments are read PD MFMA groups ahead
    static constexpr int RING = PD + 1;
    // reads still allowed in flight when MFMA group `st` starts: the B fragments ahead of it,
    // and the next K-substep's A fragments (issued after group ks*TN+1) if they came after B[st]
    static constexpr int allowed(int st)
    {
        int n = (STEPS - 1 - st) < (PD - 1) ? (STEPS - 1 - st) : (PD - 1);
        for (int ks = 0; ks + 1 < BK / 32; ++ks) {
            const int s_af = ks * TN + 1;
            const int lo = st - PD > 0 ? st - PD : 0;
            if (s_af >= lo && s_af <= st - 1) n += TM;
        }
        return n;
    }

    template <int U, int KS, int A>
    __device__ static __forceinline__ void read_a_all(bf16x8 (&af)[TM], const Addr& ad)
    {
        if constexpr (A < TM) {
            af[A] = read_a<U, KS, A>(ad);
            read_a_all<U, KS, A + 1>(af, ad);
        }
    }
    template <int U, int P>
    __device__ static __forceinline__ void read_b_first(bf16x8 (&bq)[RING], const Addr& ad)
    {
        if constexpr (P < PD) {
            bq[P] = read_b<U, P / TN, P % TN>(ad);
            read_b_first<U, P + 1>(bq, ad);
        }
    }
    template <int U, int ST>
    __device__ static __forceinline__ void step_chain(f32x4 (&acc)[TM][TN], bf16x8 (&af)[BK / 32][TM], bf16x8 (&bq)[RING], const Addr& ad)
    {
        if constexpr (ST < STEPS) {
            constexpr int ks = ST / TN, b = ST % TN;
            wait_lds<allowed(ST)>(bq[ST % RING], af[ks]);
#pragma unroll
            for (int a = 0; a < TM; ++a)
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bq[ST % RING], af[ks][a], acc[a][b], 0, 0, 0);
            if constexpr (ST + PD < STEPS) bq[(ST + PD) % RING] = read_b<U, (ST + PD) / TN, (ST + PD) % TN>(ad);
            if constexpr (b == 1 && ks + 1 < BK / 32) {
                read_a_all<U, ks + 1, 0>(af[ks + 1], ad);
            }
            __builtin_amdgcn_sched_barrier(0);
            step_chain<U, ST + 1>(acc, af, bq, ad);
        }
    }

    // ---- the same chain with the next step's barrier and first reads inside it (EARLY_) -----------
    static constexpr int EARLY = EARLY_;
    static_assert(EARLY_ == 0 || (PW_ > 0 && BK / 32 == 2 && EARLY_ >= STEPS - PD_ && EARLY_ > 1 && EARLY_ < STEPS),
                  "the early barrier needs producer waves and comes after the step's last read has been issued");
    struct Frags {
        bf16x8 af[BK / 32][TM], bq[RING];
    };
    // every read of the step has been issued: wait for all of them; the fragments still to be used are named
    __device__ static __forceinline__ void wait_rest(Frags& f)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        // (an operand named twice would make the compiler copy it -- a register with a read in flight)
        static_assert(TM == 2 || TM == 4, "the wait names two or four A fragments");
        constexpr int G = EARLY_ > 0 ? EARLY_ : STEPS - 1, REST = STEPS - G;
        static_assert(REST >= 1 && REST <= 4, "the wait names at most four B fragments");
        bf16x8(&a)[TM] = f.af[1];
        bf16x8& a2 = a[TM == 4 ? 2 : 0];   // only named when TM == 4
        bf16x8& a3 = a[TM == 4 ? 3 : 1];
        bf16x8& b0 = f.bq[G % RING];
        bf16x8& b1 = f.bq[(G + 1) % RING];
        bf16x8& b2 = f.bq[(G + 2) % RING];
        bf16x8& b3 = f.bq[(G + 3) % RING];
#define BFUSE_WAIT_REST(...)                                                                                            \
    do {                                                                                                                \
        if constexpr (TM == 4) asm volatile("s_waitcnt lgkmcnt(0)" : __VA_ARGS__, "+v"(a[0]), "+v"(a[1]), "+v"(a2), "+v"(a3)); \
        else asm volatile("s_waitcnt lgkmcnt(0)" : __VA_ARGS__, "+v"(a[0]), "+v"(a[1]));                               \
    } while (0)
        if constexpr (REST == 1) BFUSE_WAIT_REST("+v"(b0));
        else if constexpr (REST == 2) BFUSE_WAIT_REST("+v"(b0), "+v"(b1));
        else if constexpr (REST == 3) BFUSE_WAIT_REST("+v"(b0), "+v"(b1), "+v"(b2));
        else BFUSE_WAIT_REST("+v"(b0), "+v"(b1), "+v"(b2), "+v"(b3));
#undef BFUSE_WAIT_REST
#endif
    }
    // LAST: this is the final K-step, there is no next step to meet for
    template <int U, int ST, bool LAST, class Sync>
    __device__ static __forceinline__ void early_chain(f32x4 (&acc)[TM][TN], Frags& cur, Frags& nxt, const Addr& ad, Sync& sync)
    {
        if constexpr (ST < STEPS) {
            constexpr int ks = ST / TN, b = ST % TN;
            if constexpr (ST < EARLY_) {
                wait_lds<allowed(ST)>(cur.bq[ST % RING], cur.af[ks]);
            } else if constexpr (ST == EARLY_) {
                wait_rest(cur);
                if constexpr (!LAST) {
                    // K-step kt+1 is in LDS (the producers waited for it) and every wave has read all of
                    // step kt: its slot may be refilled, and step kt+1's first fragments are requested now
                    sync.bare();
                    read_a_all<(U + 1) % NSTG, 0, 0>(nxt.af[0], ad);
                    read_b_first<(U + 1) % NSTG, 0>(nxt.bq, ad);
                }
            }
#pragma unroll
            for (int a = 0; a < TM; ++a)
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.bq[ST % RING], cur.af[ks][a], acc[a][b], 0, 0, 0);
            if constexpr (ST + PD < STEPS) cur.bq[(ST + PD) % RING] = read_b<U, (ST + PD) / TN, (ST + PD) % TN>(ad);
            if constexpr (b == 1 && ks + 1 < BK / 32) {
                read_a_all<U, ks + 1, 0>(cur.af[ks + 1], ad);
            }
            __builtin_amdgcn_sched_barrier(0);
            early_chain<U, ST + 1, LAST>(acc, cur, nxt, ad, sync);
        }
    }
    // K-step S (compile-time position in a group of 2 * NSTG steps): ring slot S % NSTG, fragment set S % 2
    template <int S, bool LAST, class Sync>
    __device__ static __forceinline__ void early_step(f32x4 (&acc)[TM][TN], Frags (&fr)[2], const Addr& ad, Sync& sync)
    {
        early_chain<S % NSTG, 0, LAST>(acc, fr[S % 2], fr[(S + 1) % 2], ad, sync);
    }
    static constexpr int UNR = 2 * NSTG_;                                      // slots and fragment sets are back where they started
    static constexpr int MAIN_STEPS = NKT > 1 ? ((NKT - 1) / UNR) * UNR : 0;   // in the rolled loop; the last step is never in it
    template <int J, class Sync>
    __device__ static __forceinline__ void early_main(f32x4 (&acc)[TM][TN], Frags (&fr)[2], const Addr& ad, Sync& sync)
    {
        if constexpr (J < UNR) {
            early_step<J, false>(acc, fr, ad, sync);
            early_main<J + 1>(acc, fr, ad, sync);
        }
    }
    template <int S, class Sync>
    __device__ static __forceinline__ void early_tail(f32x4 (&acc)[TM][TN], Frags (&fr)[2], const Addr& ad, Sync& sync)
    {
        if constexpr (S < NKT) {
            early_step<S % UNR, S == NKT - 1>(acc, fr, ad, sync);
            early_tail<S + 1>(acc, fr, ad, sync);
        }
    }

    // one K-step out of LDS stage U
    // the loading half of a K-step: wait for own loads of step kt, meet, refill the stage step kt-1 used
    template <int U, class Sync>
    __device__ static __forceinline__ void load_step(int kt, const Src& src, unsigned lds, bool full, Sync& sync)
    {
        if (kt >= NKT) return;
        // loads of K-step kt have landed once at most the newer steps' loads are outstanding
        if (kt + NSTG - 2 < NKT) wait_stage<NSTG - 2>(full);
        else wait_vm<0>();
        sync.raw();  // everyone's part of step kt is in LDS; everyone is done reading step kt-1
        if (kt + NSTG - 1 < NKT) issue(src, lds, (U + NSTG - 1) % NSTG, kt + NSTG - 1, full);
    }

    // LOADS: this wave also issues loads (no producer waves); otherwise it only meets the producers
    template <int U, bool LOADS, class Sync>
    __device__ static __forceinline__ void k_step(int kt, f32x4 (&acc)[TM][TN], const Addr& ad, const Src& src,
                                                  unsigned lds, bool full, Sync& sync)
    {
        if (kt >= NKT) return;
        if constexpr (LOADS) load_step<U>(kt, src, lds, full, sync);
        else sync.raw();
        bf16x8 af[BK / 32][TM], bq[RING];
        read_a_all<U, 0, 0>(af[0], ad);
        read_b_first<U, 0>(bq, ad);
        __builtin_amdgcn_sched_barrier(0);
        step_chain<U, 0>(acc, af, bq, ad);
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        const unsigned short* __restrict__ A = static_cast<const unsigned short*>(I);
        const unsigned short* __restrict__ Wt = static_cast<const unsigned short*>(F);
        unsigned short* __restrict__ C = static_cast<unsigned short*>(O);
        const int xcd = vblock & 7, slot = vblock >> 3;
        const int nt = xcd * (NT / 8) + slot / MT, mt = slot % MT;
        const int m0 = mt * BM, n0 = nt * BN;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: scalar branches
        const bool compute = wave < NCOMP;                   // wave-uniform roles
        const bool loader = PW == 0 || !compute;
        const int lw = PW == 0 ? wave : (compute ? 0 : wave - NCOMP);   // index among the loading waves
        const int wm = (compute ? wave : 0) / WGN, wn = (compute ? wave : 0) % WGN;
        const int li = lane & 15, kq = lane >> 4;
        const bool full = lw < GEXTRA;

        // per-lane source of each of this wave's loads (K-step 0); swizzled chunk
        Src src;
        src.a_ub = reinterpret_cast<const char*>(A + (size_t)m0 * K);
        src.w_ub = reinterpret_cast<const char*>(Wt + (size_t)n0 * K);
        src.lw = lw;
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
            int row = 8 * (lw + i * NWAVES) + (lane >> 3);
            if (row >= ROWS) row = ROWS - 1;  // slot not issued (see `full`)
            const int gc = (lane & 7) ^ ((row >> 1) & 7);
            src.voff[i] = (unsigned)((row < BM ? row : row - BM) * K + gc * 8) * 2u;
        }
        // LDS byte address of this wave's first load of stage 0 (wave-uniform)
        const unsigned lds = (unsigned)(unsigned long long)(lds_u8*)sm.t + (unsigned)lw * 1024u;

        f32x4 acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

        if (loader) {
#pragma unroll
            for (int s = 0; s < NSTG - 1; ++s) issue(src, lds, s, s, full);
        }
        if (PW > 0 && !compute) {
            // a producer wave's whole K loop: the barriers of the compute waves, in the same order
#pragma unroll 1
            for (int kt0 = 0; kt0 < NKT; kt0 += NSTG) {
                load_step<0>(kt0, src, lds, full, sync);
                if constexpr (NSTG > 1) load_step<1>(kt0 + 1, src, lds, full, sync);
                if constexpr (NSTG > 2) load_step<2>(kt0 + 2, src, lds, full, sync);
                if constexpr (NSTG > 3) load_step<3>(kt0 + 3, src, lds, full, sync);
            }
            sync();  // the two barriers of the epilogue
            sync();
            return;
        }

        // LDS byte address of this lane's fragment of block 0 in stage 2h, for each 32-k substep, with
        // the chunk swizzle folded in: loop invariant
        const unsigned lds_base = (unsigned)(unsigned long long)(lds_u8*)sm.t;
        Addr ad;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            const int c = ks * 4 + kq;
            const int arow = wm * WM + li, brow = BM + wn * WN + li;
#pragma unroll
            for (int h = 0; h < (NSTG + 1) / 2; ++h) {
                ad.a[ks][h] = (int)lds_base + 2 * h * STAGE_BYTES + arow * 128 + ((c ^ ((arow >> 1) & 7)) << 4);
                ad.b[ks][h] = (int)lds_base + 2 * h * STAGE_BYTES + brow * 128 + ((c ^ ((brow >> 1) & 7)) << 4);
            }
        }

        unsigned long long stamp_c[3] = {0, 0, 0}, stamp_w[3] = {0, 0, 0};
        if constexpr (CLK_) read_clocks(stamp_c[0], stamp_w[0]);

        // K-steps are taken NSTG at a time so that the LDS stage of each is a compile-time constant;
        // the loop stays rolled whatever K is: operand registers with reads in flight must never be
        // spilled (the compiler takes an asm output for written when the asm is issued), and a
        // fully unrolled short loop is where the register allocator runs out
        // the early barrier is built on the hardware barrier: the LDS-counter barrier a side gets when its
        // partner synchronises too has LDS traffic of its own, and its inlined polls in every unrolled step
        // cost more scalar registers than there are -- that side runs the loop with the barrier on top
        if constexpr (EARLY_ > 0 && std::is_same<Sync, BlockSync>::value) {
            Frags fr[2];
            sync.raw();   // K-step 0 is in LDS
            read_a_all<0, 0, 0>(fr[0].af[0], ad);
            read_b_first<0, 0>(fr[0].bq, ad);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
            for (int kt0 = 0; kt0 < MAIN_STEPS; kt0 += UNR) early_main<0>(acc, fr, ad, sync);
            early_tail<MAIN_STEPS>(acc, fr, ad, sync);
        } else {
#pragma unroll 1
            for (int kt0 = 0; kt0 < NKT; kt0 += NSTG) {
                k_step<0, PW == 0>(kt0, acc, ad, src, lds, full, sync);
                if constexpr (NSTG > 1) k_step<1, PW == 0>(kt0 + 1, acc, ad, src, lds, full, sync);
                if constexpr (NSTG > 2) k_step<2, PW == 0>(kt0 + 2, acc, ad, src, lds, full, sync);
                if constexpr (NSTG > 3) k_step<3, PW == 0>(kt0 + 3, acc, ad, src, lds, full, sync);
            }
        }
        if constexpr (CLK_) read_clocks(stamp_c[1], stamp_w[1]);
        sync();  // all waves are done reading the last stage before the tile buffer overwrites it

        unsigned short* ct = reinterpret_cast<unsigned short*>(sm.t);
        if (compute) {
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    // the W fragment is the MFMA's first operand: a lane holds four consecutive n of
                    // one output row (m = li), eight bytes of the tile once rounded
                    const f32x4 r = acc[a][b];
                    u32x2 packed;
                    packed[0] = pack_bf16(r[0], r[1]);
                    packed[1] = pack_bf16(r[2], r[3]);
                    *reinterpret_cast<u32x2*>(ct + (wm * WM + a * 16 + li) * CPITCH + wn * WN + b * 16 + 4 * kq) = packed;
                }
        }
        sync();
        if (compute) {
#pragma unroll
            for (int i = 0; i < OCHUNKS / CTHREADS; ++i) {
                const int c = tid + i * CTHREADS;
                const int row = c / (BN / 8), col = (c % (BN / 8)) * 8;
                *reinterpret_cast<u32x4*>(C + (size_t)(m0 + row) * N + n0 + col) =
                    *reinterpret_cast<const u32x4*>(ct + row * CPITCH + col);
            }
        }
        if constexpr (CLK_) {
            wait_vm<0>();   // this wave's stores have been acknowledged
            read_clocks(stamp_c[2], stamp_w[2]);
            if (tid == 0) {
                unsigned long long* st = reinterpret_cast<unsigned long long*>(C + (size_t)M * N) + (size_t)vblock * STAMP_WORDS;
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    st[i] = stamp_c[i];
                    st[3 + i] = stamp_w[i];
                }
                st[6] = __builtin_amdgcn_s_getreg((3 << 11) | 20);    // HW_REG_XCC_ID, bits 3:0
                st[7] = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_REG_HW_ID
            }
        }
    }

    // shader-clock counter and 100 MHz wall clock, both landed before anything else is issued
    __device__ static __forceinline__ void read_clocks(unsigned long long& c, unsigned long long& w)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        c = clock64();
        w = wall_clock64();
        asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(c), "+s"(w));
#endif
    }
};

}  // namespace bfuse
