// bf16 GEMM side, continuous-stream variant:  C[M,N] = A[M,K] . W[N,K]^T  (bf16 in, fp32
// accumulate on v_mfma_f32_16x16x32_bf16, bf16 out) -- same arithmetic, operand layouts and
// tile->XCD mapping as GemmBf16NTDma; what changes is how the K loop is fed.
//
// What the measurements on MI355X said about the one-barrier-per-64-k kernel:
//   * a lone wave per SIMD issues a 16x16x32 MFMA every ~28 clocks where the pipe needs 16;
//     two waves per SIMD reach ~18.  Hence eight waves (4 x 2, each 32 x BN/2) per workgroup.
//   * global->LDS loads (global_load_lds_dwordx4) run at ~52 B/clk per CU from L2 and the
//     chip streams ~6.3 TB/s from HBM, so feeding a 128 x 224 tile over K = 4096 takes ~23 us
//     of L1 time per CU; it only overlaps with the MFMAs if many bytes are in flight, and the
//     bytes in flight are bounded by LDS (160 KB).
//   * every barrier used to cost its skew plus the first operand reads of the new stage.
//
// Design:
//   * stages of BK = 32 (rows of 64 bytes), NSTG of them in a ring (7 x 22 KB for 128 x 224),
//     NSTG - 2 in flight at any time;
//   * the barrier that certifies stage kt+1 is taken inside stage kt (after its second MFMA
//     group).  Nothing waits at a stage boundary: the operand reads of stage kt+1 are issued
//     during stage kt (B fragments six MFMA groups ahead, A fragments right after the
//     barrier), so a wave's MFMA stream is continuous from the first K-step to the last;
//   * operand reads and their waits are written by hand (ds_read_b128 + s_waitcnt lgkmcnt(n)):
//     LDS reads of a wave complete in order, so "at most n outstanding" says exactly which
//     fragments have landed, and the table of n per MFMA group is derived at compile time
//     from the issue order;
//   * a wave-level direct-to-LDS load writes 64 lanes x 16 bytes contiguously (16 rows of 64
//     bytes), so rows cannot be padded; the 16-byte chunk c of row r is stored at chunk
//     position c ^ ((r >> 1) & 3) instead.  Measured with a ds_read_b128 probe on MI355X: this
//     key reads at ~235 B/clk per CU like a contiguous pattern, whereas no swizzle, c ^ (r & 3)
//     and c ^ ((r >> 2) & 3) all conflict two ways (~120 B/clk).
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "ops_gemm_bf16.h"
#include "wave.h"

namespace bfuse {

template <int M_, int N_, int K_, int BM_, int BN_, int NSTG_ = 7, int WGM_ = 4, int WGN_ = 2>
struct GemmBf16NTRing {
    static constexpr int M = M_, N = N_, K = K_, BM = BM_, BN = BN_, NSTG = NSTG_;
    static constexpr int BK = 32;
    static constexpr int WGM = WGM_, WGN = WGN_, NWAVES = WGM_ * WGN_;
    static constexpr int THREADS = 64 * NWAVES;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 16, TN = WN / 16;
    static constexpr int NKT = K / BK;
    static constexpr int ROWS = BM + BN;
    static constexpr int GROUPS = ROWS / 16;                       // wave-level loads per stage (16 rows each)
    static constexpr int GPW = (GROUPS + NWAVES - 1) / NWAVES;     // waves < GEXTRA issue GPW of them, the others GPW - 1
    static constexpr int GEXTRA = GROUPS % NWAVES == 0 ? NWAVES : GROUPS % NWAVES;
    static constexpr int STAGE_BYTES = ROWS * 64;
    static constexpr int CPITCH = BN + 8;
    static constexpr int OCHUNKS = BM * (BN / 8);
    static constexpr int PD = TN - 1;                              // B fragments are read PD MFMA groups ahead
    static_assert(M % BM == 0 && N % BN == 0 && K % BK == 0 && NKT % 2 == 0, "tile must divide the problem");
    static_assert(BM % WGM == 0 && BN % WGN == 0 && WM % 16 == 0 && WN % 16 == 0 && ROWS % 16 == 0 && BN % 8 == 0, "tile shape");
    static_assert(TM == 2 || TM == 4, "the hand-written LDS wait lists two or four A fragments");
    static_assert(TN >= 3, "the read-ahead ring needs at least three B fragments per stage");
    static_assert(OCHUNKS % THREADS == 0 && NSTG >= 4 && NKT >= NSTG - 1, "pipeline shape");
    static constexpr int MT = M / BM, NT = N / BN;
    static_assert((MT * NT) % 8 == 0 && NT % 8 == 0, "tiles are dealt to 8 XCDs");

    static constexpr Dims3 GRID{MT * NT, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    static constexpr bool LOOP_BARRIERS = true;   // one workgroup barrier per K-stage, not only in the epilogue
    static constexpr int EPI_BYTES = BM * CPITCH * 2;
    static_assert(NSTG * STAGE_BYTES <= 160 * 1024 && EPI_BYTES <= 160 * 1024, "LDS");
    struct Smem {
        __attribute__((aligned(1024))) unsigned char t[(NSTG * STAGE_BYTES > EPI_BYTES) ? NSTG * STAGE_BYTES : EPI_BYTES];
    };
    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    // s_waitcnt vmcnt(n), other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
    template <int N_OUT>
    __device__ static __forceinline__ void wait_vm()
    {
        __builtin_amdgcn_s_waitcnt((N_OUT & 0xF) | ((N_OUT >> 4) << 14) | 0x0F70);
    }
    // own loads of the K-step that is due have landed: at most NEWER younger K-steps outstanding
    template <int NEWER>
    __device__ static __forceinline__ void wait_step(bool full)
    {
        if constexpr (GEXTRA == NWAVES) {
            wait_vm<GPW * NEWER>();
        } else {
            if (full) wait_vm<GPW * NEWER>();
            else wait_vm<(GPW - 1) * NEWER>();
        }
    }
    // this wave's loads of K-step kt into the stage at byte offset stage_off
    __device__ static __forceinline__ void issue(const unsigned short* const (&src)[GPW], lds_u8* wave_base, int stage_off, int kt, bool full)
    {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int i = 0; i < GPW; ++i)
            if (i + 1 < GPW || full)
                __builtin_amdgcn_global_load_lds(src[i] + kt * BK, wave_base + stage_off + i * NWAVES * 1024, 16, 0, 0);
#endif
    }

    __device__ static __forceinline__ bf16x8 lds_read(int addr)
    {
        bf16x8 r;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
#else
        r = bf16x8{};
#endif
        return r;
    }
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

    // ---- issue order of the operand reads, and what may still be in flight at each wait -----
    // During stage kt a wave issues, after the MFMAs of group b:
    //   b == 0 : B(kt, TN-1)
    //   b == 1 : [barrier]  B(kt+1, 0), A(kt+1, 0..TM-1)
    //   b >= 2 : B(kt+1, b-1)
    // Group b of stage kt needs B(kt, b) and A(kt, *).  Reads complete in order, so it may
    // start once at most `allowed(b)` reads issued after the youngest of those are outstanding.
    static constexpr int READS_PER_STAGE = TN + TM;
    // position, in one stage's issue sequence, of B(next, j) / B(cur, TN-1) / last A(next)
    static constexpr int pos_b_next(int j) { return j == 0 ? 1 : 1 + TM + j; }   // issued at group j+1
    static constexpr int pos_b_last() { return 0; }                              // issued at group 0
    static constexpr int pos_a_next() { return 1 + TM; }                         // last A fragment (group 1)
    // reads issued in a stage before the wait of its group b
    static constexpr int issued_before(int b) { return b == 0 ? 0 : (b == 1 ? 1 : 1 + TM + b - 1); }
    static constexpr int allowed(int b)
    {
        // youngest needed read, as (stage, position): stage -1 = the previous stage's sequence
        int need_stage = -1, need_pos = pos_a_next();            // A(kt) was issued in stage kt-1
        if (b == TN - 1) {
            need_stage = 0;
            need_pos = pos_b_last();
        } else if (pos_b_next(b) > need_pos) {
            need_pos = pos_b_next(b);
        }
        const int after_in_prev = need_stage == -1 ? READS_PER_STAGE - 1 - need_pos : 0;
        const int after_in_cur = need_stage == -1 ? issued_before(b) : issued_before(b) - 1 - need_pos;
        return after_in_prev + after_in_cur;
    }
    static_assert(TM != 2 || TN != 7 || (allowed(0) == 5 && allowed(1) == 5 && allowed(2) == 7 && allowed(6) == 7), "wait table");

    struct Ctx {
        int a_ad[TM], b_ad[TN];                 // LDS byte address of every fragment in stage 0
        const unsigned short* src[GPW];         // this lane's global source of every load, K-step 0
        lds_u8* wave_base;                      // LDS destination of this wave's first load, stage 0
        bool full;
    };

    // MFMA group B_ of stage kt (fragments af[P], bq[B_]); cur / nxt are the byte offsets of the
    // ring stages holding K-steps kt and kt+1
    template <int P, int B_, class Sync>
    __device__ static __forceinline__ void groups(int kt, int cur, int nxt, f32x4 (&acc)[TM][TN], bf16x8 (&af)[2][TM], bf16x8 (&bq)[TN],
                                                  const Ctx& c, Sync& sync)
    {
        if constexpr (B_ < TN) {
            wait_lds<allowed(B_)>(bq[B_], af[P]);
#pragma unroll
            for (int a = 0; a < TM; ++a)
                acc[a][B_] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[P][a], bq[B_], acc[a][B_], 0, 0, 0);
            if constexpr (B_ == 0) {
                bq[TN - 1] = lds_read(c.b_ad[TN - 1] + cur);
            } else if constexpr (B_ == 1) {
                // K-step kt+1 is complete in LDS once every wave's own part has landed; at this
                // point every wave has also finished reading K-step kt-1, whose stage is refilled
                if (kt + NSTG - 2 < NKT) wait_step<NSTG - 3>(c.full);
                else wait_vm<0>();
                sync.bare();
                if (kt + NSTG - 1 < NKT) {
                    int refill = cur - STAGE_BYTES;
                    if (refill < 0) refill += NSTG * STAGE_BYTES;
                    issue(c.src, c.wave_base, refill, kt + NSTG - 1, c.full);
                }
                bq[0] = lds_read(c.b_ad[0] + nxt);
#pragma unroll
                for (int a = 0; a < TM; ++a) af[P ^ 1][a] = lds_read(c.a_ad[a] + nxt);
            } else {
                bq[B_ - 1] = lds_read(c.b_ad[B_ - 1] + nxt);
            }
            __builtin_amdgcn_sched_barrier(0);
            groups<P, B_ + 1>(kt, cur, nxt, acc, af, bq, c, sync);
        }
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
        const int wm = wave / WGN, wn = wave % WGN;
        const int li = lane & 15, kq = lane >> 4;

        Ctx c;
        c.full = wave < GEXTRA;
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
            int row = 16 * (wave + i * NWAVES) + (lane >> 2);
            if (row >= ROWS) row = ROWS - 1;  // slot not issued (see `full`)
            const int gc = (lane & 3) ^ ((row >> 1) & 3);
            c.src[i] = (row < BM ? A + (size_t)(m0 + row) * K : Wt + (size_t)(n0 + row - BM) * K) + gc * 8;
        }
        c.wave_base = (lds_u8*)sm.t + wave * 1024;
        const int lds_base = (int)(unsigned)(unsigned long long)(lds_u8*)sm.t;
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int row = wm * WM + a * 16 + li;
            c.a_ad[a] = lds_base + row * 64 + ((kq ^ ((row >> 1) & 3)) << 4);
        }
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int row = BM + wn * WN + b * 16 + li;
            c.b_ad[b] = lds_base + row * 64 + ((kq ^ ((row >> 1) & 3)) << 4);
        }

        f32x4 acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

        // K-steps 0 .. NSTG-2 go out; K-step 0 is certified here, K-step kt+1 inside stage kt
#pragma unroll
        for (int s = 0; s < NSTG - 1; ++s) issue(c.src, c.wave_base, s * STAGE_BYTES, s, c.full);
        wait_step<NSTG - 2>(c.full);
        sync.raw();
        // the reads a previous stage would have left in flight, in the same order
        bf16x8 af[2][TM], bq[TN];
        bq[0] = lds_read(c.b_ad[0]);
#pragma unroll
        for (int a = 0; a < TM; ++a) af[0][a] = lds_read(c.a_ad[a]);
#pragma unroll
        for (int b = 1; b < TN - 1; ++b) bq[b] = lds_read(c.b_ad[b]);
        __builtin_amdgcn_sched_barrier(0);

        int cur = 0;
#pragma unroll 1   // stays rolled: registers with reads in flight must never be spilled
        for (int kt = 0; kt < NKT; kt += 2) {
            int nxt = cur + STAGE_BYTES;
            if (nxt == NSTG * STAGE_BYTES) nxt = 0;
            groups<0, 0>(kt, cur, nxt, acc, af, bq, c, sync);
            cur = nxt;
            nxt = cur + STAGE_BYTES;
            if (nxt == NSTG * STAGE_BYTES) nxt = 0;
            groups<1, 0>(kt + 1, cur, nxt, acc, af, bq, c, sync);
            cur = nxt;
        }
        // The last stage read ahead into a stage that holds nothing new.  Those reads must have
        // landed before their registers are reused and before the tile buffer overwrites LDS:
        // the compiler takes an asm output for written when the asm is issued, so a result
        // nobody reads would leave its register free for an accumulator while the load is
        // still in flight.  Naming every fragment after the wait keeps them allocated until here.
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int b = 0; b < TN; ++b) asm volatile("" : "+v"(bq[b]));
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            asm volatile("" : "+v"(af[0][a]));
            asm volatile("" : "+v"(af[1][a]));
        }
#endif
        sync();

        unsigned short* ct = reinterpret_cast<unsigned short*>(sm.t);
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
            const int ch = tid + i * THREADS;
            const int row = ch / (BN / 8), col = (ch % (BN / 8)) * 8;
            *reinterpret_cast<u32x4*>(C + (size_t)(m0 + row) * N + n0 + col) =
                *reinterpret_cast<const u32x4*>(ct + row * CPITCH + col);
        }
    }
};

}  // namespace bfuse
