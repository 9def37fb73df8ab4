// Memory-bound sides: elementwise bias+ReLU, LayerNorm, causal softmax, RMSNorm+RoPE.
// All use 128-bit coalesced loads/stores and wave64 DPP reductions; none needs LDS or a
// barrier, so they can sit on either side of a horizontal or block fusion.
//
// The reference generates none of these (it only fuses GEMM-like TVM kernels); their
// arithmetic follows the reference's Relay dumps, cited per operator.
#pragma once
#include <hip/hip_runtime.h>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct NoSmem {
    // empty: the operator uses no LDS
};

// y = max(x + b, 0) over COUNT floats, b a full-length vector.
// Workgroup v owns a contiguous slice of COUNT / GRID floats; consecutive lanes read
// consecutive 16-byte vectors.
template <int COUNT_, int THREADS_, int NBLOCKS_>
struct BiasRelu {
    static constexpr int COUNT = COUNT_, THREADS = THREADS_;
    static constexpr Dims3 GRID{NBLOCKS_, 1, 1};
    static constexpr Dims3 BLOCK{THREADS_, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int PER_BLOCK = COUNT / NBLOCKS_;
    static constexpr int ITERS = PER_BLOCK / (4 * THREADS);
    static_assert(COUNT % NBLOCKS_ == 0 && PER_BLOCK % (4 * THREADS) == 0, "slice must be whole vectors");
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void* F,
                                               void* O, Sync)
    {
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)vblock * (PER_BLOCK / 4);
        const f32x4* __restrict__ b = static_cast<const f32x4*>(F) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4 xv[ITERS], bv[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            xv[it] = x[it * THREADS + tid];
            bv[it] = b[it * THREADS + tid];
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            f32x4 s = xv[it] + bv[it];
            f32x4 r;
            r[0] = fmaxf(s[0], 0.f);
            r[1] = fmaxf(s[1], 0.f);
            r[2] = fmaxf(s[2], 0.f);
            r[3] = fmaxf(s[3], 0.f);
            y[it * THREADS + tid] = r;
        }
    }
};

// y = x over COUNT floats: a plain copy of known size, the calibration kernel for memory
// counters (COUNT*4 bytes read, COUNT*4 bytes written).
template <int COUNT_, int THREADS_>
struct CopyF32 {
    static constexpr int COUNT = COUNT_, THREADS = THREADS_;
    static constexpr int PER_BLOCK = 4 * THREADS * 4;  // four 128-bit vectors per thread
    static_assert(COUNT % PER_BLOCK == 0, "whole workgroups");
    static constexpr Dims3 GRID{COUNT / PER_BLOCK, 1, 1};
    static constexpr Dims3 BLOCK{THREADS_, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void*, void* O, Sync)
    {
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)vblock * (PER_BLOCK / 4);
        f32x4 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = x[i * THREADS + tid];
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i * THREADS + tid] = v[i];
    }
};

// LayerNorm over the last axis of x[ROWS, D]; F holds gamma[D] then beta[D].
//   y = (x - mean) * (1 / sqrt(var + eps)) * gamma + beta, biased variance
// (files/bert-base-uncased.txt:8-16).  One wave per row, the row lives in registers
// (D/256 128-bit vectors per lane), mean and variance are two DPP reductions.
template <int ROWS_, int D_, int WAVES_, int EPS_E12_ = 1>
struct LayerNorm {
    static constexpr int ROWS = ROWS_, D = D_, WAVES = WAVES_;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr Dims3 GRID{ROWS / WAVES, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int VEC = D / 256;  // 128-bit vectors per lane
    static_assert(ROWS % WAVES == 0 && D % 256 == 0, "one wave per row, whole vectors per lane");
    using Smem = NoSmem;

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void* F,
                                               void* O, Sync)
    {
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        const int row = vblock * WAVES + wave;
        const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)row * (D / 4);
        const f32x4* __restrict__ gamma = static_cast<const f32x4*>(F);
        const f32x4* __restrict__ beta = gamma + D / 4;
        f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)row * (D / 4);
        const float eps = 1e-12f * (float)EPS_E12_;

        f32x4 v[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = x[i * 64 + lane];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
        const float mean = wave_sum(s) / (float)D;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            v[i] -= mean;
            q += (v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3]);
        }
        const float var = wave_sum(q) / (float)D;
        const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const f32x4 g = gamma[i * 64 + lane], b = beta[i * 64 + lane];
            y[i * 64 + lane] = (v[i] * rstd) * g + b;
        }
    }
};

// softmax over the last axis of x[HEADS, S, S] with the causal mask: column j > row i is
// masked to -inf before the softmax, so its probability is exactly 0
// (files/gpt2.txt:35-36).  One wave per row; only the visible prefix is read.
template <int HEADS_, int S_, int WAVES_, int RPW_ = 1, int RB_ = 1>
struct SoftmaxCausal {
    // RPW rows per wave, processed RB at a time (RB rows' loads are in flight together)
    static constexpr int HEADS = HEADS_, S = S_, WAVES = WAVES_, RPW = RPW_, RB = RB_;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int ROWS = HEADS * S;
    static constexpr Dims3 GRID{ROWS / (WAVES * RPW), 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int VEC = S / 256;
    static_assert(ROWS % (WAVES * RPW) == 0 && S % 256 == 0 && RPW % RB == 0, "whole rows per wave, whole vectors per lane");
    using Smem = NoSmem;

    // rows row0 + b*stride, b = 0..RB-1; every row is reduced on its own, in the same order
    // whatever RB is.
    //
    // The query position i of a row is the same for every lane of the wave, so what the causal mask does
    // to each 256-column block (one f32x4 per lane) is decided by scalar branches: a block left of the
    // diagonal is visible whole (no per-element test), the block on the diagonal is masked per element,
    // a block right of it is hidden whole -- it is neither loaded nor run through max / exp / sum, its
    // probabilities are written as zeros.  Under fusion every vector instruction of this side takes an
    // issue slot on a SIMD whose matrix core the partner's GEMM keeps busy (measured on pair 4: the
    // softmax's arithmetic costs the fused kernel 0.8 us, its loads and stores 0.6), so the row's
    // instruction count is what is minimised: exp(x - m) is one fused multiply-add and one v_exp_f32
    // per element, the row's reciprocal one v_rcp_f32.
    __device__ static __forceinline__ void rows(int row0, int stride, int lane, const void* I, void* O)
    {
        const float ninf = -__builtin_inff();
        f32x4 v[RB][VEC];
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            const int row = row0 + b * stride;
            const int i = row % S;  // query position: columns 0..i are visible
            const f32x4* __restrict__ x = static_cast<const f32x4*>(I) + (size_t)row * (S / 4);
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                if (256 * c + 255 <= i) {                 // visible whole (scalar branch)
                    v[b][c] = x[c * 64 + lane];
                } else if (256 * c <= i) {                // on the diagonal
                    const int col = (c * 64 + lane) * 4;
                    v[b][c] = f32x4{ninf, ninf, ninf, ninf};
                    if (col <= i) {
                        const f32x4 t = x[c * 64 + lane];
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[b][c][e] = (col + e <= i) ? t[e] : ninf;
                    }
                }
            }
        }
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            const int row = row0 + b * stride;
            const int i = row % S;
            f32x4* __restrict__ y = static_cast<f32x4*>(O) + (size_t)row * (S / 4);
            float m = ninf;
#pragma unroll
            for (int c = 0; c < VEC; ++c)
                if (256 * c <= i) m = fmaxf(fmaxf(m, fmaxf(v[b][c][0], v[b][c][1])), fmaxf(v[b][c][2], v[b][c][3]));
            m = wave_max(m);
            const float mneg = -m * 1.4426950408889634f;
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                if (256 * c <= i) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)   // exp(x - m) = 2^(x log2 e - m log2 e): one fma, one v_exp_f32; masked columns give 2^-inf == 0
                        v[b][c][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[b][c][e], 1.4426950408889634f, mneg));
                    s += (v[b][c][0] + v[b][c][1]) + (v[b][c][2] + v[b][c][3]);
                }
            }
            s = wave_sum(s);
            const float rs = __builtin_amdgcn_rcpf(s);   // s >= 1 (the row's maximum contributes 2^0)
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                if (256 * c <= i) y[c * 64 + lane] = v[b][c] * rs;
                else y[c * 64 + lane] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void*,
                                               void* O, Sync)
    {
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        // consecutive waves take consecutive rows; a wave's RPW rows are WAVES*GRID apart so
        // that every pass over the grid touches one contiguous slab of the matrix
        constexpr int stride = GRID.size() * WAVES;
        for (int r = 0; r < RPW; r += RB)
            rows((r * GRID.size() + vblock) * WAVES + wave, stride, lane, I, O);
    }
};

// RMSNorm over x[S, HEADS*HD] (bf16) followed by rotate-half RoPE per head, bf16 out:
//   t = w * (x * (1/sqrt(mean(x^2) + 1e-5)))                     files/Meta-Llama-3-8B.txt:5-14
//   out = t*cos + concat(-t[HD/2:], t[:HD/2])*sin                 files/Meta-Llama-3-8B.txt:19-26
// evaluated in fp32 from the bf16 inputs, rounded once (to nearest even) to bf16.
// F holds w[HEADS*HD] (bf16), then cos[S,HD] and sin[S,HD] (fp32), as the dump holds them
// as (1,1,S,HD) constants.  One wave per row (sequence position); a lane owns, for each of
// its (head, octet) slots, the eight elements j..j+7 AND their rotation partners j+HD/2.., so
// the rotation needs no cross-lane traffic and every load/store is 128 bits.
template <int S_, int HEADS_, int HD_, int WAVES_>
struct RmsNormRope {
    static constexpr int S = S_, HEADS = HEADS_, HD = HD_, WAVES = WAVES_;
    static constexpr int D = HEADS * HD, HALF = HD / 2;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr Dims3 GRID{S / WAVES, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = false;
    static constexpr int OCT = HALF / 8;                 // octets per half head
    static constexpr int SLOTS = HEADS * OCT / 64;       // (head, octet) slots per lane
    // Sections of the body when it runs under JoinSync (its partner's loop barriers), a yield after
    // each but the last: every load the row needs is requested | WAIT_STEPS - 1 empty sections that
    // let the partner's steps pass while the data arrives | the reduction | one slot each.
    static constexpr int WAIT_STEPS = 3;
    static constexpr int YIELDS = WAIT_STEPS + SLOTS;
    static_assert(S % WAVES == 0 && HALF % 8 == 0 && (HEADS * OCT) % 64 == 0, "whole slots per lane");
    static_assert(64 % OCT == 0, "a lane's octet offset does not depend on the slot");
    static constexpr size_t COS_OFFSET = (size_t)D * 2;                 // bytes into F
    static constexpr size_t SIN_OFFSET = COS_OFFSET + (size_t)S * HD * 4;
    static constexpr size_t F_BYTES = SIN_OFFSET + (size_t)S * HD * 4;
    using Smem = NoSmem;

    __device__ static __forceinline__ void unpack(const u16x8& h, float (&f)[8])
    {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = __builtin_bit_cast(float, (unsigned int)h[e] << 16);
    }
    // The arithmetic of one element pair (j, j + HALF) -- the one place it is written, whichever way
    // the inputs arrived:  t = w (x r);  out_lo = t_lo cos_lo - t_hi sin_lo;  out_hi = t_hi cos_hi + t_lo sin_hi
    __device__ static __forceinline__ void rotate_pair(float w_lo, float w_hi, float x_lo, float x_hi, float r, float c_lo, float s_lo,
                                                       float c_hi, float s_hi, float& o_lo, float& o_hi)
    {
        const float tl = w_lo * (x_lo * r), th = w_hi * (x_hi * r);
        o_lo = tl * c_lo + (-th) * s_lo;
        o_hi = th * c_hi + tl * s_hi;
    }
    // eight fp32 -> eight bf16 (round to nearest even), two per conversion instruction
    __device__ static __forceinline__ u16x8 round_octet(const float (&f)[8])
    {
        u32x4 p;
#pragma unroll
        for (int e = 0; e < 4; ++e) p[e] = pack_bf16(f[2 * e], f[2 * e + 1]);
        return __builtin_bit_cast(u16x8, p);
    }
    __device__ static __forceinline__ int slot_base(int slot) { return (slot / OCT) * HD + (slot % OCT) * 8; }
    __device__ static __forceinline__ void load_octets(u16x8& lo, u16x8& hi, int slot, const unsigned short* __restrict__ p)
    {
        lo = *reinterpret_cast<const u16x8*>(p + slot_base(slot));
        hi = *reinterpret_cast<const u16x8*>(p + slot_base(slot) + HALF);
    }

    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem&, const void* I, const void* F,
                                               void* O, Sync sync)
    {
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave-uniform: addresses built on it stay in scalar registers
        const int pos = vblock * WAVES + wave;
        if constexpr (Sync::kYields) {
            // sections must stay sections: memory operations may not cross the yields
            I = opaque_pointer(I);
            F = opaque_pointer(F);
            O = opaque_pointer(O);
        }
        const unsigned short* __restrict__ x = static_cast<const unsigned short*>(I) + (size_t)pos * D;
        const unsigned short* __restrict__ w = static_cast<const unsigned short*>(F);
        const float* __restrict__ cosv = reinterpret_cast<const float*>(static_cast<const char*>(F) + COS_OFFSET) + (size_t)pos * HD;
        const float* __restrict__ sinv = reinterpret_cast<const float*>(static_cast<const char*>(F) + SIN_OFFSET) + (size_t)pos * HD;
        unsigned short* __restrict__ y = static_cast<unsigned short*>(O) + (size_t)pos * D;

        // the row stays in registers as it was loaded (bf16, four registers per octet) and is widened
        // where it is used: half the registers of an fp32 copy
        u16x8 xl[SLOTS], xh[SLOTS];
        float ss = 0.f;
        // held operands of the sectioned form: weights of every slot and the cos / sin values of the
        // lane's octet, which are the same for every slot
        u16x8 wlo[SLOTS], whi[SLOTS];
        f32x4 cl[2], ch[2], sl[2], sh[2];
        if constexpr (Sync::kYields) {
            // Nothing the row needs depends on the reduction, so everything is requested first and is
            // on its way while the partner's steps pass: a section that had to wait for memory would
            // hold up the partner's barrier for as long.
            const int j = (lane % OCT) * 8;
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) load_octets(xl[s], xh[s], s * 64 + lane, x);
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) load_octets(wlo[s], whi[s], s * 64 + lane, w);
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                cl[q] = *reinterpret_cast<const f32x4*>(cosv + j + 4 * q);
                ch[q] = *reinterpret_cast<const f32x4*>(cosv + j + HALF + 4 * q);
                sl[q] = *reinterpret_cast<const f32x4*>(sinv + j + 4 * q);
                sh[q] = *reinterpret_cast<const f32x4*>(sinv + j + HALF + 4 * q);
            }
#pragma unroll
            for (int i = 0; i < WAIT_STEPS; ++i) sync.yield();   // the loads stay in flight across them
        }
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            if constexpr (!Sync::kYields) load_octets(xl[s], xh[s], s * 64 + lane, x);
            float lo[8], hi[8];
            unpack(xl[s], lo);
            unpack(xh[s], hi);
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += lo[e] * lo[e] + hi[e] * hi[e];
        }
        const float r = 1.0f / sqrtf(wave_sum(ss) / (float)D + 1e-5f);

        if constexpr (Sync::kYields) {
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                float rs = r;
                sync.yield(rs);   // short sections: the partner waits at its barrier while one runs
                // the row's octets are widened again here rather than kept widened since the reduction
                opaque_value(xl[s]);
                opaque_value(xh[s]);
                const int slot = s * 64 + lane;
                float wl[8], wh[8], lo[8], hi[8];
                unpack(wlo[s], wl);
                unpack(whi[s], wh);
                unpack(xl[s], lo);
                unpack(xh[s], hi);
                float ol[8], oh[8];
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    rotate_pair(wl[e], wh[e], lo[e], hi[e], rs, cl[e / 4][e % 4], sl[e / 4][e % 4], ch[e / 4][e % 4], sh[e / 4][e % 4], ol[e], oh[e]);
                *reinterpret_cast<u16x8*>(y + slot_base(slot)) = round_octet(ol);
                *reinterpret_cast<u16x8*>(y + slot_base(slot) + HALF) = round_octet(oh);
            }
        } else {
            // on its own the body leaves the order of the operand loads to the compiler (it requests
            // all of them before the reduction)
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const int slot = s * 64 + lane;
                const int j = (slot % OCT) * 8;
                const int base = (slot / OCT) * HD + j;
                float wl[8], wh[8], lo[8], hi[8];
                unpack(*reinterpret_cast<const u16x8*>(w + base), wl);
                unpack(*reinterpret_cast<const u16x8*>(w + base + HALF), wh);
                unpack(xl[s], lo);
                unpack(xh[s], hi);
                float ol[8], oh[8];
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    rotate_pair(wl[e], wh[e], lo[e], hi[e], r, cosv[j + e], sinv[j + e], cosv[j + HALF + e], sinv[j + HALF + e], ol[e], oh[e]);
                *reinterpret_cast<u16x8*>(y + base) = round_octet(ol);
                *reinterpret_cast<u16x8*>(y + base + HALF) = round_octet(oh);
            }
        }
    }
};

}  // namespace bfuse
