// Wave64 primitives for gfx950: DPP reductions and the two synchronisation policies an
// operator body can be instantiated with.
#pragma once
#include <hip/hip_runtime.h>

namespace bfuse {

// ---- DPP cross-lane moves -------------------------------------------------------------
// dpp_ctrl encodings (GCN3+/CDNA): quad_perm 0x00-0xff, row_mirror 0x140, row_half_mirror 0x141.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v)
{
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, false));
}

struct SumOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

// All 64 lanes end up holding the reduction over the wave.  Inside each row of 16 lanes the
// reduction is a butterfly on DPP (no LDS traffic); the four row results are combined in
// lane order 0,16,32,48 through scalar registers, so the operation order is fixed and is
// the same in every kernel the body is instantiated in.
template <class Op>
__device__ __forceinline__ float wave_reduce(float v, Op op)
{
    v = op(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
    v = op(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
    v = op(v, dpp_mov<0x141>(v));  // row_half_mirror
    v = op(v, dpp_mov<0x140>(v));  // row_mirror
    const int i = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 48));
    return op(op(r0, r1), op(r2, r3));
}

__device__ __forceinline__ float wave_sum(float v) { return wave_reduce(v, SumOp{}); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce(v, MaxOp{}); }

// ---- direct global -> LDS load with a scalar base ------------------------------------
// 64 lanes x 16 bytes: lane L fetches base + voff (its own 32-bit byte offset) and the data lands at
// LDS byte address lds_addr + 16 L.  `base` and `lds_addr` must be wave-uniform (they travel in
// scalar registers).  Written as asm because the address then costs no vector instruction: the
// compiler's own selection of this load turns "uniform base + lane offset" into a 64-bit vector add
// per load whenever the offset was computed outside the loop, and on a SIMD that is streaming MFMAs
// every vector ALU instruction, from whichever wave, takes ~20 clocks out of that stream.
// The compiler does not count this load in vmcnt: callers wait with explicit s_waitcnt vmcnt(n).
__device__ __forceinline__ void dma_load_lds_b128(unsigned voff, const void* base, unsigned lds_addr)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
#endif
}

// two fp32 -> two bf16 in one word (lo in the low half), round to nearest even: v_cvt_pk_bf16_f32
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned int pack_bf16(float lo, float hi)
{
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
}

// ---- synchronisation policies ---------------------------------------------------------
// Counts waits that gave up (see GroupSync); read back by the host after a fused launch.
static __device__ unsigned int g_sync_timeouts;

// Whole-workgroup barrier: standalone kernels and block-fused kernels (each workgroup runs
// one operator; waves outside the operator's thread range have already exited, and the
// hardware barrier only counts waves that are still alive).
struct BlockSync {
    static constexpr bool kYields = false;
    __device__ __forceinline__ void yield() const {}   // see JoinSync
    __device__ __forceinline__ void yield(float&) const {}
    __device__ __forceinline__ void operator()() const { __syncthreads(); }
    // Barrier WITHOUT a memory fence: only this wave's LDS accesses are drained.  For
    // pipelines that keep global->LDS loads in flight across the barrier and account for
    // them with explicit s_waitcnt vmcnt(n) (a fence would wait for all of them).
    __device__ __forceinline__ void raw() const
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    // The instruction alone: nothing of this wave is drained.  For kernels that keep LDS reads
    // in flight across the barrier and count them by hand; the caller guarantees that whatever
    // another wave may overwrite after the barrier has already been consumed by this one.
    __device__ __forceinline__ void bare() const
    {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
};

// How many polls a side barrier makes before it gives up.  Device data so that the host can lower
// it (bfuse_set_sync_spin_limit) -- read only by a wave that already has to wait.
static __device__ unsigned int g_sync_spin_limit = 1u << 22;

// Barrier over the waves of ONE side of a horizontally fused workgroup.  gfx950 has no
// partial-workgroup barrier (s_barrier always spans the workgroup), so the side's waves
// meet on an LDS counter: lane 0 of each wave adds 1, then the wave polls until the counter
// reaches waves * epoch.  All waves of a workgroup are resident on one CU for the whole
// kernel, so the wait cannot depend on a wave that has not been scheduled.  The poll is
// bounded: a side whose waves disagree on the number of barriers gives up after
// g_sync_spin_limit polls, records it in g_sync_timeouts and carries on, so the grid always
// drains; the host reads the counter at its next synchronisation and reports BFUSE_ERR_SYNC.
struct GroupSync {
    static constexpr bool kYields = false;
    __device__ __forceinline__ void yield() const {}   // see JoinSync
    __device__ __forceinline__ void yield(float&) const {}
    unsigned int* counter;  // in LDS, zeroed before the sides diverge
    unsigned int waves;
    unsigned int epoch;

    __device__ __forceinline__ void poll(unsigned int target)
    {
        if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) return;
        const unsigned int limit = *(volatile unsigned int*)&g_sync_spin_limit;
        unsigned int spins = 0;
        do {
            __builtin_amdgcn_s_sleep(1);
            if (++spins >= limit) {
                if ((threadIdx.x & 63) == 0) atomicAdd(&g_sync_timeouts, 1u);
                break;
            }
        } while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target);
    }

    __device__ __forceinline__ void operator()()
    {
        ++epoch;
        // order this wave's earlier LDS writes before its arrival
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if ((threadIdx.x & 63) == 0) atomicAdd(counter, 1u);
        poll(waves * epoch);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }

    // Same meeting point without fences (see BlockSync::raw): the caller has already waited
    // for the loads the other waves depend on; LDS operations of one wave execute in order,
    // so reads issued after the poll see what the other waves wrote before they arrived.
    // the counter barrier uses LDS operations itself, so it cannot leave the caller's in flight
    __device__ __forceinline__ void bare() { raw(); }
    __device__ __forceinline__ void raw()
    {
        ++epoch;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if ((threadIdx.x & 63) == 0) atomicAdd(counter, 1u);
        poll(waves * epoch);
        asm volatile("" ::: "memory");
    }
};

// Policy of a barrier-FREE side whose partner in a horizontally fused workgroup keeps the hardware
// barrier inside its main loop.  s_barrier counts every live wave of the workgroup, so the partner's
// first barrier would wait until this side's waves have exited -- the two sides would run one after
// the other.  Instead this side takes part: its body is cut into sections at yield() calls, each
// yield() is one s_barrier, matched with the partner's 1st, 2nd, ... loop barrier.  While this side
// is alive the partner advances one loop step per section; after its last section it exits and the
// hardware stops counting its waves.  A body may yield at most as often as every wave of the partner
// is certain to synchronise (Op::YIELDS <= Partner::MIN_BARRIERS, checked at compile time), and it
// keeps its loads in flight across the yield: it issues them before and waits for them after, so a
// section costs the partner's step nothing but the arrival.
// The compiler-level fences keep memory operations and the schedule on their side of the barrier.
struct JoinSync {
    static constexpr bool kYields = true;
    __device__ __forceinline__ void yield() const
    {
        float none = 0.f;
        yield(none);
    }
    // `carried` comes out as a value the compiler knows nothing about (unchanged).  The barrier is
    // written as asm with `carried` as its operand so that it sits in the data flow: what `carried`
    // was computed from is finished before the barrier, and arithmetic that uses it afterwards
    // cannot be moved to before it.  (The memory clobber orders memory operations only, and only
    // through pointers the compiler cannot trace -- see opaque_pointer; pure arithmetic it would
    // otherwise compute early and keep in registers across the sections before.)
    __device__ __forceinline__ void yield(float& carried) const
    {
        __builtin_amdgcn_sched_barrier(0);
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_barrier" : "+v"(carried) : : "memory");
#endif
        __builtin_amdgcn_sched_barrier(0);
    }
    // a side run under this policy has no barriers of its own (HAS_BARRIERS = false)
    __device__ __forceinline__ void operator()() const {}
};

// The value, unchanged, as one the compiler knows nothing about: what was derived from it before
// (say its widened copy) is not kept for later uses, it is derived again.
template <class V>
__device__ __forceinline__ void opaque_value(V& v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(v));
#endif
}

// A kernel-argument pointer (wave-uniform, `__restrict__`) as the compiler sees an unknown pointer
// into device memory.  The memory clobbers in JoinSync::yield() order nothing against memory that
// is only reachable through a noalias argument (an asm without pointer operands cannot touch it, so
// loads and stores through it may cross); a body that must keep its sections apart takes its
// pointers through here.
template <class T>
__device__ __forceinline__ T* opaque_pointer(T* p)
{
    unsigned long long bits = (unsigned long long)p;
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+s"(bits));
#endif
    // an integer turned into a pointer to global memory: accesses stay global_load / global_store
    return (T*)(__attribute__((address_space(1))) T*)bits;
}

// An operator with BYTES more of LDS per workgroup than it uses: bounds how many of its workgroups are resident
// on a CU (160 KB / (BYTES + its own)).  The one-wave batched products run best at one wave per SIMD -- every wave
// streams its operands straight into registers, and the two or three waves per SIMD their registers allow only
// queue behind each other in the memory pipeline: with 32 KB reserved (four workgroups per CU) the 1024-fold
// products with 64 x 64 tiles took 461 / 703 / 124 / 147 us instead of 561 / 937 / 131 / 166, and 208 x 208 x 64
// with 208 x 32 tiles 75 us instead of 94 (24 KB, six per CU: 119; 40 KB, three per CU: 92).  The one-wave
// convolutions on three input channels want about three waves per SIMD (the 7 x 7 on RGB at batch 1024: 3.53 ms
// with twelve workgroups per CU, 4.43 with the sixteen its registers allow, 4.2 with six).
template <class Op, int BYTES>
struct LdsReserve : Op {
    struct Smem {
        typename Op::Smem s;
        unsigned char reserve[BYTES];
    };
    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F, void* O, Sync sync)
    {
        if (vblock < 0) sm.reserve[tid] = 1;   // never true (workgroup ids are not negative): keeps the reservation allocated
        Op::run(vblock, tid, sm.s, I, F, O, sync);
    }
};

}  // namespace bfuse
