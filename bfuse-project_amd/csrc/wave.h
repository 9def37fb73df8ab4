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

// ---- synchronisation policies ---------------------------------------------------------
// Counts waits that gave up (see GroupSync); read back by the host after a fused launch.
static __device__ unsigned int g_sync_timeouts;

// Whole-workgroup barrier: standalone kernels and block-fused kernels (each workgroup runs
// one operator; waves outside the operator's thread range have already exited, and the
// hardware barrier only counts waves that are still alive).
struct BlockSync {
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

}  // namespace bfuse
