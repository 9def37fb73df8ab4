// The three ways an operator body is instantiated, and the kernel registry.
//
//   single : one operator, the standalone ("unfused") kernel
//   bfuse  : block fusion  -- fused grid = sum of grids, blockIdx.x selects operator and
//            virtual block through a compile-time BlockPlan; LDS is a union of both sides
//            (the reference's emitted form: horizontal-fuser/src/Matchers.cc:523-602,
//            union layout Tools.cc:219-251)
//   bfuse_rt : block fusion whose BlockPlan is DATA (set by the host before the launch) and
//            whose workgroups are persistent: workgroup w handles fused block ids w, w + gridDim.x,
//            ...  Launched with gridDim.x = the plan's fused grid it is plain block fusion with
//            a run-time pattern (what the reference's legacy ratio sweep re-generated and
//            re-compiled for every M:N, legacy/tests/single_bgemm_conv2d/auto.py:9-14); launched
//            with a few workgroups per CU it is the persistent-block form of
//            legacy/tests/thread_pooling_test/temp.cu:576-612
//   hfuse  : horizontal fusion -- one workgroup hosts both operators on disjoint wave
//            ranges; LDS is the sum of both sides; where CUDA has bar.sync id,count
//            (Matchers.cc:288-320, 655-727) a side keeps the hardware barrier when that is
//            harmless, gets the LDS-counter GroupSync, or keeps the hardware barrier while the
//            barrier-free partner joins it (JoinSync) -- chosen per pair at compile time
//
// Every instantiation calls the same Op::run body with a virtual (block, thread) id -- the
// counterpart of the reference rewriting blockIdx/threadIdx to locals (Matchers.cc:255-286)
// -- so a fused kernel executes, per output element, the instruction sequence of the
// standalone kernel and the results are bit-identical.
//
// Kernel ABI, as in the reference (macro_h.py:182-198): extern "C", three pointers per
// operator (input, second operand, output), six for a fused pair (operator 1's three, then
// operator 2's), 1-D launch, no dynamic shared memory.
#pragma once
#include <hip/hip_runtime.h>

#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "dispatch.h"
#include "wave.h"

namespace bfuse {

// Every kernel is compiled to fit two waves per SIMD (at most 256 of the 512 VGPRs): a fused
// kernel allocates the larger side's registers for BOTH sides' waves, and with more than
// 256 a memory-bound workgroup could never be resident next to a GEMM workgroup.
constexpr int kMinWavesPerEu = 2;

template <class Op>
__device__ __forceinline__ void single_body(const void* I, const void* F, void* O)
{
    __shared__ typename Op::Smem sm;
    Op::run((int)blockIdx.x, (int)threadIdx.x, sm, I, F, O, BlockSync{});
}

template <class A, class B, int PATTERN, int P0, int P1>
struct BfusePair {
    static constexpr LaunchDims dims[2] = {{A::GRID, A::BLOCK}, {B::GRID, B::BLOCK}};
    static constexpr BlockPlan plan() { return make_block_plan(PATTERN, 2, dims, P0, P1); }
    static constexpr int THREADS = imax(A::THREADS, B::THREADS);
    static constexpr int GRID = A::GRID.size() + B::GRID.size();
    // a guarded side must be masked on whole waves, or its barrier would wait on lanes that never arrive
    static_assert(A::THREADS % kWaveSize == 0 && B::THREADS % kWaveSize == 0, "block sizes must be whole waves");
};

template <class A, class B, int PATTERN, int P0, int P1>
__device__ __forceinline__ void bfuse_body(const void* I1, const void* F1, void* O1, const void* I2,
                                           const void* F2, void* O2)
{
    using Pair = BfusePair<A, B, PATTERN, P0, P1>;
    union ShrdUnion {
        typename A::Smem a;
        typename B::Smem b;
    };
    __shared__ ShrdUnion su;
    constexpr BlockPlan plan = Pair::plan();
    int virt = 0;
    const int kernel_id = map_block(plan, (int)blockIdx.x, &virt);
    const int tid = (int)threadIdx.x;
    if (kernel_id == 0 && tid < A::THREADS) {
        A::run(virt, tid, su.a, I1, F1, O1, BlockSync{});
    } else if (kernel_id == 1 && tid < B::THREADS) {
        B::run(virt, tid, su.b, I2, F2, O2, BlockSync{});
    }
}

template <class A, class B>
struct BfuseRtPair {
    static constexpr int THREADS = imax(A::THREADS, B::THREADS);
    static constexpr int GRID = A::GRID.size() + B::GRID.size();
    static_assert(A::THREADS % kWaveSize == 0 && B::THREADS % kWaveSize == 0, "block sizes must be whole waves");
};

// A workgroup runs blocks of both operators one after the other, so waves that one operator
// does not use cannot simply exit as they do under plain block fusion; they skip the body and
// wait at the next iteration's workgroup barrier.  An operator narrower than the workgroup
// therefore cannot use s_barrier inside its body (the idle waves would be counted): it gets the
// LDS-counter barrier over its own waves, as under horizontal fusion.
template <class A, class B>
__device__ __forceinline__ void bfuse_rt_body(const BlockPlan& plan, const void* I1, const void* F1, void* O1,
                                              const void* I2, const void* F2, void* O2)
{
    struct Shrd {
        union {
            typename A::Smem a;
            typename B::Smem b;
        } u;
        // arrival counters of the LDS-counter barriers, three sets used in rotation: the set
        // zeroed at the top of iteration i is the one iteration i+1 will use, and it is not the
        // one a slow wave may still be polling from iteration i-1
        unsigned int arrive[3][2];
    };
    __shared__ Shrd sh;
    constexpr int T = BfuseRtPair<A, B>::THREADS;
    const int tid = (int)threadIdx.x;
    const int total = plan.fused_grid;
    if (tid < 6) (&sh.arrive[0][0])[tid] = 0u;
    int set = 0;
    for (int id = (int)blockIdx.x; id < total; id += (int)gridDim.x) {
        const int next = set == 2 ? 0 : set + 1;
        if (tid < 2) sh.arrive[next][tid] = 0u;
        __syncthreads();  // every wave has left the previous iteration: its LDS contents are dead
        int virt = 0;
        const int kernel_id = map_block(plan, id, &virt);   // scalar: the plan is a kernel argument
        if (kernel_id == 0 && tid < A::THREADS) {
            if constexpr (A::THREADS == T) A::run(virt, tid, sh.u.a, I1, F1, O1, BlockSync{});
            else A::run(virt, tid, sh.u.a, I1, F1, O1, GroupSync{&sh.arrive[set][0], (unsigned)(A::THREADS / kWaveSize), 0u});
        } else if (kernel_id == 1 && tid < B::THREADS) {
            if constexpr (B::THREADS == T) B::run(virt, tid, sh.u.b, I2, F2, O2, BlockSync{});
            else B::run(virt, tid, sh.u.b, I2, F2, O2, GroupSync{&sh.arrive[set][1], (unsigned)(B::THREADS / kWaveSize), 0u});
        }
        set = next;
    }
}

// does the operator take a workgroup barrier inside its main loop (it says so with LOOP_BARRIERS)?
template <class Op, class = void>
struct loop_barriers : std::false_type {};
template <class Op>
struct loop_barriers<Op, std::void_t<decltype(Op::LOOP_BARRIERS)>> : std::bool_constant<Op::LOOP_BARRIERS> {};

// how often the operator's body yields when run under JoinSync (0: it has no yield points), and how
// many workgroup barriers every wave of the operator is certain to execute
template <class Op, class = void>
struct yield_count : std::integral_constant<int, 0> {};
template <class Op>
struct yield_count<Op, std::void_t<decltype(Op::YIELDS)>> : std::integral_constant<int, Op::YIELDS> {};
template <class Op, class = void>
struct min_barriers : std::integral_constant<int, 0> {};
template <class Op>
struct min_barriers<Op, std::void_t<decltype(Op::MIN_BARRIERS)>> : std::integral_constant<int, Op::MIN_BARRIERS> {};

// Side X keeps the hardware barrier in its main loop and side Y, which has no barriers, joins the
// first yield_count<Y> of them (JoinSync): possible when Y has yield points and X synchronises at
// least that often.
template <class X, class Y>
constexpr bool joins_barriers = loop_barriers<X>::value && !Y::HAS_BARRIERS && yield_count<Y>::value > 0 &&
                                yield_count<Y>::value <= min_barriers<X>::value;

template <class A, class B>
struct HfusePair {
    static constexpr LaunchDims dims[2] = {{A::GRID, A::BLOCK}, {B::GRID, B::BLOCK}};
    static constexpr ThreadPlan plan() { return plan_threads(2, dims, kWaveSize); }
    static constexpr int THREADS = round_up(A::THREADS, kWaveSize) + round_up(B::THREADS, kWaveSize);
    static constexpr int GRID = imax(A::GRID.size(), B::GRID.size());
};

template <class A, class B>
__device__ __forceinline__ void hfuse_body(const void* I1, const void* F1, void* O1, const void* I2,
                                           const void* F2, void* O2)
{
    struct ShrdSum {
        typename A::Smem a;
        typename B::Smem b;
        unsigned int arrive[2];
    };
    __shared__ ShrdSum ss;
    constexpr ThreadPlan plan = HfusePair<A, B>::plan();
    // the only whole-workgroup barrier: zero the per-side arrival counters before the sides diverge
    if (threadIdx.x < 2) ss.arrive[threadIdx.x] = 0u;
    __syncthreads();
    int local = 0;
    const int kernel_id = map_thread(plan, (int)blockIdx.x, (int)threadIdx.x, &local);
    // A side whose partner has no barriers can keep the hardware barrier: s_barrier counts the waves
    // of the workgroup that are still alive, the partner's waves never take part and leave when
    // they are done -- so this side's FIRST barrier waits until they have left.  That is free for a
    // side that synchronises only in its epilogue (the split-K GEMMs, the convolutions) and would
    // serialise the two sides if the barrier sat in the K loop: such a side (LOOP_BARRIERS), and
    // both sides whenever both synchronise, get barriers of their own (the LDS arrival counters).
    // A side with a barrier in its K loop would pay one LDS-counter barrier per step; if its partner
    // can yield (see JoinSync) it keeps the hardware barrier and the partner's waves take part in the
    // first few of them.
    if (kernel_id == 0) {
        if constexpr (joins_barriers<A, B>) A::run((int)blockIdx.x, local, ss.a, I1, F1, O1, BlockSync{});
        else if constexpr (joins_barriers<B, A>) A::run((int)blockIdx.x, local, ss.a, I1, F1, O1, JoinSync{});
        else if constexpr (!B::HAS_BARRIERS && !loop_barriers<A>::value) A::run((int)blockIdx.x, local, ss.a, I1, F1, O1, BlockSync{});
        else A::run((int)blockIdx.x, local, ss.a, I1, F1, O1, GroupSync{&ss.arrive[0], (unsigned)(round_up(A::THREADS, kWaveSize) / kWaveSize), 0u});
    } else if (kernel_id == 1) {
        if constexpr (joins_barriers<B, A>) B::run((int)blockIdx.x, local, ss.b, I2, F2, O2, BlockSync{});
        else if constexpr (joins_barriers<A, B>) B::run((int)blockIdx.x, local, ss.b, I2, F2, O2, JoinSync{});
        else if constexpr (!A::HAS_BARRIERS && !loop_barriers<B>::value) B::run((int)blockIdx.x, local, ss.b, I2, F2, O2, BlockSync{});
        else B::run((int)blockIdx.x, local, ss.b, I2, F2, O2, GroupSync{&ss.arrive[1], (unsigned)(round_up(B::THREADS, kWaveSize) / kWaveSize), 0u});
    }
}

// ---- registry ---------------------------------------------------------------------------
enum KernelKind : int { kSingle = 0, kBfuse = 1, kHfuse = 2, kBfuseRt = 3 };

struct TensorDesc {
    int shape[4];   // padded with 1s, as the reference's macro.h tables (macro_h.py:28-42)
    int elem_bytes;
};

struct KernelEntry {
    std::string name;
    const void* func;       // host-side handle of the __global__ function
    int kind;
    unsigned grid[3], block[3];
    bool has_barriers;
    TensorDesc io[3];       // single: I, F, O
    std::string side[2];    // fused: names of the two standalone kernels
    int pattern, p0, p1;    // bfuse: dispatch pattern and its parameters
    unsigned (*read_sync_timeouts)();  // device counter of GroupSync give-ups in this module (read and reset)
    int (*set_spin_limit)(unsigned);   // polls a side barrier of this module makes before it gives up (0 = ok)
    int (*set_plan)(const BlockPlan*); // bfuse_rt: per-kernel hook called when a plan is installed (0 = ok); the plan itself travels as a kernel argument
};

// per-module (translation unit) access to its own copies of the side-barrier device variables
struct ModuleHooks {
    unsigned (*read_sync_timeouts)();
    int (*set_spin_limit)(unsigned);
};

std::vector<KernelEntry>& registry();

struct Registrar {
    explicit Registrar(const KernelEntry& e) { registry().push_back(e); }
};

template <class Op>
KernelEntry make_single_entry(const char* name, const void* func, TensorDesc i, TensorDesc f, TensorDesc o,
                              const ModuleHooks& hooks)
{
    KernelEntry e{};
    e.name = name;
    e.func = func;
    e.kind = kSingle;
    e.grid[0] = Op::GRID.size(); e.grid[1] = 1; e.grid[2] = 1;
    e.block[0] = Op::THREADS; e.block[1] = 1; e.block[2] = 1;
    e.has_barriers = Op::HAS_BARRIERS;
    e.io[0] = i; e.io[1] = f; e.io[2] = o;
    e.read_sync_timeouts = hooks.read_sync_timeouts;
    e.set_spin_limit = hooks.set_spin_limit;
    return e;
}

template <class Pair>
KernelEntry make_fused_entry(const char* name, const void* func, int kind, const char* k1, const char* k2,
                             bool barriers, int pattern, int p0, int p1, const ModuleHooks& hooks)
{
    KernelEntry e{};
    e.name = name;
    e.func = func;
    e.kind = kind;
    e.grid[0] = Pair::GRID; e.grid[1] = 1; e.grid[2] = 1;
    e.block[0] = Pair::THREADS; e.block[1] = 1; e.block[2] = 1;
    e.has_barriers = barriers;
    e.side[0] = k1; e.side[1] = k2;
    e.pattern = pattern; e.p0 = p0; e.p1 = p1;
    e.read_sync_timeouts = hooks.read_sync_timeouts;
    e.set_spin_limit = hooks.set_spin_limit;
    return e;
}

}  // namespace bfuse

// ---- definition macros (one extern "C" device symbol per kernel, reference naming) -----
#define BFUSE_MODULE_PROLOGUE()                                                                     \
    static unsigned bfuse_module_read_sync_timeouts()                                               \
    {                                                                                               \
        unsigned v = 0, z = 0;                                                                      \
        if (hipMemcpyFromSymbol(&v, HIP_SYMBOL(bfuse::g_sync_timeouts), sizeof(v)) != hipSuccess) return ~0u; \
        if (v) (void)hipMemcpyToSymbol(HIP_SYMBOL(bfuse::g_sync_timeouts), &z, sizeof(z));          \
        return v;                                                                                   \
    }                                                                                               \
    static int bfuse_module_set_spin_limit(unsigned polls)                                          \
    {                                                                                               \
        return hipMemcpyToSymbol(HIP_SYMBOL(bfuse::g_sync_spin_limit), &polls, sizeof(polls)) == hipSuccess ? 0 : -1; \
    }                                                                                               \
    static const bfuse::ModuleHooks bfuse_module_hooks{&bfuse_module_read_sync_timeouts, &bfuse_module_set_spin_limit};

#define BFUSE_KERNEL(NAME, OP, IDESC, FDESC, ODESC)                                                  \
    extern "C" __global__ __launch_bounds__(OP::THREADS, bfuse::kMinWavesPerEu) void NAME(const void* __restrict__ I,       \
                                                                   const void* __restrict__ F,       \
                                                                   void* __restrict__ O)             \
    {                                                                                               \
        bfuse::single_body<OP>(I, F, O);                                                            \
    }                                                                                               \
    static bfuse::Registrar reg_##NAME(bfuse::make_single_entry<OP>(                                \
        #NAME, (const void*)&NAME, bfuse::TensorDesc IDESC, bfuse::TensorDesc FDESC, bfuse::TensorDesc ODESC, \
        bfuse_module_hooks));

#define BFUSE_BFUSE_KERNEL(K1, OP1, K2, OP2, SUFFIX, PATTERN, P0, P1)                                \
    extern "C" __global__ __launch_bounds__((bfuse::BfusePair<OP1, OP2, PATTERN, P0, P1>::THREADS), bfuse::kMinWavesPerEu)  \
    void K1##_##K2##_fused_bfuse##SUFFIX(const void* __restrict__ I1, const void* __restrict__ F1,   \
                                         void* __restrict__ O1, const void* __restrict__ I2,         \
                                         const void* __restrict__ F2, void* __restrict__ O2)         \
    {                                                                                               \
        bfuse::bfuse_body<OP1, OP2, PATTERN, P0, P1>(I1, F1, O1, I2, F2, O2);                        \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_bfuse##SUFFIX(                                         \
        bfuse::make_fused_entry<bfuse::BfusePair<OP1, OP2, PATTERN, P0, P1>>(                        \
            #K1 "_" #K2 "_fused_bfuse" #SUFFIX, (const void*)&K1##_##K2##_fused_bfuse##SUFFIX,       \
            bfuse::kBfuse, #K1, #K2, OP1::HAS_BARRIERS || OP2::HAS_BARRIERS, PATTERN, P0, P1,        \
            bfuse_module_hooks));

#define BFUSE_HFUSE_KERNEL(K1, OP1, K2, OP2)                                                         \
    extern "C" __global__ __launch_bounds__((bfuse::HfusePair<OP1, OP2>::THREADS), bfuse::kMinWavesPerEu)                  \
    void K1##_##K2##_fused_hfuse(const void* __restrict__ I1, const void* __restrict__ F1,           \
                                 void* __restrict__ O1, const void* __restrict__ I2,                 \
                                 const void* __restrict__ F2, void* __restrict__ O2)                 \
    {                                                                                               \
        bfuse::hfuse_body<OP1, OP2>(I1, F1, O1, I2, F2, O2);                                         \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_hfuse(                                                 \
        bfuse::make_fused_entry<bfuse::HfusePair<OP1, OP2>>(                                         \
            #K1 "_" #K2 "_fused_hfuse", (const void*)&K1##_##K2##_fused_hfuse, bfuse::kHfuse, #K1, #K2, \
            OP1::HAS_BARRIERS || OP2::HAS_BARRIERS, -1, 0, 0, bfuse_module_hooks));

// The plan is the kernel's seventh argument, passed by value: it arrives with the kernel arguments
// (scalar loads that hit at once) instead of costing every workgroup a chain of dependent loads
// from device memory before it can start.  The host keeps the installed plan and appends it at launch.
#define BFUSE_BFUSE_RT_KERNEL(K1, OP1, K2, OP2)                                                      \
    extern "C" __global__ __launch_bounds__((bfuse::BfuseRtPair<OP1, OP2>::THREADS), bfuse::kMinWavesPerEu)                 \
    void K1##_##K2##_fused_bfuse_rt(const void* __restrict__ I1, const void* __restrict__ F1,        \
                                    void* __restrict__ O1, const void* __restrict__ I2,              \
                                    const void* __restrict__ F2, void* __restrict__ O2,              \
                                    const bfuse::BlockPlan plan)                                     \
    {                                                                                               \
        bfuse::bfuse_rt_body<OP1, OP2>(plan, I1, F1, O1, I2, F2, O2);                                \
    }                                                                                               \
    static int set_plan_##K1##_##K2##_rt(const bfuse::BlockPlan*) { return 0; }                      \
    static bfuse::Registrar reg_##K1##_##K2##_bfuse_rt([] {                                          \
        bfuse::KernelEntry e = bfuse::make_fused_entry<bfuse::BfuseRtPair<OP1, OP2>>(                \
            #K1 "_" #K2 "_fused_bfuse_rt", (const void*)&K1##_##K2##_fused_bfuse_rt, bfuse::kBfuseRt, #K1, #K2, \
            true, -1, 0, 0, bfuse_module_hooks);                                       \
        e.set_plan = &set_plan_##K1##_##K2##_rt;                                                     \
        return e;                                                                                   \
    }());
