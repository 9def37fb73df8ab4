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
//
// The reference's emitter fuses a LIST of kernels (horizontal-fuser/src/Algorithms.cc:23-35,
// 540-566: the maps take any number of grids; Matchers.cc:523-602 concatenates the parameter
// lists).  The pair templates below are the tuned forms the five headline pairs use; the
// *_group templates further down are the same three fusions over up to kMaxKernels operators,
// with 3 x n pointers in operator order.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
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


// ---- fusions of more than two operators ----------------------------------------------------
struct SidePtrs {
    const void* i;
    const void* f;
    void* o;
};

// LDS of the operators as a union (block fusion: one operator per workgroup) or one after the
// other (horizontal fusion: all of them in every workgroup), Tools.cc:219-251
template <class... Ops>
union SmemUnion;
template <class A>
union SmemUnion<A> {
    typename A::Smem head;
};
template <class A, class... R>
union SmemUnion<A, R...> {
    typename A::Smem head;
    SmemUnion<R...> tail;
};
template <class... Ops>
struct SmemSum;
template <class A>
struct SmemSum<A> {
    typename A::Smem head;
};
template <class A, class... R>
struct SmemSum<A, R...> {
    typename A::Smem head;
    SmemSum<R...> tail;
};
template <int K, class U>
__device__ __forceinline__ auto& smem_at(U& u)
{
    if constexpr (K == 0) return u.head;
    else return smem_at<K - 1>(u.tail);
}

template <class... Ops>
struct GroupDims {
    static constexpr int N = sizeof...(Ops);
    static_assert(N >= 2 && N <= kMaxKernels, "a fusion takes two to kMaxKernels operators");
    static_assert(((Ops::THREADS % kWaveSize == 0) && ...), "block sizes must be whole waves");
    static constexpr LaunchDims dims[N] = {{Ops::GRID, Ops::BLOCK}...};
    static constexpr int WIDEST = std::max({Ops::THREADS...});
    static constexpr int SUM_THREADS = (round_up(Ops::THREADS, kWaveSize) + ...);
    static constexpr int SUM_GRID = (Ops::GRID.size() + ...);
    static constexpr int MAX_GRID = std::max({Ops::GRID.size()...});
    static constexpr int BARRIER_SIDES = (int(Ops::HAS_BARRIERS) + ...);
};

template <int PATTERN, int P0, int P1, class... Ops>
struct BfuseGroup : GroupDims<Ops...> {
    using D = GroupDims<Ops...>;
    static constexpr BlockPlan plan() { return make_block_plan(PATTERN, D::N, D::dims, P0, P1); }
    static constexpr int THREADS = D::WIDEST;
    static constexpr int GRID = D::SUM_GRID;
};

template <int PATTERN, int P0, int P1, class... Ops, int... K>
__device__ __forceinline__ void bfuse_group_body(const SidePtrs (&p)[sizeof...(Ops)], std::integer_sequence<int, K...>)
{
    __shared__ SmemUnion<Ops...> su;
    constexpr BlockPlan plan = BfuseGroup<PATTERN, P0, P1, Ops...>::plan();
    int virt = 0;
    const int kernel_id = map_block(plan, (int)blockIdx.x, &virt);
    const int tid = (int)threadIdx.x;
    // exactly one operator's body runs in a workgroup; waves past its block size leave
    ((kernel_id == K && tid < Ops::THREADS ? (Ops::run(virt, tid, smem_at<K>(su), p[K].i, p[K].f, p[K].o, BlockSync{}), 0) : 0), ...);
}

template <class... Ops>
struct BfuseRtGroup : GroupDims<Ops...> {
    static constexpr int THREADS = GroupDims<Ops...>::WIDEST;
    static constexpr int GRID = GroupDims<Ops...>::SUM_GRID;
};

template <int K, int T, class Op>
__device__ __forceinline__ void rt_run_side(int virt, int tid, typename Op::Smem& sm, const SidePtrs& p, unsigned int* arrive)
{
    // see bfuse_rt_body: an operator narrower than the workgroup synchronises over its own waves
    if constexpr (Op::THREADS == T) Op::run(virt, tid, sm, p.i, p.f, p.o, BlockSync{});
    else Op::run(virt, tid, sm, p.i, p.f, p.o, GroupSync{arrive, (unsigned)(Op::THREADS / kWaveSize), 0u});
}

template <class... Ops, int... K>
__device__ __forceinline__ void bfuse_rt_group_body(const BlockPlan& plan, const SidePtrs (&p)[sizeof...(Ops)],
                                                    std::integer_sequence<int, K...>)
{
    constexpr int N = sizeof...(Ops);
    struct Shrd {
        SmemUnion<Ops...> u;
        unsigned int arrive[3][N];   // three sets in rotation, as in bfuse_rt_body
    };
    __shared__ Shrd sh;
    constexpr int T = BfuseRtGroup<Ops...>::THREADS;
    const int tid = (int)threadIdx.x;
    const int total = plan.fused_grid;
    if (tid < 3 * N) (&sh.arrive[0][0])[tid] = 0u;
    int set = 0;
    for (int id = (int)blockIdx.x; id < total; id += (int)gridDim.x) {
        const int next = set == 2 ? 0 : set + 1;
        if (tid < N) sh.arrive[next][tid] = 0u;
        __syncthreads();
        int virt = 0;
        const int kernel_id = map_block(plan, id, &virt);
        ((kernel_id == K && tid < Ops::THREADS ? (rt_run_side<K, T, Ops>(virt, tid, smem_at<K>(sh.u), p[K], &sh.arrive[set][K]), 0) : 0), ...);
        set = next;
    }
}

template <class... Ops>
struct HfuseGroup : GroupDims<Ops...> {
    using D = GroupDims<Ops...>;
    static constexpr ThreadPlan plan() { return plan_threads(D::N, D::dims, kWaveSize); }
    static constexpr int THREADS = D::SUM_THREADS;
    static constexpr int GRID = D::MAX_GRID;
};

template <int BARRIER_SIDES, class Op>
__device__ __forceinline__ void hfuse_run_side(int local, typename Op::Smem& sm, const SidePtrs& p, unsigned int* arrive)
{
    // The only side that synchronises keeps the hardware barrier unless the barrier sits in its main
    // loop (its first barrier waits until the other sides' waves have left, see hfuse_body); every
    // other synchronising side meets on its own LDS arrival counter.
    constexpr bool alone = BARRIER_SIDES - int(Op::HAS_BARRIERS) == 0;
    if constexpr (alone && !loop_barriers<Op>::value) Op::run((int)blockIdx.x, local, sm, p.i, p.f, p.o, BlockSync{});
    else Op::run((int)blockIdx.x, local, sm, p.i, p.f, p.o, GroupSync{arrive, (unsigned)(round_up(Op::THREADS, kWaveSize) / kWaveSize), 0u});
}

template <class... Ops, int... K>
__device__ __forceinline__ void hfuse_group_body(const SidePtrs (&p)[sizeof...(Ops)], std::integer_sequence<int, K...>)
{
    constexpr int N = sizeof...(Ops);
    struct ShrdSum {
        SmemSum<Ops...> s;
        unsigned int arrive[N];
    };
    __shared__ ShrdSum ss;
    constexpr ThreadPlan plan = HfuseGroup<Ops...>::plan();
    if (threadIdx.x < N) ss.arrive[threadIdx.x] = 0u;
    __syncthreads();
    int local = 0;
    const int kernel_id = map_thread(plan, (int)blockIdx.x, (int)threadIdx.x, &local);
    ((kernel_id == K ? (hfuse_run_side<GroupDims<Ops...>::BARRIER_SIDES, Ops>(local, smem_at<K>(ss.s), p[K], &ss.arrive[K]), 0) : 0), ...);
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
    int n_sides;            // fused: how many standalone kernels it runs (2 .. kMaxKernels)
    std::string side[kMaxKernels];   // fused: their names, in pointer order
    int pattern, p0, p1;    // bfuse: dispatch pattern and its parameters
    unsigned (*read_sync_timeouts)();  // device counter of GroupSync give-ups in this module (read and reset)
    int (*set_spin_limit)(unsigned);   // polls a side barrier of this module makes before it gives up (0 = ok)
    int (*set_plan)(const BlockPlan*); // bfuse_rt: per-kernel hook called when a plan is installed (0 = ok); the plan itself travels as a kernel argument
    const char* op_type = "";          // single: the operator's C++ type, spelled so that it can be compiled again
    int smem_bytes = -1;               // single: sizeof(Op::Smem), the LDS the operator's body declares
    bool matrix_cores = false;         // single: the operator declares MATRIX_CORES (its inner loop is a stream of MFMAs)
};

template <class Op, class = void>
struct UsesMatrixCores : std::false_type {};
template <class Op>
struct UsesMatrixCores<Op, std::void_t<decltype(Op::MATRIX_CORES)>> : std::bool_constant<Op::MATRIX_CORES> {};

// The operator type as the compiler spells it, every template argument written out
// ("bfuse::GemmF32Dma<512, 768, 768, 32, 48, 4, 0, 3>"): what a module of fused kernels built later for a
// pair of registered kernels names its sides by.
template <class Op>
const char* op_type_name()
{
    const char* pretty = __PRETTY_FUNCTION__;        // "... [Op = <type>]"
    static const std::string name = [pretty] {
        const std::string f = pretty;
        const size_t a = f.find("Op = "), b = f.rfind(']');
        return (a == std::string::npos || b == std::string::npos || b < a + 5) ? std::string() : f.substr(a + 5, b - a - 5);
    }();
    return name.c_str();
}

// per-module (translation unit) access to its own copies of the side-barrier device variables
struct ModuleHooks {
    unsigned (*read_sync_timeouts)();
    int (*set_spin_limit)(unsigned);
};

std::vector<KernelEntry>& registry();

// Adds an entry to the registry.  A module of fused kernels built against other headers than the library it is
// loaded into would hand over entries of another layout: the size travels with the entry and such entries are
// refused (bfuse_load_kernels then fails).
void register_kernel(const KernelEntry& e, size_t entry_size);

struct Registrar {
    explicit Registrar(const KernelEntry& e) { register_kernel(e, sizeof(KernelEntry)); }
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
    e.op_type = op_type_name<Op>();
    e.smem_bytes = (int)sizeof(typename Op::Smem);
    e.matrix_cores = UsesMatrixCores<Op>::value;
    return e;
}

template <class Pair>
KernelEntry make_group_entry(const char* name, const void* func, int kind, std::initializer_list<const char*> sides,
                             bool barriers, int pattern, int p0, int p1, const ModuleHooks& hooks)
{
    KernelEntry e{};
    e.name = name;
    e.func = func;
    e.kind = kind;
    e.grid[0] = Pair::GRID; e.grid[1] = 1; e.grid[2] = 1;
    e.block[0] = Pair::THREADS; e.block[1] = 1; e.block[2] = 1;
    e.has_barriers = barriers;
    e.n_sides = 0;
    for (const char* k : sides) e.side[e.n_sides++] = k;
    e.pattern = pattern; e.p0 = p0; e.p1 = p1;
    e.read_sync_timeouts = hooks.read_sync_timeouts;
    e.set_spin_limit = hooks.set_spin_limit;
    return e;
}

template <class Pair>
KernelEntry make_fused_entry(const char* name, const void* func, int kind, const char* k1, const char* k2,
                             bool barriers, int pattern, int p0, int p1, const ModuleHooks& hooks)
{
    return make_group_entry<Pair>(name, func, kind, {k1, k2}, barriers, pattern, p0, p1, hooks);
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

namespace bfuse {
// The waves per SIMD a kernel is compiled for (the register budget of its waves: 512 / waves): kMinWavesPerEu,
// unless one of its operators says that it needs more of the register file (MIN_WAVES_PER_EU).  A fused kernel
// takes the smallest of its sides': it holds the registers of the side that needs most.
template <class Op, class = void>
struct min_waves_of : std::integral_constant<int, kMinWavesPerEu> {};
template <class Op>
struct min_waves_of<Op, std::void_t<decltype(Op::MIN_WAVES_PER_EU)>> : std::integral_constant<int, Op::MIN_WAVES_PER_EU> {};
template <class... Ops>
constexpr int min_waves()
{
    int m = kMinWavesPerEu;
    ((m = min_waves_of<Ops>::value < m ? min_waves_of<Ops>::value : m), ...);
    return m;
}
}  // namespace bfuse

#define BFUSE_KERNEL(NAME, OP, IDESC, FDESC, ODESC)                                                  \
    extern "C" __global__ __launch_bounds__(OP::THREADS, bfuse::min_waves<OP>()) void NAME(const void* __restrict__ I,       \
                                                                   const void* __restrict__ F,       \
                                                                   void* __restrict__ O)             \
    {                                                                                               \
        bfuse::single_body<OP>(I, F, O);                                                            \
    }                                                                                               \
    static bfuse::Registrar reg_##NAME(bfuse::make_single_entry<OP>(                                \
        #NAME, (const void*)&NAME, bfuse::TensorDesc IDESC, bfuse::TensorDesc FDESC, bfuse::TensorDesc ODESC, \
        bfuse_module_hooks));

#define BFUSE_BFUSE_KERNEL(K1, OP1, K2, OP2, SUFFIX, PATTERN, P0, P1)                                \
    extern "C" __global__ __launch_bounds__((bfuse::BfusePair<OP1, OP2, PATTERN, P0, P1>::THREADS), (bfuse::min_waves<OP1, OP2>()))  \
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
    extern "C" __global__ __launch_bounds__((bfuse::HfusePair<OP1, OP2>::THREADS), (bfuse::min_waves<OP1, OP2>()))                  \
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
    extern "C" __global__ __launch_bounds__((bfuse::BfuseRtPair<OP1, OP2>::THREADS), (bfuse::min_waves<OP1, OP2>()))                 \
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

// ---- three and four operators: 3 x n pointers in operator order, names joined as the reference's
//      emitter joins them (Contexts.cc:56-92) ---------------------------------------------------
#define BFUSE_PTRS3(N) const void* __restrict__ I##N, const void* __restrict__ F##N, void* __restrict__ O##N
#define BFUSE_SIDE(N) {I##N, F##N, O##N}

#define BFUSE_BFUSE3_KERNEL(K1, OP1, K2, OP2, K3, OP3, SUFFIX, PATTERN, P0, P1)                      \
    using grp_##K1##_##K2##_##K3##_bfuse##SUFFIX = bfuse::BfuseGroup<PATTERN, P0, P1, OP1, OP2, OP3>; \
    extern "C" __global__ __launch_bounds__(grp_##K1##_##K2##_##K3##_bfuse##SUFFIX::THREADS, bfuse::kMinWavesPerEu) \
    void K1##_##K2##_##K3##_fused_bfuse##SUFFIX(BFUSE_PTRS3(1), BFUSE_PTRS3(2), BFUSE_PTRS3(3))      \
    {                                                                                               \
        const bfuse::SidePtrs p[3] = {BFUSE_SIDE(1), BFUSE_SIDE(2), BFUSE_SIDE(3)};                 \
        bfuse::bfuse_group_body<PATTERN, P0, P1, OP1, OP2, OP3>(p, std::make_integer_sequence<int, 3>{}); \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_##K3##_bfuse##SUFFIX(                                  \
        bfuse::make_group_entry<grp_##K1##_##K2##_##K3##_bfuse##SUFFIX>(                             \
            #K1 "_" #K2 "_" #K3 "_fused_bfuse" #SUFFIX, (const void*)&K1##_##K2##_##K3##_fused_bfuse##SUFFIX, \
            bfuse::kBfuse, {#K1, #K2, #K3}, OP1::HAS_BARRIERS || OP2::HAS_BARRIERS || OP3::HAS_BARRIERS, \
            PATTERN, P0, P1, bfuse_module_hooks));

#define BFUSE_BFUSE4_KERNEL(K1, OP1, K2, OP2, K3, OP3, K4, OP4, SUFFIX, PATTERN, P0, P1)             \
    using grp_##K1##_##K2##_##K3##_##K4##_bfuse##SUFFIX = bfuse::BfuseGroup<PATTERN, P0, P1, OP1, OP2, OP3, OP4>; \
    extern "C" __global__ __launch_bounds__(grp_##K1##_##K2##_##K3##_##K4##_bfuse##SUFFIX::THREADS, bfuse::kMinWavesPerEu) \
    void K1##_##K2##_##K3##_##K4##_fused_bfuse##SUFFIX(BFUSE_PTRS3(1), BFUSE_PTRS3(2), BFUSE_PTRS3(3), BFUSE_PTRS3(4)) \
    {                                                                                               \
        const bfuse::SidePtrs p[4] = {BFUSE_SIDE(1), BFUSE_SIDE(2), BFUSE_SIDE(3), BFUSE_SIDE(4)};  \
        bfuse::bfuse_group_body<PATTERN, P0, P1, OP1, OP2, OP3, OP4>(p, std::make_integer_sequence<int, 4>{}); \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_##K3##_##K4##_bfuse##SUFFIX(                           \
        bfuse::make_group_entry<grp_##K1##_##K2##_##K3##_##K4##_bfuse##SUFFIX>(                      \
            #K1 "_" #K2 "_" #K3 "_" #K4 "_fused_bfuse" #SUFFIX,                                      \
            (const void*)&K1##_##K2##_##K3##_##K4##_fused_bfuse##SUFFIX, bfuse::kBfuse, {#K1, #K2, #K3, #K4}, \
            OP1::HAS_BARRIERS || OP2::HAS_BARRIERS || OP3::HAS_BARRIERS || OP4::HAS_BARRIERS, PATTERN, P0, P1, \
            bfuse_module_hooks));

#define BFUSE_HFUSE3_KERNEL(K1, OP1, K2, OP2, K3, OP3)                                               \
    using grp_##K1##_##K2##_##K3##_hfuse = bfuse::HfuseGroup<OP1, OP2, OP3>;                         \
    extern "C" __global__ __launch_bounds__(grp_##K1##_##K2##_##K3##_hfuse::THREADS, bfuse::kMinWavesPerEu) \
    void K1##_##K2##_##K3##_fused_hfuse(BFUSE_PTRS3(1), BFUSE_PTRS3(2), BFUSE_PTRS3(3))              \
    {                                                                                               \
        const bfuse::SidePtrs p[3] = {BFUSE_SIDE(1), BFUSE_SIDE(2), BFUSE_SIDE(3)};                 \
        bfuse::hfuse_group_body<OP1, OP2, OP3>(p, std::make_integer_sequence<int, 3>{});            \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_##K3##_hfuse(bfuse::make_group_entry<grp_##K1##_##K2##_##K3##_hfuse>( \
        #K1 "_" #K2 "_" #K3 "_fused_hfuse", (const void*)&K1##_##K2##_##K3##_fused_hfuse, bfuse::kHfuse,  \
        {#K1, #K2, #K3}, OP1::HAS_BARRIERS || OP2::HAS_BARRIERS || OP3::HAS_BARRIERS, -1, 0, 0, bfuse_module_hooks));

#define BFUSE_HFUSE4_KERNEL(K1, OP1, K2, OP2, K3, OP3, K4, OP4)                                      \
    using grp_##K1##_##K2##_##K3##_##K4##_hfuse = bfuse::HfuseGroup<OP1, OP2, OP3, OP4>;             \
    extern "C" __global__ __launch_bounds__(grp_##K1##_##K2##_##K3##_##K4##_hfuse::THREADS, bfuse::kMinWavesPerEu) \
    void K1##_##K2##_##K3##_##K4##_fused_hfuse(BFUSE_PTRS3(1), BFUSE_PTRS3(2), BFUSE_PTRS3(3), BFUSE_PTRS3(4)) \
    {                                                                                               \
        const bfuse::SidePtrs p[4] = {BFUSE_SIDE(1), BFUSE_SIDE(2), BFUSE_SIDE(3), BFUSE_SIDE(4)};  \
        bfuse::hfuse_group_body<OP1, OP2, OP3, OP4>(p, std::make_integer_sequence<int, 4>{});       \
    }                                                                                               \
    static bfuse::Registrar reg_##K1##_##K2##_##K3##_##K4##_hfuse(                                   \
        bfuse::make_group_entry<grp_##K1##_##K2##_##K3##_##K4##_hfuse>(                              \
            #K1 "_" #K2 "_" #K3 "_" #K4 "_fused_hfuse", (const void*)&K1##_##K2##_##K3##_##K4##_fused_hfuse, \
            bfuse::kHfuse, {#K1, #K2, #K3, #K4},                                                     \
            OP1::HAS_BARRIERS || OP2::HAS_BARRIERS || OP3::HAS_BARRIERS || OP4::HAS_BARRIERS, -1, 0, 0, \
            bfuse_module_hooks));

// run-time plan over three operators: the plan is the kernel's last argument, as for pairs
#define BFUSE_BFUSE_RT3_KERNEL(K1, OP1, K2, OP2, K3, OP3)                                            \
    using grp_##K1##_##K2##_##K3##_bfuse_rt = bfuse::BfuseRtGroup<OP1, OP2, OP3>;                    \
    extern "C" __global__ __launch_bounds__(grp_##K1##_##K2##_##K3##_bfuse_rt::THREADS, bfuse::kMinWavesPerEu) \
    void K1##_##K2##_##K3##_fused_bfuse_rt(BFUSE_PTRS3(1), BFUSE_PTRS3(2), BFUSE_PTRS3(3), const bfuse::BlockPlan plan) \
    {                                                                                               \
        const bfuse::SidePtrs p[3] = {BFUSE_SIDE(1), BFUSE_SIDE(2), BFUSE_SIDE(3)};                 \
        bfuse::bfuse_rt_group_body<OP1, OP2, OP3>(plan, p, std::make_integer_sequence<int, 3>{});   \
    }                                                                                               \
    static int set_plan_##K1##_##K2##_##K3##_rt(const bfuse::BlockPlan*) { return 0; }               \
    static bfuse::Registrar reg_##K1##_##K2##_##K3##_bfuse_rt([] {                                   \
        bfuse::KernelEntry e = bfuse::make_group_entry<grp_##K1##_##K2##_##K3##_bfuse_rt>(           \
            #K1 "_" #K2 "_" #K3 "_fused_bfuse_rt", (const void*)&K1##_##K2##_##K3##_fused_bfuse_rt, bfuse::kBfuseRt, \
            {#K1, #K2, #K3}, true, -1, 0, 0, bfuse_module_hooks);                                    \
        e.set_plan = &set_plan_##K1##_##K2##_##K3##_rt;                                              \
        return e;                                                                                   \
    }());
