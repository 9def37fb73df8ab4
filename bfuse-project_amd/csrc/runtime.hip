// libbfuse_rt: the C ABI declared in include/bfuse_rt.h over the HIP runtime.
// Host-side counterpart of the reference's generated harness
// (test-utils/test-suite-files/operation_cu.py, main_cc.py, utils_cc.py).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <dlfcn.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <map>
#include <vector>

#include "../../include/bfuse_rt.h"
#include "dispatch.h"
#include "fuse.h"

namespace bfuse {
std::vector<KernelEntry>& registry()
{
    static std::vector<KernelEntry> r;
    return r;
}

static int g_refused_entries = 0;   // entries of another layout (a module built against other headers)

void register_kernel(const KernelEntry& e, size_t entry_size)
{
    if (entry_size != sizeof(KernelEntry)) {
        ++g_refused_entries;
        return;
    }
    registry().push_back(e);
}
}  // namespace bfuse

using namespace bfuse;

static_assert(sizeof(bfuse_block_plan) == sizeof(BlockPlan), "C and C++ plan layouts must agree");
static_assert(sizeof(bfuse_thread_plan) == sizeof(ThreadPlan), "C and C++ plan layouts must agree");
static_assert(sizeof(bfuse_launch_dims) == sizeof(LaunchDims), "C and C++ dims layouts must agree");
static_assert(BFUSE_MAX_KERNELS == kMaxKernels && BFUSE_MAX_SEGMENTS == kMaxSegments, "limits must agree");

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(call)                                                                          \
    do {                                                                                       \
        hipError_t st_ = (call);                                                               \
        if (st_ != hipSuccess)                                                                 \
            return fail(BFUSE_ERR_HIP, "HIP error (%s:%d): %s: %s", __FILE__, __LINE__, #call, \
                        hipGetErrorString(st_));                                               \
    } while (0)

struct Side {
    void* buf[3] = {nullptr, nullptr, nullptr};  // I, F, O on the device
    size_t bytes[3] = {0, 0, 0};
    int elem[3] = {4, 4, 4};
    hipStream_t stream = nullptr;                // S1 / S2
    bool live = false;
};

struct State {
    bool inited = false;
    int device = -1;
    Side side[kMaxKernels];   // the harness functions use the first two; launch lists may use all
} g;

// 0 for a shape with a dimension below 1 (callers refuse empty tensors)
size_t shape_bytes(const int* s, int elem)
{
    for (int d = 0; d < 4; ++d)
        if (s[d] < 1) return 0;
    return (size_t)s[0] * s[1] * s[2] * s[3] * (size_t)elem;
}

// device memory and events that an early return must not leak
struct DevBuf {
    void* p = nullptr;
    ~DevBuf() { if (p) (void)hipFree(p); }
    template <class T> T* as() const { return static_cast<T*>(p); }
};
struct EventList {
    std::vector<hipEvent_t> v;
    explicit EventList(size_t n) : v(n, nullptr) {}
    ~EventList() { for (auto e : v) if (e) (void)hipEventDestroy(e); }
};

// Fused kernels launched since the last synchronisation whose side barriers can give up, and code
// objects launched from: their give-up counters are read at the next synchronisation, whichever
// entry point performs it.
std::vector<const void*> g_pending_fused;
std::vector<int> g_pending_modules;

// ---- staging memory of bfuse_map_blocks_device_noalloc ----------------------------------------
// A fixed device array (kernel and block index of up to kNoAllocMaxIds fused blocks) that lives as
// long as the process does.  `scratch` is only the host-side name of the symbol: the address a
// kernel or a copy can use is looked up once per device (scratch_of) and kept.
constexpr int kNoAllocMaxIds = BFUSE_NOALLOC_MAX_IDS;
static __device__ __align__(256) int scratch[2 * kNoAllocMaxIds];
constexpr int kMaxDevices = 64;
int* g_scratch_ptr[kMaxDevices] = {};

int scratch_of(int device, int** out);

int init_side(int idx, const int* I, const int* F, const int* O)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!I || !F || !O) return fail(BFUSE_ERR_ARG, "null shape");
    Side& s = g.side[idx];
    if (s.live) return fail(BFUSE_ERR_STATE, "kernel%d is already initialized", idx + 1);
    const int* shp[3] = {I, F, O};
    size_t bytes[3];
    for (int i = 0; i < 3; ++i) {
        bytes[i] = shape_bytes(shp[i], s.elem[i]);
        if (bytes[i] == 0) return fail(BFUSE_ERR_ARG, "tensor %d of kernel%d is empty or has a dimension below 1", i, idx + 1);
    }
    // all or nothing: a failure part-way leaves the side as it was
    DevBuf tmp[3];
    for (int i = 0; i < 3; ++i) HIP_TRY(hipMalloc(&tmp[i].p, bytes[i]));
    HIP_TRY(hipStreamCreate(&s.stream));
    for (int i = 0; i < 3; ++i) {
        s.buf[i] = tmp[i].p;
        tmp[i].p = nullptr;
        s.bytes[i] = bytes[i];
    }
    s.live = true;
    return BFUSE_OK;
}

int fini_side(int idx)
{
    Side& s = g.side[idx];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", idx + 1);
    HIP_TRY(hipStreamDestroy(s.stream));
    for (int i = 2; i >= 0; --i) {
        HIP_TRY(hipFree(s.buf[i]));
        s.buf[i] = nullptr;
    }
    s.live = false;
    return BFUSE_OK;
}

int check_shapes(int idx, const int* I, const int* F, const int* O)
{
    Side& s = g.side[idx];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", idx + 1);
    const int* shp[3] = {I, F, O};
    for (int i = 0; i < 3; ++i)
        if (!shp[i] || shape_bytes(shp[i], s.elem[i]) != s.bytes[i])
            return fail(BFUSE_ERR_ARG, "shape of tensor %d does not match initialize_kernel%d", i, idx + 1);
    return BFUSE_OK;
}

dim3 d3(const unsigned* v) { return dim3(v[0], v[1], v[2]); }

const KernelEntry* entry_of(const void* func)
{
    for (const auto& e : registry())
        if (e.func == func) return &e;
    return nullptr;
}

// The grid and block a caller passes must be the ones the kernel was built for: the bodies
// index memory from compile-time shapes, so any other launch shape would read or write out
// of bounds.
// plans currently installed in run-time-plan kernels (host copies, for launch validation)
std::map<const void*, BlockPlan>& installed_plans()
{
    static std::map<const void*, BlockPlan> m;
    return m;
}

int check_launch(const void* func, const unsigned* grid, const unsigned* block, int want_ptrs)
{
    if (!func || !grid || !block) return fail(BFUSE_ERR_ARG, "null launch argument");
    const KernelEntry* e = entry_of(func);
    if (!e) return fail(BFUSE_ERR_ARG, "func is not a kernel of this library");
    const int ptrs = e->kind == kSingle ? 3 : 3 * e->n_sides;
    if (ptrs != want_ptrs) return fail(BFUSE_ERR_ARG, "%s takes %d pointers, not %d", e->name.c_str(), ptrs, want_ptrs);
    if (e->kind == kBfuseRt) {
        // persistent workgroups stride over the plan's fused grid: any grid from 1 to that size covers it
        auto it = installed_plans().find(func);
        if (it == installed_plans().end()) return fail(BFUSE_ERR_STATE, "%s has no plan: call bfuse_set_plan first", e->name.c_str());
        for (int i = 0; i < 3; ++i)
            if (block[i] != e->block[i])
                return fail(BFUSE_ERR_ARG, "%s must be launched with block (%u,%u,%u)", e->name.c_str(), e->block[0], e->block[1], e->block[2]);
        if (grid[1] != 1 || grid[2] != 1 || grid[0] < 1 || grid[0] > (unsigned)it->second.fused_grid)
            return fail(BFUSE_ERR_ARG, "%s takes a 1-D grid of 1..%d workgroups", e->name.c_str(), it->second.fused_grid);
        return BFUSE_OK;
    }
    for (int i = 0; i < 3; ++i)
        if (grid[i] != e->grid[i] || block[i] != e->block[i])
            return fail(BFUSE_ERR_ARG, "%s must be launched with grid (%u,%u,%u) block (%u,%u,%u)", e->name.c_str(),
                        e->grid[0], e->grid[1], e->grid[2], e->block[0], e->block[1], e->block[2]);
    return BFUSE_OK;
}

// Buffers a single kernel touches must be at least as large as the shapes it was built for.
int check_side_fits(const void* func, int idx)
{
    const KernelEntry* e = entry_of(func);
    if (!e || e->kind != kSingle) return BFUSE_OK;
    const Side& s = g.side[idx];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", idx + 1);
    for (int i = 0; i < 3; ++i) {
        const size_t need = shape_bytes(e->io[i].shape, e->io[i].elem_bytes);
        if (s.bytes[i] < need)
            return fail(BFUSE_ERR_ARG, "%s needs %zu bytes for tensor %d, side %d holds %zu", e->name.c_str(), need, i,
                        idx + 1, s.bytes[i]);
    }
    return BFUSE_OK;
}

// `sides` (0-based, one per operator of the fused kernel) or nullptr for sides 0, 1, ...
int check_fused_fits(const void* func, const int* sides = nullptr)
{
    const KernelEntry* e = entry_of(func);
    if (!e || e->kind == kSingle) return fail(BFUSE_ERR_ARG, "not a fused kernel");
    for (int k = 0; k < e->n_sides; ++k) {
        const KernelEntry* sk = nullptr;
        for (const auto& c : registry())
            if (c.kind == kSingle && c.name == e->side[k]) sk = &c;
        if (!sk) return fail(BFUSE_ERR_ARG, "fused kernel %s names unknown side %s", e->name.c_str(), e->side[k].c_str());
        int rc = check_side_fits(sk->func, sides ? sides[k] : k);
        if (rc) return rc;
    }
    return BFUSE_OK;
}

int launch3(const void* func, const unsigned* grid, const unsigned* block, int idx, hipStream_t stream,
            hipEvent_t ev0 = nullptr, hipEvent_t ev1 = nullptr)
{
    Side& s = g.side[idx];
    void* args[3] = {&s.buf[0], &s.buf[1], &s.buf[2]};
    if (ev0 || ev1)
        HIP_TRY(hipExtLaunchKernel(func, d3(grid), d3(block), args, 0, stream, ev0, ev1, 0));
    else
        HIP_TRY(hipLaunchKernel(func, d3(grid), d3(block), args, 0, stream));
    return BFUSE_OK;
}

// A fused kernel over n sides (0-based indices, operator order): 3 x n pointers.
int launch_fused(const void* func, const unsigned* grid, const unsigned* block, int n, const int* sides, hipStream_t stream,
                 hipEvent_t ev0 = nullptr, hipEvent_t ev1 = nullptr)
{
    void* args[3 * kMaxKernels + 1] = {};
    for (int k = 0; k < n; ++k)
        for (int i = 0; i < 3; ++i) args[3 * k + i] = &g.side[sides[k]].buf[i];
    // a run-time-plan kernel takes its installed plan by value as its last argument
    auto it = installed_plans().find(func);
    if (it != installed_plans().end()) args[3 * n] = &it->second;
    bool known = false;
    for (const void* f : g_pending_fused) known = known || f == func;
    if (!known) g_pending_fused.push_back(func);
    if (ev0 || ev1)
        HIP_TRY(hipExtLaunchKernel(func, d3(grid), d3(block), args, 0, stream, ev0, ev1, 0));
    else
        HIP_TRY(hipLaunchKernel(func, d3(grid), d3(block), args, 0, stream));
    return BFUSE_OK;
}

int launch6(const void* func, const unsigned* grid, const unsigned* block, hipStream_t stream,
            hipEvent_t ev0 = nullptr, hipEvent_t ev1 = nullptr)
{
    const int sides[2] = {0, 1};
    return launch_fused(func, grid, block, 2, sides, stream, ev0, ev1);
}

// kernels of a loaded code object report give-ups of their side barriers in this device variable
// (the front end emits it next to every horizontally fused kernel)
const char* const kModuleSyncCounter = "bfuse_sync_timeouts";
std::vector<hipModule_t>& modules();

// Device synchronisation, launch errors, and the side barriers' give-up counters of everything
// launched since the last call: a barrier that gave up let its side run on unsynchronised, so
// outputs and timings of that launch are not to be trusted.
int sync_and_check()
{
    // Both lists are taken over first, so that whatever happens below they are empty afterwards: a
    // give-up of this launch set is reported by this call or not at all, never by a later, unrelated one.
    std::vector<const void*> fused;
    std::vector<int> mods;
    fused.swap(g_pending_fused);
    mods.swap(g_pending_modules);
    int rc = BFUSE_OK;
    auto note_hip = [&rc](hipError_t e, const char* what) {
        if (e != hipSuccess && rc == BFUSE_OK) rc = fail(BFUSE_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
        return e == hipSuccess;
    };
    note_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
    note_hip(hipGetLastError(), "launch");
    // every counter is read (and thereby reset) even after an error above; the first error is the one returned
    for (const void* f : fused) {
        const KernelEntry* e = entry_of(f);
        if (!e || !(e->kind == kHfuse || e->kind == kBfuseRt) || !e->read_sync_timeouts) continue;
        const unsigned n = e->read_sync_timeouts();   // reads and resets
        if (n && rc == BFUSE_OK) rc = fail(BFUSE_ERR_SYNC, "%s: %u side-barrier waits gave up", e->name.c_str(), n);
    }
    for (int id : mods) {
        if (id < 0 || id >= (int)modules().size() || !modules()[id]) continue;
        hipDeviceptr_t dp = nullptr;
        size_t bytes = 0;
        if (hipModuleGetGlobal(&dp, &bytes, modules()[id], kModuleSyncCounter) != hipSuccess || bytes != sizeof(unsigned)) {
            (void)hipGetLastError();   // a module without the counter has no side barriers
            continue;
        }
        unsigned n = 0, z = 0;
        if (!note_hip(hipMemcpy(&n, dp, sizeof(n), hipMemcpyDeviceToHost), "reading a code object's give-up counter")) continue;
        if (n) {
            note_hip(hipMemcpy(dp, &z, sizeof(z), hipMemcpyHostToDevice), "clearing a code object's give-up counter");
            if (rc == BFUSE_OK) rc = fail(BFUSE_ERR_SYNC, "code object %d: %u side-barrier waits gave up", id, n);
        }
    }
    return rc;
}

int validate_mode(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb,
                  const unsigned* gb, const unsigned* bb)
{
    int rc;
    switch (mode) {
        case BFUSE_MODE_KERNEL1:
            if ((rc = check_launch(fa, ga, ba, 3)) || (rc = check_side_fits(fa, 0))) return rc;
            break;
        case BFUSE_MODE_KERNEL2:
            if ((rc = check_launch(fa, ga, ba, 3)) || (rc = check_side_fits(fa, 1))) return rc;
            break;
        case BFUSE_MODE_PARALLEL:
        case BFUSE_MODE_SERIAL:
            if ((rc = check_launch(fa, ga, ba, 3)) || (rc = check_side_fits(fa, 0))) return rc;
            if ((rc = check_launch(fb, gb, bb, 3)) || (rc = check_side_fits(fb, 1))) return rc;
            break;
        case BFUSE_MODE_HFUSE:
        case BFUSE_MODE_BFUSE: {
            if ((rc = check_launch(fa, ga, ba, 6)) || (rc = check_fused_fits(fa))) return rc;
            const KernelEntry* e = entry_of(fa);
            if ((mode == BFUSE_MODE_HFUSE) != (e->kind == kHfuse))  // bfuse mode takes compile-time and run-time plans alike
                return fail(BFUSE_ERR_ARG, "%s is not a %s kernel", e->name.c_str(), mode == BFUSE_MODE_HFUSE ? "hfuse" : "bfuse");
            break;
        }
        default:
            return fail(BFUSE_ERR_ARG, "unknown mode %d", mode);
    }
    return BFUSE_OK;
}

// Enqueue one repetition. ev = {start_a, stop_a, start_b, stop_b} or nullptr.
int enqueue_mode(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb,
                 const unsigned* gb, const unsigned* bb, hipEvent_t* ev)
{
    hipEvent_t e0 = ev ? ev[0] : nullptr, e1 = ev ? ev[1] : nullptr, e2 = ev ? ev[2] : nullptr, e3 = ev ? ev[3] : nullptr;
    int rc;
    switch (mode) {
        case BFUSE_MODE_KERNEL1: return launch3(fa, ga, ba, 0, nullptr, e0, e1);
        case BFUSE_MODE_KERNEL2: return launch3(fa, ga, ba, 1, nullptr, e0, e1);
        case BFUSE_MODE_PARALLEL:
            if ((rc = launch3(fa, ga, ba, 0, g.side[0].stream, e0, e1))) return rc;
            return launch3(fb, gb, bb, 1, g.side[1].stream, e2, e3);
        case BFUSE_MODE_SERIAL:
            if ((rc = launch3(fa, ga, ba, 0, nullptr, e0, e1))) return rc;
            return launch3(fb, gb, bb, 1, nullptr, e2, e3);
        case BFUSE_MODE_HFUSE:
        case BFUSE_MODE_BFUSE: return launch6(fa, ga, ba, nullptr, e0, e1);
    }
    return fail(BFUSE_ERR_ARG, "unknown mode %d", mode);
}

__global__ void map_blocks_kernel(BlockPlan plan, int lo, int hi, int* kernel_out, int* virt_out)
{
    const int bid = lo + (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (bid < hi) {
        int v = -1;
        const int k = map_block(plan, bid, &v);
        kernel_out[bid - lo] = k;
        virt_out[bid - lo] = v;
    }
}

// Where the hardware put each workgroup: HW_ID (wave, SIMD, CU, shader array, shader engine) and
// XCC_ID of the wave that runs thread 0, plus a wall-clock stamp.  The workgroup spins for
// `hold` clock reads so that later workgroups cannot reuse its slot.
__global__ void placement_kernel(unsigned* hw_id, unsigned* xcc_id, unsigned long long* t_start, int hold)
{
    const unsigned long long t0 = wall_clock64();
    if (threadIdx.x == 0) {
        hw_id[blockIdx.x] = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_REG_HW_ID, 32 bits
        xcc_id[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | 20);   // HW_REG_XCC_ID, bits 3:0
        t_start[blockIdx.x] = t0;
    }
    for (int i = 0; i < hold; ++i)
        if (wall_clock64() == 0ull) hw_id[0] = 0u;  // never true: keeps the loop
}

__host__ __device__ inline unsigned long long splitmix64(unsigned long long x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
__host__ __device__ inline double u01(unsigned long long seed, unsigned long long i)  // in (0,1)
{
    const unsigned long long r = splitmix64(seed * 0xD1342543DE82EF95ull + i);
    return ((double)(r >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

std::vector<hipModule_t>& modules()
{
    static std::vector<hipModule_t> m;
    return m;
}

// Address of the staging array on `device` (which must be current): looked up on first use,
// then kept -- every device holds its own copy of the array at its own address.
int scratch_of(int device, int** out)
{
    if (device < 0 || device >= kMaxDevices) return fail(BFUSE_ERR_ARG, "device %d: at most %d devices are supported", device, kMaxDevices);
    if (!g_scratch_ptr[device]) {
        int* ptr = nullptr;
        hipError_t st = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (st != hipSuccess || !ptr)
            return fail(BFUSE_ERR_HIP, "hipGetSymbolAddress(staging array) on device %d: %s", device, hipGetErrorString(st));
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return BFUSE_OK;
}

}  // namespace

extern "C" {

const char* bfuse_last_error(void) { return g_err; }

static int load_env_modules();

int bfuse_init(int device)
{
    int n = 0;
    hipError_t st = hipGetDeviceCount(&n);
    if (st != hipSuccess || n <= 0)
        return fail(BFUSE_ERR_HIP, "no HIP device available (%s); this library has no CPU path",
                    st == hipSuccess ? "device count is 0" : hipGetErrorString(st));
    if (device < 0 || device >= n) return fail(BFUSE_ERR_ARG, "device %d out of range (0..%d)", device, n - 1);
    if (int rc = load_env_modules()) return rc;   // a module named in BFUSE_KERNEL_MODULES that does not load is an error here, not a shorter registry
    if (g.inited && device != g.device)
        for (int i = 0; i < kMaxKernels; ++i)
            if (g.side[i].live)
                return fail(BFUSE_ERR_STATE, "side %d holds buffers on device %d: finalize it before moving to device %d", i + 1, g.device, device);
    HIP_TRY(hipSetDevice(device));
    // the allocation-free entry point's staging array: its address on this device, looked up now so
    // that the entry point itself calls nothing that could allocate
    int* sp = nullptr;
    int rc = scratch_of(device, &sp);
    if (rc) return rc;
    g.device = device;
    g.inited = true;
    return BFUSE_OK;
}

int bfuse_shutdown(void)
{
    if (!g.inited) return BFUSE_OK;
    // nothing may still run on buffers or code objects that are about to go
    int rc = sync_and_check();
    if (rc && rc != BFUSE_ERR_SYNC) return rc;
    for (int i = 0; i < kMaxKernels; ++i)
        if (g.side[i].live) {
            int rc2 = fini_side(i);
            if (rc2) return rc2;
        }
    for (auto& m : modules())
        if (m) {
            HIP_TRY(hipModuleUnload(m));
            m = nullptr;
        }
    g.inited = false;
    return rc;
}

int bfuse_device_info(char* name, size_t name_len, int* cus, int* lds, int* wave)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, g.device));
    if (name && name_len) snprintf(name, name_len, "%s%s%s", p.name, p.name[0] ? " " : "", p.gcnArchName);
    if (cus) *cus = p.multiProcessorCount;
    if (lds) *lds = (int)p.sharedMemPerBlock;
    if (wave) *wave = p.warpSize;
    return BFUSE_OK;
}

int bfuse_device_memory(size_t* free_bytes, size_t* total_bytes)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    size_t f = 0, t = 0;
    HIP_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return BFUSE_OK;
}

// ---- index maps -------------------------------------------------------------------------
int bfuse_plan_threads(int n, const bfuse_launch_dims* k, int pad, bfuse_thread_plan* out)
{
    if (n < 1 || n > kMaxKernels || !k || !out || pad < 1) return fail(BFUSE_ERR_ARG, "bad argument");
    for (int i = 0; i < n; ++i)
        for (int d = 0; d < 3; ++d)
            if (k[i].grid[d] < 1 || k[i].block[d] < 1) return fail(BFUSE_ERR_ARG, "launch dims must be positive");
    const ThreadPlan p = plan_threads(n, reinterpret_cast<const LaunchDims*>(k), pad);
    memcpy(out, &p, sizeof(p));
    return BFUSE_OK;
}

int bfuse_plan_blocks(int pattern, int n, const bfuse_launch_dims* k, int p0, int p1, bfuse_block_plan* out)
{
    if (n < 1 || n > kMaxKernels || !k || !out) return fail(BFUSE_ERR_ARG, "bad argument");
    if (pattern < kZigzag || pattern > kRanges) return fail(BFUSE_ERR_ARG, "unknown pattern %d", pattern);
    for (int i = 0; i < n; ++i)
        for (int d = 0; d < 3; ++d)
            if (k[i].grid[d] < 1 || k[i].block[d] < 1) return fail(BFUSE_ERR_ARG, "launch dims must be positive");
    if ((pattern == kZigzag && (p0 < 1 || p1 < 1)) || ((pattern == kProportional || pattern == kChunked) && p0 < 1))
        return fail(BFUSE_ERR_ARG, "pattern parameters must be positive");
    const BlockPlan p = make_block_plan(pattern, n, reinterpret_cast<const LaunchDims*>(k), p0, p1);
    memcpy(out, &p, sizeof(p));
    return BFUSE_OK;
}

int bfuse_map_block(const bfuse_block_plan* plan, int bid, int* virt)
{
    if (!plan) {
        if (virt) *virt = -1;
        (void)fail(BFUSE_ERR_ARG, "null plan");
        return -1;
    }
    int v = -1;
    const int k = map_block(*reinterpret_cast<const BlockPlan*>(plan), bid, &v);
    if (virt) *virt = v;
    return k;
}

int bfuse_map_thread(const bfuse_thread_plan* plan, int bid, int tid, int* local)
{
    if (!plan) {
        if (local) *local = -1;
        (void)fail(BFUSE_ERR_ARG, "null plan");
        return -1;
    }
    int l = -1;
    const int k = map_thread(*reinterpret_cast<const ThreadPlan*>(plan), bid, tid, &l);
    if (local) *local = l;
    return k;
}

int bfuse_map_blocks_device(const bfuse_block_plan* plan, int lo, int hi, int* kernel_out, int* virt_out)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!plan || !kernel_out || !virt_out || hi <= lo) return fail(BFUSE_ERR_ARG, "bad argument");
    const int n = hi - lo;
    DevBuf dk, dv;
    HIP_TRY(hipMalloc(&dk.p, sizeof(int) * (size_t)n));
    HIP_TRY(hipMalloc(&dv.p, sizeof(int) * (size_t)n));
    BlockPlan p;
    memcpy(&p, plan, sizeof(p));
    hipLaunchKernelGGL(map_blocks_kernel, dim3((n + 255) / 256), dim3(256), 0, nullptr, p, lo, hi, dk.as<int>(), dv.as<int>());
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(kernel_out, dk.p, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(virt_out, dv.p, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
    return BFUSE_OK;
}

// The same evaluation with no allocation anywhere: the two tables are staged in the library's fixed
// device array (first half kernel ids, second half virtual block ids) instead of buffers allocated
// per call.  Every entry of [lo,hi) is written before it is copied out, so nothing has to be
// cleared between calls; the array keeps the last call's contents, and two calls that overlap on
// one device would race on it.
int bfuse_map_blocks_device_noalloc(const bfuse_block_plan* plan, int lo, int hi, int* kernel_out, int* virt_out)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!plan || !kernel_out || !virt_out || hi <= lo) return fail(BFUSE_ERR_ARG, "bad argument");
    const long long n = (long long)hi - (long long)lo;
    if (n > kNoAllocMaxIds)
        return fail(BFUSE_ERR_ARG, "bfuse_map_blocks_device_noalloc: %lld block ids requested, the fixed staging array holds %d; "
                                   "split the range or use bfuse_map_blocks_device", n, kNoAllocMaxIds);
    if (g.device < 0 || g.device >= kMaxDevices || !g_scratch_ptr[g.device])
        return fail(BFUSE_ERR_STATE, "no staging array address for device %d", g.device);
    int* dk = g_scratch_ptr[g.device];
    int* dv = dk + kNoAllocMaxIds;
    BlockPlan p;
    memcpy(&p, plan, sizeof(p));
    hipLaunchKernelGGL(map_blocks_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, nullptr, p, lo, hi, dk, dv);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(kernel_out, dk, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(virt_out, dv, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
    return BFUSE_OK;
}

int bfuse_probe_placement(int workgroups, int threads, int hold, unsigned* xcc, unsigned* se, unsigned* cu, unsigned* simd,
                          unsigned long long* start_ticks)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (workgroups < 1 || workgroups > (1 << 20) || threads < 64 || threads > 1024 || threads % 64 || hold < 0 || hold > 100000)
        return fail(BFUSE_ERR_ARG, "bad argument");
    DevBuf b_hw, b_xcc, b_t;
    HIP_TRY(hipMalloc(&b_hw.p, sizeof(unsigned) * (size_t)workgroups));
    HIP_TRY(hipMalloc(&b_xcc.p, sizeof(unsigned) * (size_t)workgroups));
    HIP_TRY(hipMalloc(&b_t.p, sizeof(unsigned long long) * (size_t)workgroups));
    unsigned *d_hw = b_hw.as<unsigned>(), *d_xcc = b_xcc.as<unsigned>();
    unsigned long long* d_t = b_t.as<unsigned long long>();
    hipLaunchKernelGGL(placement_kernel, dim3(workgroups), dim3(threads), 0, nullptr, d_hw, d_xcc, d_t, hold);
    HIP_TRY(hipGetLastError());
    std::vector<unsigned> hw((size_t)workgroups), xc((size_t)workgroups);
    std::vector<unsigned long long> ts((size_t)workgroups);
    HIP_TRY(hipMemcpy(hw.data(), d_hw, sizeof(unsigned) * hw.size(), hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(xc.data(), d_xcc, sizeof(unsigned) * xc.size(), hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(ts.data(), d_t, sizeof(unsigned long long) * ts.size(), hipMemcpyDeviceToHost));
    for (int i = 0; i < workgroups; ++i) {
        const unsigned h = hw[(size_t)i];  // gfx9 layout: wave 3:0, simd 5:4, pipe 7:6, cu 11:8, sh 12, se 15:13
        if (xcc) xcc[i] = xc[(size_t)i] & 0xFu;
        if (se) se[i] = (h >> 13) & 0x7u;
        if (cu) cu[i] = ((h >> 12) & 0x1u) * 16u + ((h >> 8) & 0xFu);
        if (simd) simd[i] = (h >> 4) & 0x3u;
        if (start_ticks) start_ticks[i] = ts[(size_t)i];
    }
    return BFUSE_OK;
}

int bfuse_set_plan(const void* func, const bfuse_block_plan* plan)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!func || !plan) return fail(BFUSE_ERR_ARG, "null argument");
    const KernelEntry* e = entry_of(func);
    if (!e || e->kind != kBfuseRt || !e->set_plan) return fail(BFUSE_ERR_ARG, "func is not a run-time-plan (bfuse_rt) kernel");
    BlockPlan p;
    memcpy(&p, plan, sizeof(p));
    // The kernel trusts the plan for every index it forms, so it is checked here in full: it must
    // send the fused block ids one-to-one onto the blocks of the kernel's sides.
    const int ns = e->n_sides;
    int side_grid[kMaxKernels] = {};
    int sum_grid = 0;
    for (int k = 0; k < ns; ++k) {
        for (const auto& c : registry())
            if (c.kind == kSingle && c.name == e->side[k]) side_grid[k] = (int)c.grid[0];
        sum_grid += side_grid[k];
    }
    if (p.n_kernels != ns || p.n_seg < 1 || p.n_seg > kMaxSegments) return fail(BFUSE_ERR_ARG, "plan: bad kernel or segment count");
    if (p.fused_grid != sum_grid)
        return fail(BFUSE_ERR_ARG, "plan covers %d blocks, the %d sides of %s have %d", p.fused_grid, ns, e->name.c_str(), sum_grid);
    for (int i = 0; i < p.n_seg; ++i) {
        const Segment& sg = p.seg[i];
        if (sg.period < 1 || sg.n_slot < 1 || sg.n_slot > kMaxKernels || sg.lo < 0 || sg.hi < sg.lo) return fail(BFUSE_ERR_ARG, "plan: malformed segment %d", i);
        for (int j = 0; j < sg.n_slot; ++j)
            if (sg.slot[j].kern < 0 || sg.slot[j].kern >= ns || sg.slot[j].width < 1 || sg.slot[j].off < 0 || sg.slot[j].base < 0)
                return fail(BFUSE_ERR_ARG, "plan: malformed slot %d of segment %d", j, i);
    }
    std::vector<unsigned char> seen[kMaxKernels];
    for (int k = 0; k < ns; ++k) seen[k].assign((size_t)side_grid[k], 0);
    for (int bid = 0; bid < p.fused_grid; ++bid) {
        int v = -1;
        const int k = map_block(p, bid, &v);
        if (k < 0 || k >= ns || v < 0 || v >= side_grid[k] || seen[k][(size_t)v])
            return fail(BFUSE_ERR_ARG, "plan: fused block %d maps to kernel %d block %d (out of range or visited twice)", bid, k, v);
        seen[k][(size_t)v] = 1;
    }
    HIP_TRY(hipDeviceSynchronize());  // no launch may still be reading the old plan
    if (e->set_plan(&p)) {
        (void)hipGetLastError();
        return fail(BFUSE_ERR_HIP, "could not copy the plan to the device");
    }
    installed_plans()[func] = p;
    return BFUSE_OK;
}

int bfuse_set_sync_spin_limit(const void* func, unsigned polls)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!func || polls < 1) return fail(BFUSE_ERR_ARG, "null kernel or a limit below 1");
    const KernelEntry* e = entry_of(func);
    if (!e) return fail(BFUSE_ERR_ARG, "func is not a kernel of this library");
    if (!e->set_spin_limit) return fail(BFUSE_ERR_ARG, "%s has no side barriers that poll (only thread-fused and run-time-plan kernels do)", e->name.c_str());
    HIP_TRY(hipDeviceSynchronize());   // no launch may be polling with the old limit
    if (e->set_spin_limit(polls)) {
        (void)hipGetLastError();
        return fail(BFUSE_ERR_HIP, "could not set the spin limit of %s's module", e->name.c_str());
    }
    return BFUSE_OK;
}

// ---- registry ---------------------------------------------------------------------------
static void fill_info(const KernelEntry& e, bfuse_kernel_info* o)
{
    memset(o, 0, sizeof(*o));
    snprintf(o->name, sizeof(o->name), "%s", e.name.c_str());
    o->func = e.func;
    o->kind = e.kind;
    for (int i = 0; i < 3; ++i) {
        o->grid[i] = e.grid[i];
        o->block[i] = e.block[i];
        for (int d = 0; d < 4; ++d) o->shape[i][d] = e.io[i].shape[d];
        o->elem_bytes[i] = e.io[i].elem_bytes;
    }
    o->has_barriers = e.has_barriers;
    o->regs = -1;
    o->lds_bytes = -1;
    if (g.inited) {
        hipFuncAttributes a;
        if (hipFuncGetAttributes(&a, e.func) == hipSuccess) {
            o->regs = a.numRegs;
            o->lds_bytes = (int)a.sharedSizeBytes;
        } else {
            (void)hipGetLastError();
        }
    }
    snprintf(o->side[0], sizeof(o->side[0]), "%s", e.side[0].c_str());
    snprintf(o->side[1], sizeof(o->side[1]), "%s", e.side[1].c_str());
    o->n_sides = e.kind == kSingle ? 1 : e.n_sides;
    for (int k = 2; k < kMaxKernels; ++k) snprintf(o->side_more[k - 2], sizeof(o->side_more[k - 2]), "%s", e.side[k].c_str());
    o->pattern = e.pattern;
    o->p0 = e.p0;
    o->p1 = e.p1;
    o->matrix_cores = e.kind == kSingle && e.matrix_cores;
}

// Kernels whose names start with `selftest_` exist for the library's own tests (operators that are
// malformed on purpose, to drive the give-up path of the side barriers).  The enumeration leaves them
// out, so that nothing that walks the registry (suite, configure, tuner, a user's loop) ever launches
// them; bfuse_kernel_find still finds them by name.
static bool enumerated(const KernelEntry& e) { return e.name.rfind("selftest_", 0) != 0; }

// Modules of fused kernels built after the library (one shared object per suite): loading one runs its
// registrars, which append to the registry above.  BFUSE_KERNEL_MODULES (paths separated by ':') names modules
// to load before the first look at the registry, so that every program over this library -- the command-line
// driver included -- sees them without an option of its own.
static int load_kernels(const char* path)
{
    static std::vector<std::string> loaded;
    for (const auto& p : loaded)
        if (p == path) return BFUSE_OK;
    const size_t before = registry().size();
    const int refused = bfuse::g_refused_entries;
    void* h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return fail(BFUSE_ERR_ARG, "cannot load kernel module '%s': %s", path, dlerror());
    if (bfuse::g_refused_entries != refused) {
        // its kernels that did register stay (their code is loaded); the caller is told to rebuild
        return fail(BFUSE_ERR_ARG, "'%s' was built against other headers than this library (%d kernels refused): rebuild it (build_pairs)",
                    path, bfuse::g_refused_entries - refused);
    }
    if (registry().size() == before) {
        dlclose(h);
        return fail(BFUSE_ERR_ARG, "'%s' registered no kernel: not a module built against this library", path);
    }
    loaded.emplace_back(path);
    return BFUSE_OK;
}

static int load_env_modules()
{
    static bool done = false;
    static int status = BFUSE_OK;
    if (done) return status;
    done = true;
    const char* env = getenv("BFUSE_KERNEL_MODULES");
    if (!env) return status;
    std::string all(env);
    size_t a = 0;
    while (a <= all.size()) {
        size_t b = all.find(':', a);
        if (b == std::string::npos) b = all.size();
        if (b > a && (status = load_kernels(all.substr(a, b - a).c_str()))) return status;
        a = b + 1;
    }
    return status;
}

int bfuse_load_kernels(const char* shared_object_path)
{
    if (!shared_object_path || !*shared_object_path) return fail(BFUSE_ERR_ARG, "null module path");
    int rc = load_env_modules();
    if (rc) return rc;
    return load_kernels(shared_object_path);
}

const char* bfuse_kernel_op_type(const char* name)
{
    if (!name || load_env_modules()) return nullptr;
    for (const auto& e : registry())
        if (e.name == name) return e.kind == kSingle ? e.op_type : nullptr;
    return nullptr;
}

int bfuse_kernel_op_lds(const char* name)
{
    if (!name || load_env_modules()) return -1;
    for (const auto& e : registry())
        if (e.name == name) return e.kind == kSingle ? e.smem_bytes : -1;
    return -1;
}

int bfuse_kernel_count(void)
{
    if (load_env_modules()) return 0;
    int n = 0;
    for (const auto& e : registry()) n += enumerated(e);
    return n;
}

int bfuse_kernel_at(int index, bfuse_kernel_info* out)
{
    if (index < 0 || !out) return fail(BFUSE_ERR_ARG, "index out of range");
    if (int rc = load_env_modules()) return rc;
    for (const auto& e : registry())
        if (enumerated(e) && index-- == 0) {
            fill_info(e, out);
            return BFUSE_OK;
        }
    return fail(BFUSE_ERR_ARG, "index out of range");
}

int bfuse_kernel_find(const char* name, bfuse_kernel_info* out)
{
    if (!name || !out) return fail(BFUSE_ERR_ARG, "null argument");
    if (int rc = load_env_modules()) return rc;
    for (const auto& e : registry())
        if (e.name == name) {
            fill_info(e, out);
            return BFUSE_OK;
        }
    return fail(BFUSE_ERR_ARG, "unknown kernel '%s'", name);
}

// ---- harness ----------------------------------------------------------------------------
int bfuse_set_elem_bytes(int side, int ib, int fb, int ob)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    if (g.side[side - 1].live) return fail(BFUSE_ERR_STATE, "set element sizes before initialize_kernel%d", side);
    const int v[3] = {ib, fb, ob};
    for (int i = 0; i < 3; ++i) {
        if (v[i] != 1 && v[i] != 2 && v[i] != 4 && v[i] != 8) return fail(BFUSE_ERR_ARG, "element size must be 1, 2, 4 or 8");
        g.side[side - 1].elem[i] = v[i];
    }
    return BFUSE_OK;
}

int initialize_kernel1(const int* I, const int* F, const int* O) { return init_side(0, I, F, O); }
int initialize_kernel2(const int* I, const int* F, const int* O) { return init_side(1, I, F, O); }
int finalize_kernel1(void) { return fini_side(0); }
int finalize_kernel2(void) { return fini_side(1); }
int bfuse_initialize_side(int side, const int* I, const int* F, const int* O)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    return init_side(side - 1, I, F, O);
}
int bfuse_finalize_side(int side)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    return fini_side(side - 1);
}

static int run_single(int idx, const void* I, const void* F, void* O, const int* Is, const int* Fs, const int* Os,
                      const void* func, const unsigned* grid, const unsigned* block)
{
    int rc;
    if (!I || !F || !O) return fail(BFUSE_ERR_ARG, "null host buffer");
    if ((rc = check_shapes(idx, Is, Fs, Os))) return rc;
    if ((rc = validate_mode(idx == 0 ? BFUSE_MODE_KERNEL1 : BFUSE_MODE_KERNEL2, func, grid, block, nullptr, nullptr, nullptr))) return rc;
    Side& s = g.side[idx];
    HIP_TRY(hipMemcpy(s.buf[0], I, s.bytes[0], hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(s.buf[1], F, s.bytes[1], hipMemcpyHostToDevice));
    if ((rc = launch3(func, grid, block, idx, nullptr))) return rc;
    if ((rc = sync_and_check())) return rc;
    HIP_TRY(hipMemcpy(O, s.buf[2], s.bytes[2], hipMemcpyDeviceToHost));
    return BFUSE_OK;
}

int run_kernel1(const void* I, const void* F, void* O, const int* Is, const int* Fs, const int* Os,
                bfuse_kernel3_fn func, const unsigned* grid, const unsigned* block, size_t)
{
    return run_single(0, I, F, O, Is, Fs, Os, (const void*)func, grid, block);
}

int run_kernel2(const void* I, const void* F, void* O, const int* Is, const int* Fs, const int* Os,
                bfuse_kernel3_fn func, const unsigned* grid, const unsigned* block, size_t)
{
    return run_single(1, I, F, O, Is, Fs, Os, (const void*)func, grid, block);
}

static int upload_both(const void* I1, const void* F1, const void* I2, const void* F2)
{
    Side &a = g.side[0], &b = g.side[1];
    HIP_TRY(hipMemcpy(a.buf[0], I1, a.bytes[0], hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(a.buf[1], F1, a.bytes[1], hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(b.buf[0], I2, b.bytes[0], hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(b.buf[1], F2, b.bytes[1], hipMemcpyHostToDevice));
    return BFUSE_OK;
}

static int download_both(void* O1, void* O2)
{
    Side &a = g.side[0], &b = g.side[1];
    HIP_TRY(hipMemcpy(O1, a.buf[2], a.bytes[2], hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(O2, b.buf[2], b.bytes[2], hipMemcpyDeviceToHost));
    return BFUSE_OK;
}

int run_parallel(const void* I1, const void* F1, void* O1, const void* I2, const void* F2, void* O2, const int* I1s,
                 const int* F1s, const int* O1s, const int* I2s, const int* F2s, const int* O2s,
                 bfuse_kernel3_fn func1, bfuse_kernel3_fn func2, const unsigned* g1, const unsigned* b1,
                 const unsigned* g2, const unsigned* b2, size_t, size_t)
{
    int rc;
    if (!I1 || !F1 || !O1 || !I2 || !F2 || !O2) return fail(BFUSE_ERR_ARG, "null host buffer");
    if ((rc = check_shapes(0, I1s, F1s, O1s)) || (rc = check_shapes(1, I2s, F2s, O2s))) return rc;
    if ((rc = validate_mode(BFUSE_MODE_PARALLEL, (const void*)func1, g1, b1, (const void*)func2, g2, b2))) return rc;
    if ((rc = upload_both(I1, F1, I2, F2))) return rc;
    if ((rc = enqueue_mode(BFUSE_MODE_PARALLEL, (const void*)func1, g1, b1, (const void*)func2, g2, b2, nullptr))) return rc;
    if ((rc = sync_and_check())) return rc;
    return download_both(O1, O2);
}

int run_fuse(const void* I1, const void* F1, void* O1, const void* I2, const void* F2, void* O2, const int* I1s,
             const int* F1s, const int* O1s, const int* I2s, const int* F2s, const int* O2s, bfuse_kernel6_fn func,
             const unsigned* grid, const unsigned* block, size_t, size_t)
{
    int rc;
    if (!I1 || !F1 || !O1 || !I2 || !F2 || !O2) return fail(BFUSE_ERR_ARG, "null host buffer");
    if ((rc = check_shapes(0, I1s, F1s, O1s)) || (rc = check_shapes(1, I2s, F2s, O2s))) return rc;
    const KernelEntry* e = entry_of((const void*)func);
    if (!e || e->kind == kSingle) return fail(BFUSE_ERR_ARG, "func is not a fused kernel of this library");
    const int mode = e->kind == kHfuse ? BFUSE_MODE_HFUSE : BFUSE_MODE_BFUSE;
    if ((rc = validate_mode(mode, (const void*)func, grid, block, nullptr, nullptr, nullptr))) return rc;
    if ((rc = upload_both(I1, F1, I2, F2))) return rc;
    if ((rc = launch6((const void*)func, grid, block, nullptr))) return rc;
    if ((rc = sync_and_check())) return rc;
    return download_both(O1, O2);
}

// ---- device-resident operation and timing -------------------------------------------------
int bfuse_upload(int side, const void* I, const void* F)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (!I || !F) return fail(BFUSE_ERR_ARG, "null host buffer");
    HIP_TRY(hipMemcpy(s.buf[0], I, s.bytes[0], hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(s.buf[1], F, s.bytes[1], hipMemcpyHostToDevice));
    return BFUSE_OK;
}

int bfuse_zero_output(int side)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    HIP_TRY(hipMemset(s.buf[2], 0, s.bytes[2]));
    return BFUSE_OK;
}

int bfuse_download(int side, void* O)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (!O) return fail(BFUSE_ERR_ARG, "null host buffer");
    // the output is copied out even when a side barrier gave up (the caller may want to look at
    // it), but the call then reports BFUSE_ERR_SYNC
    const int rc = sync_and_check();
    if (rc && rc != BFUSE_ERR_SYNC) return rc;
    HIP_TRY(hipMemcpy(O, s.buf[2], s.bytes[2], hipMemcpyDeviceToHost));
    return rc;
}

int bfuse_upload_part(int side, int tensor, size_t offset, const void* src, size_t bytes)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (tensor != 0 && tensor != 1) return fail(BFUSE_ERR_ARG, "tensor must be 0 (I) or 1 (F)");
    if (!src) return fail(BFUSE_ERR_ARG, "null host buffer");
    if (offset > s.bytes[tensor] || bytes > s.bytes[tensor] - offset)
        return fail(BFUSE_ERR_ARG, "bytes %zu .. %zu are outside the tensor's %zu", offset, offset + bytes, s.bytes[tensor]);
    if (bytes) HIP_TRY(hipMemcpy(static_cast<char*>(s.buf[tensor]) + offset, src, bytes, hipMemcpyHostToDevice));
    return BFUSE_OK;
}

int bfuse_download_part(int side, size_t offset, void* dst, size_t bytes)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (!dst) return fail(BFUSE_ERR_ARG, "null host buffer");
    if (offset > s.bytes[2] || bytes > s.bytes[2] - offset)
        return fail(BFUSE_ERR_ARG, "bytes %zu .. %zu are outside the output's %zu", offset, offset + bytes, s.bytes[2]);
    const int rc = sync_and_check();
    if (rc && rc != BFUSE_ERR_SYNC) return rc;
    if (bytes) HIP_TRY(hipMemcpy(dst, static_cast<const char*>(s.buf[2]) + offset, bytes, hipMemcpyDeviceToHost));
    return rc;
}

// Two order-independent sums (mod 2^64) over the 32-bit words of each chunk: the words themselves, and the
// words weighted by their position in the chunk.  grid = (parts, chunks).
__global__ void checksum_kernel(const unsigned* __restrict__ p, size_t words_per_chunk, unsigned long long* __restrict__ sums)
{
    const unsigned* __restrict__ q = p + (size_t)blockIdx.y * words_per_chunk;
    unsigned long long a = 0, b = 0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words_per_chunk; i += (size_t)gridDim.x * blockDim.x) {
        const unsigned w = q[i];
        a += w;
        b += (unsigned long long)w * (unsigned long long)(i % 65521u + 1u);
    }
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_down(a, off, 64);
        b += __shfl_down(b, off, 64);
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&sums[2 * (size_t)blockIdx.y], a);
        atomicAdd(&sums[2 * (size_t)blockIdx.y + 1], b);
    }
}

int bfuse_checksum_output(int side, size_t chunk_bytes, unsigned long long* sums)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (!sums) return fail(BFUSE_ERR_ARG, "null result buffer");
    if (chunk_bytes == 0 || chunk_bytes % 4 != 0 || s.bytes[2] % chunk_bytes != 0)
        return fail(BFUSE_ERR_ARG, "the chunk size %zu must be a multiple of 4 that divides the output's %zu bytes", chunk_bytes, s.bytes[2]);
    const size_t chunks = s.bytes[2] / chunk_bytes, words = chunk_bytes / 4;
    if (chunks > 65535) return fail(BFUSE_ERR_ARG, "%zu chunks: at most 65535", chunks);
    const int rc = sync_and_check();
    if (rc && rc != BFUSE_ERR_SYNC) return rc;
    DevBuf d;
    HIP_TRY(hipMalloc(&d.p, chunks * 2 * sizeof(unsigned long long)));
    HIP_TRY(hipMemset(d.p, 0, chunks * 2 * sizeof(unsigned long long)));
    size_t parts = (words + 256 * 16 - 1) / (256 * 16);   // ~16 words per thread
    if (parts > 64) parts = 64;
    if (parts < 1) parts = 1;
    hipLaunchKernelGGL(checksum_kernel, dim3((unsigned)parts, (unsigned)chunks), dim3(256), 0, nullptr,
                       static_cast<const unsigned*>(s.buf[2]), words, d.as<unsigned long long>());
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(sums, d.p, chunks * 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    return rc;
}

// The values of bfuse_fill_uniform (and of bfuse_f32_to_bf16 over them), written where they are needed: integer
// hash, two double operations and a conversion, the same on both sides.
__global__ void fill_uniform_kernel(void* __restrict__ out, size_t n, int elem, unsigned long long seed, float lo, float hi)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float v = (float)((double)lo + ((double)hi - (double)lo) * u01(seed, i));
        if (elem == 4) {
            static_cast<float*>(out)[i] = v;
        } else {
            unsigned u = __float_as_uint(v);
            static_cast<unsigned short*>(out)[i] = (u & 0x7fffffffu) > 0x7f800000u
                                                       ? (unsigned short)((u >> 16) | 0x0040u)
                                                       : (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        }
    }
}

int bfuse_fill_uniform_device(int side, int tensor, unsigned long long seed, float lo, float hi)
{
    if (side < 1 || side > kMaxKernels) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    Side& s = g.side[side - 1];
    if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
    if (tensor != 0 && tensor != 1) return fail(BFUSE_ERR_ARG, "tensor must be 0 (I) or 1 (F)");
    if (s.elem[tensor] != 4 && s.elem[tensor] != 2)
        return fail(BFUSE_ERR_ARG, "device fill writes fp32 or bf16 tensors, this one has %d-byte elements", s.elem[tensor]);
    if (int rc = sync_and_check()) return rc;   // nothing launched earlier may still be reading the operand
    const size_t n = s.bytes[tensor] / (size_t)s.elem[tensor];
    size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
    if (blocks > 16384) blocks = 16384;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(fill_uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, nullptr, s.buf[tensor], n, s.elem[tensor], seed, lo, hi);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipDeviceSynchronize());
    return BFUSE_OK;
}

int bfuse_synchronize(void)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    return sync_and_check();
}

int bfuse_launch(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb, const unsigned* gb,
                 const unsigned* bb)
{
    int rc;
    if ((rc = validate_mode(mode, fa, ga, ba, fb, gb, bb))) return rc;
    return enqueue_mode(mode, fa, ga, ba, fb, gb, bb, nullptr);
}

int bfuse_time(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb, const unsigned* gb,
               const unsigned* bb, int warmup, int reps, float* us_total, float* us_a, float* us_b)
{
    int rc;
    if (warmup < 0 || reps < 1 || reps > 100000 || !us_total) return fail(BFUSE_ERR_ARG, "bad repetition count or null output");
    if ((rc = validate_mode(mode, fa, ga, ba, fb, gb, bb))) return rc;
    const bool two = (mode == BFUSE_MODE_PARALLEL || mode == BFUSE_MODE_SERIAL);
    for (int i = 0; i < warmup; ++i)
        if ((rc = enqueue_mode(mode, fa, ga, ba, fb, gb, bb, nullptr))) return rc;
    HIP_TRY(hipDeviceSynchronize());
    EventList evl((size_t)reps * 4);
    std::vector<hipEvent_t>& ev = evl.v;
    const int per = two ? 4 : 2;
    for (int r = 0; r < reps; ++r)
        for (int j = 0; j < per; ++j) HIP_TRY(hipEventCreate(&ev[(size_t)r * 4 + j]));
    for (int r = 0; r < reps; ++r) {
        if ((rc = enqueue_mode(mode, fa, ga, ba, fb, gb, bb, &ev[(size_t)r * 4]))) return rc;
        // Two streams run ahead of each other: without a meeting point per repetition the short
        // kernel's stream would be hundreds of launches ahead and "first start -> last end" of
        // repetition r would span all of them.  The reference synchronises after every run_parallel
        // (operation_cu.py:199-228).
        if (mode == BFUSE_MODE_PARALLEL) HIP_TRY(hipDeviceSynchronize());
    }
    if ((rc = sync_and_check())) return rc;
    for (int r = 0; r < reps; ++r) {
        hipEvent_t* e = &ev[(size_t)r * 4];
        float ms_a = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms_a, e[0], e[1]));
        if (us_a) us_a[r] = ms_a * 1000.f;
        if (!two) {
            us_total[r] = ms_a * 1000.f;
            if (us_b) us_b[r] = 0.f;
        } else {
            float ms_b = 0.f, s_ab = 0.f;
            HIP_TRY(hipEventElapsedTime(&ms_b, e[2], e[3]));
            HIP_TRY(hipEventElapsedTime(&s_ab, e[0], e[2]));  // start_b - start_a (may be negative)
            if (us_b) us_b[r] = ms_b * 1000.f;
            // first start -> last end (scripts/analyze_test_suite.py:142-154)
            const float first = s_ab < 0.f ? s_ab : 0.f;
            const float end_a = ms_a, end_b = s_ab + ms_b;
            us_total[r] = ((end_a > end_b ? end_a : end_b) - first) * 1000.f;
        }
    }
    return BFUSE_OK;
}

int bfuse_time_batched(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb,
                       const unsigned* gb, const unsigned* bb, int warmup, int reps, float* us_per_launch)
{
    int rc;
    if (warmup < 0 || reps < 1 || !us_per_launch) return fail(BFUSE_ERR_ARG, "bad repetition count or null output");
    if (mode == BFUSE_MODE_PARALLEL) return fail(BFUSE_ERR_ARG, "batched timing is single-stream");
    if ((rc = validate_mode(mode, fa, ga, ba, fb, gb, bb))) return rc;
    for (int i = 0; i < warmup; ++i)
        if ((rc = enqueue_mode(mode, fa, ga, ba, fb, gb, bb, nullptr))) return rc;
    HIP_TRY(hipDeviceSynchronize());
    EventList evl(2);
    hipEvent_t &e0 = evl.v[0], &e1 = evl.v[1];
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    HIP_TRY(hipEventRecord(e0, nullptr));
    for (int r = 0; r < reps; ++r)
        if ((rc = enqueue_mode(mode, fa, ga, ba, fb, gb, bb, nullptr))) return rc;
    HIP_TRY(hipEventRecord(e1, nullptr));
    if ((rc = sync_and_check())) return rc;
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    *us_per_launch = ms * 1000.f / (float)reps;
    return BFUSE_OK;
}

// One repetition of `mode` recorded into the capture that is open on s0 (s1: the second stream of mode 2).
static int capture_mode(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb,
                        const unsigned* gb, const unsigned* bb, hipStream_t s0, hipStream_t s1, hipEvent_t fork, hipEvent_t join)
{
    int rc;
    switch (mode) {
        case BFUSE_MODE_KERNEL1: return launch3(fa, ga, ba, 0, s0);
        case BFUSE_MODE_KERNEL2: return launch3(fa, ga, ba, 1, s0);
        case BFUSE_MODE_SERIAL:
            if ((rc = launch3(fa, ga, ba, 0, s0))) return rc;
            return launch3(fb, gb, bb, 1, s0);
        case BFUSE_MODE_PARALLEL:
            HIP_TRY(hipEventRecord(fork, s0));
            HIP_TRY(hipStreamWaitEvent(s1, fork, 0));
            if ((rc = launch3(fa, ga, ba, 0, s0))) return rc;
            if ((rc = launch3(fb, gb, bb, 1, s1))) return rc;
            HIP_TRY(hipEventRecord(join, s1));
            HIP_TRY(hipStreamWaitEvent(s0, join, 0));
            return BFUSE_OK;
        case BFUSE_MODE_HFUSE:
        case BFUSE_MODE_BFUSE: return launch6(fa, ga, ba, s0);
    }
    return fail(BFUSE_ERR_ARG, "unknown mode %d", mode);
}

int bfuse_time_graph(int mode, const void* fa, const unsigned* ga, const unsigned* ba, const void* fb,
                     const unsigned* gb, const unsigned* bb, int chain, int reps, float* us_per_repetition)
{
    int rc;
    if (chain < 1 || chain > 1000 || reps < 1 || !us_per_repetition) return fail(BFUSE_ERR_ARG, "bad repetition count or null output");
    if ((rc = validate_mode(mode, fa, ga, ba, fb, gb, bb))) return rc;
    // rocprofv3's kernel tracing takes a segmentation fault in its own code on the first graph launch here
    // (ROCm 7.2): refused with a message instead
    {
        const char* pre = getenv("LD_PRELOAD");
        const char* tool = getenv("ROCP_TOOL_LIBRARIES");
        if ((pre && strstr(pre, "rocprofiler")) || (tool && *tool))
            return fail(BFUSE_ERR_STATE, "graph replays are not timed under rocprofv3: its tracing does not survive a graph launch on this ROCm");
    }
    if ((rc = sync_and_check())) return rc;   // nothing of an earlier launch is pending when the capture starts
    hipStream_t s0 = g.side[mode == BFUSE_MODE_KERNEL2 ? 1 : 0].stream, s1 = g.side[1].stream;   // the legacy stream cannot be captured
    if (!s0 || (mode == BFUSE_MODE_PARALLEL && !s1)) return fail(BFUSE_ERR_STATE, "the side has no stream: initialize_kernel first");
    EventList evl(4);
    for (int i = 0; i < 2; ++i) HIP_TRY(hipEventCreateWithFlags(&evl.v[i], hipEventDisableTiming));   // fork, join
    for (int i = 2; i < 4; ++i) HIP_TRY(hipEventCreate(&evl.v[i]));
    struct Graph {
        hipGraph_t g = nullptr;
        hipGraphExec_t x = nullptr;
        ~Graph()
        {
            if (x) (void)hipGraphExecDestroy(x);
            if (g) (void)hipGraphDestroy(g);
        }
    } gr;
    HIP_TRY(hipStreamBeginCapture(s0, hipStreamCaptureModeThreadLocal));
    for (int c = 0; c < chain && rc == BFUSE_OK; ++c) rc = capture_mode(mode, fa, ga, ba, fb, gb, bb, s0, s1, evl.v[0], evl.v[1]);
    const hipError_t ended = hipStreamEndCapture(s0, &gr.g);   // always: the stream must leave capture mode
    if (rc) return rc;
    HIP_TRY(ended);
    HIP_TRY(hipGraphInstantiate(&gr.x, gr.g, nullptr, nullptr, 0));
    HIP_TRY(hipGraphLaunch(gr.x, s0));
    if ((rc = sync_and_check())) return rc;
    HIP_TRY(hipEventRecord(evl.v[2], s0));
    for (int r = 0; r < reps; ++r) HIP_TRY(hipGraphLaunch(gr.x, s0));
    HIP_TRY(hipEventRecord(evl.v[3], s0));
    if ((rc = sync_and_check())) return rc;
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, evl.v[2], evl.v[3]));
    *us_per_repetition = ms * 1000.f / ((float)reps * (float)chain);
    return BFUSE_OK;
}

// ---- launch lists: any registered kernel over any sides -------------------------------------
static int validate_list(int n, const bfuse_launch_desc* l)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (n < 1 || n > 16 || !l) return fail(BFUSE_ERR_ARG, "a launch list holds 1 .. 16 launches");
    for (int j = 0; j < n; ++j) {
        const bfuse_launch_desc& d = l[j];
        const KernelEntry* e = entry_of(d.func);
        if (!e) return fail(BFUSE_ERR_ARG, "launch %d: func is not a kernel of this library", j);
        const int want = e->kind == kSingle ? 1 : e->n_sides;
        if (d.n_sides != want) return fail(BFUSE_ERR_ARG, "launch %d: %s runs over %d sides, not %d", j, e->name.c_str(), want, d.n_sides);
        int rc;
        if ((rc = check_launch(d.func, d.grid, d.block, 3 * want))) return rc;
        int sides0[kMaxKernels];
        for (int k = 0; k < want; ++k) {
            if (d.sides[k] < 1 || d.sides[k] > kMaxKernels) return fail(BFUSE_ERR_ARG, "launch %d: side must be 1 .. %d", j, kMaxKernels);
            for (int m = 0; m < k; ++m)
                if (d.sides[m] == d.sides[k]) return fail(BFUSE_ERR_ARG, "launch %d: side %d named twice", j, d.sides[k]);
            sides0[k] = d.sides[k] - 1;
        }
        if ((rc = e->kind == kSingle ? check_side_fits(d.func, sides0[0]) : check_fused_fits(d.func, sides0))) return rc;
    }
    return BFUSE_OK;
}

static int enqueue_list(int n, const bfuse_launch_desc* l, hipEvent_t* ev /* 2 per launch or nullptr */)
{
    for (int j = 0; j < n; ++j) {
        const bfuse_launch_desc& d = l[j];
        int sides0[kMaxKernels];
        for (int k = 0; k < d.n_sides; ++k) sides0[k] = d.sides[k] - 1;
        const KernelEntry* e = entry_of(d.func);
        hipEvent_t e0 = ev ? ev[2 * j] : nullptr, e1 = ev ? ev[2 * j + 1] : nullptr;
        int rc = e->kind == kSingle ? launch3(d.func, d.grid, d.block, sides0[0], nullptr, e0, e1)
                                    : launch_fused(d.func, d.grid, d.block, d.n_sides, sides0, nullptr, e0, e1);
        if (rc) return rc;
    }
    return BFUSE_OK;
}

int bfuse_launch_list(int n, const bfuse_launch_desc* launches)
{
    int rc = validate_list(n, launches);
    if (rc) return rc;
    return enqueue_list(n, launches, nullptr);
}

int bfuse_time_list(int n, const bfuse_launch_desc* launches, int warmup, int reps, float* us_each, float* us_queued)
{
    int rc = validate_list(n, launches);
    if (rc) return rc;
    if (warmup < 0 || reps < 1 || reps > 100000 || (!us_each && !us_queued)) return fail(BFUSE_ERR_ARG, "bad repetition count or no output");
    for (int i = 0; i < warmup; ++i)
        if ((rc = enqueue_list(n, launches, nullptr))) return rc;
    HIP_TRY(hipDeviceSynchronize());
    if (us_each) {
        EventList evl((size_t)reps * 2 * n);
        for (auto& e : evl.v) HIP_TRY(hipEventCreate(&e));
        for (int r = 0; r < reps; ++r)
            if ((rc = enqueue_list(n, launches, &evl.v[(size_t)r * 2 * n]))) return rc;
        if ((rc = sync_and_check())) return rc;
        for (int j = 0; j < n; ++j) {
            double sum = 0.0;
            for (int r = 0; r < reps; ++r) {
                float ms = 0.f;
                HIP_TRY(hipEventElapsedTime(&ms, evl.v[((size_t)r * n + j) * 2], evl.v[((size_t)r * n + j) * 2 + 1]));
                sum += ms;
            }
            us_each[j] = (float)(sum * 1000.0 / reps);
        }
    }
    if (us_queued) {
        EventList evl(2);
        HIP_TRY(hipEventCreate(&evl.v[0]));
        HIP_TRY(hipEventCreate(&evl.v[1]));
        HIP_TRY(hipEventRecord(evl.v[0], nullptr));
        for (int r = 0; r < reps; ++r)
            if ((rc = enqueue_list(n, launches, nullptr))) return rc;
        HIP_TRY(hipEventRecord(evl.v[1], nullptr));
        if ((rc = sync_and_check())) return rc;
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, evl.v[0], evl.v[1]));
        *us_queued = ms * 1000.f / (float)reps;
    }
    return BFUSE_OK;
}

// ---- kernels from a code object -------------------------------------------------------------

int bfuse_module_load(const char* path, int* module_id)
{
    if (!g.inited) return fail(BFUSE_ERR_STATE, "bfuse_init has not been called");
    if (!path || !module_id) return fail(BFUSE_ERR_ARG, "null argument");
    hipModule_t mod = nullptr;
    hipError_t st = hipModuleLoad(&mod, path);
    if (st != hipSuccess) {
        (void)hipGetLastError();  // do not leave the failure for the next call to find
        return fail(BFUSE_ERR_HIP, "hipModuleLoad(%s): %s", path, hipGetErrorString(st));
    }
    auto& ms = modules();
    for (size_t i = 0; i < ms.size(); ++i)
        if (!ms[i]) {
            ms[i] = mod;
            *module_id = (int)i;
            return BFUSE_OK;
        }
    ms.push_back(mod);
    *module_id = (int)ms.size() - 1;
    return BFUSE_OK;
}

int bfuse_module_unload(int id)
{
    auto& ms = modules();
    if (id < 0 || id >= (int)ms.size() || !ms[id]) return fail(BFUSE_ERR_ARG, "unknown module %d", id);
    const int rc = sync_and_check();   // nothing of the module may still run; its counter is read while it exists
    if (rc == BFUSE_ERR_HIP) return rc;   // the device did not come to rest: the module stays loaded (bfuse_shutdown tries again)
    HIP_TRY(hipModuleUnload(ms[id]));
    ms[id] = nullptr;
    return rc;
}

int bfuse_module_launch(int id, const char* name, const unsigned* grid, const unsigned* block, int n_ptrs, int side,
                        float* us_out)
{
    auto& ms = modules();
    if (id < 0 || id >= (int)ms.size() || !ms[id]) return fail(BFUSE_ERR_ARG, "unknown module %d", id);
    if (!name || !grid || !block) return fail(BFUSE_ERR_ARG, "null argument");
    if (n_ptrs < 3 || n_ptrs > 3 * kMaxKernels || n_ptrs % 3) return fail(BFUSE_ERR_ARG, "n_ptrs must be 3, 6, ... %d", 3 * kMaxKernels);
    if (n_ptrs == 3 && (side < 1 || side > kMaxKernels)) return fail(BFUSE_ERR_ARG, "side must be 1 .. %d", kMaxKernels);
    for (int i = 0; i < 3; ++i)
        if (grid[i] == 0 || block[i] == 0) return fail(BFUSE_ERR_ARG, "empty launch shape");
    if ((size_t)block[0] * block[1] * block[2] > 1024) return fail(BFUSE_ERR_ARG, "more than 1024 threads per workgroup");
    hipFunction_t fn = nullptr;
    hipError_t st = hipModuleGetFunction(&fn, ms[id], name);
    if (st != hipSuccess) {
        (void)hipGetLastError();
        return fail(BFUSE_ERR_ARG, "kernel '%s' is not in module %d: %s", name, id, hipGetErrorString(st));
    }
    void* ptrs[3 * kMaxKernels];
    if (n_ptrs == 3) {
        Side& s = g.side[side - 1];
        if (!s.live) return fail(BFUSE_ERR_STATE, "kernel%d is not initialized", side);
        for (int i = 0; i < 3; ++i) ptrs[i] = s.buf[i];
    } else {
        for (int k = 0; k < n_ptrs / 3; ++k) {
            if (!g.side[k].live) return fail(BFUSE_ERR_STATE, "sides 1 .. %d must be initialized", n_ptrs / 3);
            for (int i = 0; i < 3; ++i) ptrs[3 * k + i] = g.side[k].buf[i];
        }
    }
    void* args[3 * kMaxKernels];
    for (int i = 0; i < n_ptrs; ++i) args[i] = &ptrs[i];
    EventList evl(2);
    hipEvent_t &e0 = evl.v[0], &e1 = evl.v[1];
    if (us_out) {
        HIP_TRY(hipEventCreate(&e0));
        HIP_TRY(hipEventCreate(&e1));
    }
    bool known = false;
    for (int m : g_pending_modules) known = known || m == id;
    if (!known) g_pending_modules.push_back(id);
    HIP_TRY(hipExtModuleLaunchKernel(fn, grid[0] * block[0], grid[1] * block[1], grid[2] * block[2], block[0], block[1],
                                     block[2], 0, nullptr, args, nullptr, e0, e1, 0));
    if (us_out) {
        int rc = sync_and_check();
        if (rc) return rc;
        float ms_ = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms_, e0, e1));
        *us_out = ms_ * 1000.f;
    }
    return BFUSE_OK;
}

// ---- synthetic inputs and checks ------------------------------------------------------------
void bfuse_fill_uniform(unsigned long long seed, size_t n, float lo, float hi, float* out)
{
    for (size_t i = 0; i < n; ++i) out[i] = (float)((double)lo + ((double)hi - (double)lo) * u01(seed, i));
}

void bfuse_fill_normal(unsigned long long seed, size_t n, float mean, float std, float* out)
{
    const double two_pi = 6.283185307179586476925;
    for (size_t i = 0; i < n; ++i) {
        const double u1 = u01(seed, 2 * (unsigned long long)i), u2 = u01(seed, 2 * (unsigned long long)i + 1);
        out[i] = (float)((double)mean + (double)std * std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2));
    }
}

void bfuse_f32_to_bf16(size_t n, const float* in, unsigned short* out)
{
    for (size_t i = 0; i < n; ++i) {
        unsigned u;
        memcpy(&u, &in[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            out[i] = (unsigned short)((u >> 16) | 0x0040u);
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            out[i] = (unsigned short)(u >> 16);
        }
    }
}

void bfuse_bf16_to_f32(size_t n, const unsigned short* in, float* out)
{
    for (size_t i = 0; i < n; ++i) {
        const unsigned u = (unsigned)in[i] << 16;
        memcpy(&out[i], &u, 4);
    }
}

long bfuse_check_matrix(const float* O, const float* A, size_t count, float eps)
{
    long bad = 0;
    for (size_t i = 0; i < count; ++i) {
        const float o = O[i], a = A[i];
        if (std::isnan(o) || std::isnan(a)) {
            bad += !(std::isnan(o) && std::isnan(a));
            continue;
        }
        if (std::fabs(o - a) > eps && (a == 0.f || std::fabs((o - a) / a) > eps)) ++bad;
    }
    return bad;
}

}  // extern "C"
