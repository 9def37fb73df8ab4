// Fusion index maps: which operator a fused workgroup (or thread) belongs to and which
// virtual block of that operator it executes.
//
// One implementation, `constexpr`, shared by the host (C ABI bfuse_plan_*) and by the fused
// kernels, where the plan is a compile-time constant and the lookup folds to a handful of
// compares and one div/mod by a constant.
//
// The maps are the ones the reference's fuser emits as text
// (horizontal-fuser/src/Algorithms.cc): hfusePattern :19-116, coarseInterleavePattern
// :118-317, coarseInterleaveWithoutSMPattern :319-526, coarseInterleaveWithoutSMPattern2
// :528-739.  Here every block-fusion pattern is lowered to one table form -- a list of
// *segments* of the fused grid, each a periodic interleave of slots:
//
//     bid in [lo, hi):  rel = bid - lo,  q = rel / period,  r = rel % period
//     slot s owns r in [off_s, off_s + width_s):  kernel = kern_s,
//                                                 virt   = base_s + q * width_s + (r - off_s)
//
// A contiguous range (the reference's "tail" branches, and the plain blockIdx-range
// dispatch) is a segment with one slot whose period is its own length.
#pragma once

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define BFUSE_HD __host__ __device__
#else
#define BFUSE_HD
#endif

namespace bfuse {

constexpr int kMaxKernels = 4;
constexpr int kMaxSegments = 2 * kMaxKernels;
constexpr int kWaveSize = 64;  // gfx950 wavefront; the reference pads thread ranges to 32

struct Dims3 {
    int x, y, z;
    BFUSE_HD constexpr int size() const { return x * y * z; }
};

struct LaunchDims {  // GridDim / BlockDim of one operator (Contexts.h:13-26)
    Dims3 grid, block;
};

struct Slot {
    int kern, off, width, base;
};

struct Segment {
    int lo, hi, period, n_slot;
    Slot slot[kMaxKernels];
};

struct BlockPlan {
    int n_kernels;
    int n_seg;
    Segment seg[kMaxSegments];
    int fused_grid;   // sum of grids   (Algorithms.cc:719-736)
    int fused_block;  // max of blocks
    int threads[kMaxKernels];
};

struct ThreadPlan {  // horizontal (thread-level) fusion
    int n_kernels;
    int thr_lo[kMaxKernels], thr_hi[kMaxKernels];  // [start_k, start_k + T_k)
    int blocks[kMaxKernels];                        // side k is live for bid < blocks[k]
    int fused_grid;                                 // max of grids (Algorithms.cc:98-113)
    int fused_block;                                // sum of padded thread counts
};

BFUSE_HD constexpr int round_up(int v, int m) { return (v + m - 1) / m * m; }
BFUSE_HD constexpr int imin(int a, int b) { return a < b ? a : b; }
BFUSE_HD constexpr int imax(int a, int b) { return a > b ? a : b; }

// ---- horizontal fusion --------------------------------------------------------------
// Thread ranges are laid end to end, each padded to `pad` threads so that no wavefront
// holds threads of two operators (pad = 64 on gfx950; 32 reproduces the reference).
BFUSE_HD constexpr ThreadPlan plan_threads(int n, const LaunchDims* k, int pad)
{
    ThreadPlan p{};
    p.n_kernels = n;
    int acc = 0;
    for (int i = 0; i < n; ++i) {
        const int t = k[i].block.size();
        p.thr_lo[i] = acc;
        p.thr_hi[i] = acc + t;
        p.blocks[i] = k[i].grid.size();
        acc += round_up(t, pad);
        p.fused_grid = imax(p.fused_grid, p.blocks[i]);
    }
    p.fused_block = acc;
    return p;
}

// Returns the operator owning (bid, tid) or -1; *local_tid is the thread id inside it.
BFUSE_HD constexpr int map_thread(const ThreadPlan& p, int bid, int tid, int* local_tid)
{
    for (int i = 0; i < p.n_kernels; ++i) {
        if (tid >= p.thr_lo[i] && tid < p.thr_hi[i] && bid < p.blocks[i]) {
            *local_tid = tid - p.thr_lo[i];
            return i;
        }
    }
    return -1;
}

// ---- block fusion -------------------------------------------------------------------
namespace detail {

BFUSE_HD constexpr void finish_dims(BlockPlan& p, int n, const LaunchDims* k)
{
    p.n_kernels = n;
    p.fused_grid = 0;
    p.fused_block = 0;
    for (int i = 0; i < n; ++i) {
        p.threads[i] = k[i].block.size();
        p.fused_grid += k[i].grid.size();
        p.fused_block = imax(p.fused_block, p.threads[i]);
    }
}

BFUSE_HD constexpr void push_range(BlockPlan& p, int& cursor, int kern, int count, int base)
{
    if (count <= 0) return;
    Segment& s = p.seg[p.n_seg++];
    s.lo = cursor;
    s.hi = cursor + count;
    s.period = count;
    s.n_slot = 1;
    s.slot[0] = Slot{kern, 0, count, base};
    cursor += count;
}

// One interleaved segment with `ratio[i]` consecutive blocks of operator i per period,
// repeated while every operator still has a full share, then each operator's remainder as a
// contiguous range in listed order.
BFUSE_HD constexpr BlockPlan plan_from_ratios(int n, const LaunchDims* k, const int* ratio)
{
    BlockPlan p{};
    finish_dims(p, n, k);
    int rounds = -1, period = 0;
    for (int i = 0; i < n; ++i) {
        const int q = k[i].grid.size() / ratio[i];
        rounds = rounds < 0 ? q : imin(rounds, q);
        period += ratio[i];
    }
    int cursor = 0;
    if (rounds > 0) {
        Segment& s = p.seg[p.n_seg++];
        s.lo = 0;
        s.hi = rounds * period;
        s.period = period;
        s.n_slot = n;
        int off = 0;
        for (int i = 0; i < n; ++i) {
            s.slot[i] = Slot{i, off, ratio[i], 0};
            off += ratio[i];
        }
        cursor = s.hi;
    }
    for (int i = 0; i < n; ++i)
        push_range(p, cursor, i, k[i].grid.size() - ratio[i] * rounds, ratio[i] * rounds);
    return p;
}

}  // namespace detail

// Zig-zag interleave with a capped ratio: operator i contributes
// min(g_i / g_min, M) * N consecutive blocks per period (M = N = 1: strict alternation).
BFUSE_HD constexpr BlockPlan plan_zigzag(int n, const LaunchDims* k, int M, int N)
{
    int gmin = k[0].grid.size();
    for (int i = 1; i < n; ++i) gmin = imin(gmin, k[i].grid.size());
    int ratio[kMaxKernels] = {};
    for (int i = 0; i < n; ++i) ratio[i] = imin(k[i].grid.size() / gmin, M) * N;
    return detail::plan_from_ratios(n, k, ratio);
}

// Interleave in proportion to the grid sizes: ratio g_i / max(1, g_min / min_option).
BFUSE_HD constexpr BlockPlan plan_proportional(int n, const LaunchDims* k, int min_option)
{
    int gmin = k[0].grid.size();
    for (int i = 1; i < n; ++i) gmin = imin(gmin, k[i].grid.size());
    const int unit = imax(1, gmin / min_option);
    int ratio[kMaxKernels] = {};
    for (int i = 0; i < n; ++i) ratio[i] = k[i].grid.size() / unit;
    return detail::plan_from_ratios(n, k, ratio);
}

// Alternate whole chunks of `chunk` blocks among the operators that still have a full chunk
// left (smallest grid drops out first), then every operator's sub-chunk remainder in listed
// order.  The reference sizes the chunk to the SM count; on MI355X a multiple of 8 keeps
// each operator's blocks spread over all eight XCDs (consecutive workgroup ids go to
// consecutive XCDs), and 256 gives one chunk per CU round.
BFUSE_HD constexpr BlockPlan plan_chunked(int n, const LaunchDims* k, int chunk)
{
    BlockPlan p{};
    detail::finish_dims(p, n, k);
    int order[kMaxKernels] = {};
    for (int i = 0; i < n; ++i) order[i] = i;
    for (int i = 1; i < n; ++i)  // ascending grid size, listed order on ties
        for (int j = i; j > 0 && k[order[j - 1]].grid.size() > k[order[j]].grid.size(); --j) {
            const int t = order[j];
            order[j] = order[j - 1];
            order[j - 1] = t;
        }
    int cursor = 0, done = 0;  // `done` = blocks every live operator has already issued
    for (int i = 0; i < n; ++i) {
        const int full = k[order[i]].grid.size() / chunk * chunk;
        const int alive = n - i;
        if (full > done) {
            Segment& s = p.seg[p.n_seg++];
            s.lo = cursor;
            s.hi = cursor + (full - done) * alive;
            s.period = chunk * alive;
            s.n_slot = alive;
            for (int j = i; j < n; ++j) s.slot[j - i] = Slot{order[j], (j - i) * chunk, chunk, done};
            cursor = s.hi;
            done = full;
        }
    }
    for (int i = 0; i < n; ++i) {
        const int g = k[i].grid.size();
        detail::push_range(p, cursor, i, g % chunk, g - g % chunk);
    }
    return p;
}

// Plain blockIdx-range dispatch: all blocks of operator 0, then operator 1, ...
BFUSE_HD constexpr BlockPlan plan_ranges(int n, const LaunchDims* k)
{
    BlockPlan p{};
    detail::finish_dims(p, n, k);
    int cursor = 0;
    for (int i = 0; i < n; ++i) detail::push_range(p, cursor, i, k[i].grid.size(), 0);
    return p;
}

// Returns the operator owning fused block `bid` (or -1) and its virtual block index.
BFUSE_HD constexpr int map_block(const BlockPlan& p, int bid, int* virt)
{
    for (int s = 0; s < p.n_seg; ++s) {
        const Segment& g = p.seg[s];
        if (bid >= g.lo && bid < g.hi) {
            const int rel = bid - g.lo;
            const int q = rel / g.period, r = rel % g.period;
            for (int j = 0; j < g.n_slot; ++j) {
                const Slot& sl = g.slot[j];
                if (r >= sl.off && r < sl.off + sl.width) {
                    *virt = sl.base + q * sl.width + (r - sl.off);
                    return sl.kern;
                }
            }
        }
    }
    return -1;
}

// Pattern selector used by the C ABI and by the fused-kernel templates.
enum Pattern : int {
    kZigzag = 0,        // p0 = M, p1 = N
    kProportional = 1,  // p0 = min_option
    kChunked = 2,       // p0 = chunk
    kRanges = 3,
};

BFUSE_HD constexpr BlockPlan make_block_plan(int pattern, int n, const LaunchDims* k, int p0, int p1)
{
    switch (pattern) {
        case kZigzag: return plan_zigzag(n, k, p0, p1);
        case kProportional: return plan_proportional(n, k, p0);
        case kChunked: return plan_chunked(n, k, p0);
        default: return plan_ranges(n, k);
    }
}

// Virtual (x, y, z) ids from a linear id, x fastest (Algorithms.cc:687-692).
BFUSE_HD constexpr Dims3 delinearize(int linear, const Dims3& extent)
{
    return Dims3{linear % extent.x, linear / extent.x % extent.y, linear / (extent.x * extent.y)};
}

// GEMM tile of a workgroup id, dealt over the eight XCDs.
//
// The hardware sends consecutive workgroup ids to consecutive XCDs, and every XCD has an L2 of its
// own: an operand slab that tiles on k different XCDs share is fetched k times (from HBM or the
// last-level cache).  Here id % 8 is taken as the XCD and the GX x GY tile grid is cut into AX x AY
// rectangles, one per XCD; id / 8 walks the rectangle.  An XCD then fetches GY / AY row slabs of A
// (BM rows each) and GX / AX column slabs of B (BN columns each); AX x AY = 8 is chosen to make
// that sum smallest.  When the grid cannot be cut that way the plain x-fastest order is kept.
template <int GX, int GY, int BM, int BN>
struct XcdTiles {
    static constexpr int cost(int ax, int ay) { return (GY / ay) * BM + (GX / ax) * BN; }
    static constexpr bool fits(int ax, int ay) { return GX % ax == 0 && GY % ay == 0; }
    static constexpr int pick_ax()
    {
        int best = 0, best_cost = 0;
        for (int ax = 1; ax <= 8; ax *= 2) {
            const int ay = 8 / ax;
            if (fits(ax, ay) && (best == 0 || cost(ax, ay) < best_cost)) {
                best = ax;
                best_cost = cost(ax, ay);
            }
        }
        return best;
    }
    static constexpr int AX = pick_ax();                 // 0: the grid cannot be cut into eight equal rectangles
    static constexpr int AY = AX ? 8 / AX : 0;
    BFUSE_HD static constexpr Dims3 tile(int id)
    {
        if constexpr (AX == 0) {
            return Dims3{id % GX, id / GX, 0};
        } else {
            constexpr int RX = GX / AX;
            const int xcd = id & 7, slot = id >> 3;
            return Dims3{(xcd % AX) * RX + slot % RX, (xcd / AX) * (GY / AY) + slot / RX, 0};
        }
    }
};

}  // namespace bfuse
