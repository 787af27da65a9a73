// Per-graph partition of a compressed structure for the merge-path kernels
// (the product of spmm.hip, the fused attention kernels of gat.hip) and the
// tile kernels (entry_tiles.hip).  Everything here depends on the offsets
// alone, so it is computed once per graph and kept by the caller; the
// reference's aggregate is a single launch per call (ops/cpp/aggregate_op.cc:93-106)
// and with a plan so is ours on graphs without long rows.
//
// Chunks.  The R row-end markers and the E entries form one sequence of
// M = R + E items; chunk k nominally starts at item k * chunk.  A boundary that
// falls inside a row of at most chunk / 2 entries is moved back to that row's
// first entry, so a short row is always summed by one wavefront, start to end,
// and only rows longer than that are ever cut into pieces.  start[k] = (row,
// entry) at which chunk k begins; start[nchunks] = (R, E).  Chunks stay within
// chunk / 2 items of their nominal size and none is empty: two boundaries can
// only be moved to the same row if that row holds both, and then it is longer
// than a chunk.
//
// Lists.  fix[] = the chunks whose first row began in an earlier chunk and ends
// in this one (its pieces have to be added up); grp[] = the groups of kPlanGroup
// chunks past whose end a row continues (their pieces are pre-summed).  Both
// ascending; their lengths sit at the start of the plan.  A plan for the product
// leaves out the groups of rows that cross at most kSpmmInlineGroups group
// boundaries: the kernel that finishes such a row sums its groups itself, and on
// a graph without longer rows no group kernel is launched at all.
#include <stdlib.h>

#include "common.h"

namespace jg {

__global__ void plan_chunk_starts(const int32_t *__restrict__ off, int R, int E, int chunk, int nchunks, int snap,
                                  int2 *__restrict__ start)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k > nchunks) return;
    if (k == nchunks) {
        start[k] = make_int2(R, E);
        return;
    }
    const int64_t p = (int64_t)k * chunk;
    int lo = 0, hi = R;                      // largest r in [0,R) with off[r] + r <= p
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)off[mid] + mid <= p) lo = mid; else hi = mid;
    }
    const int s = off[lo];
    const int len = off[lo + 1] - s;
    int j = (int)(p - lo);
    if (len <= snap && (int64_t)s + lo < p) j = s;
    start[k] = make_int2(lo, j);
}

// Ordered compaction by one workgroup: walks the candidates 1024 at a time and appends the
// selected ones in ascending order.
constexpr int kListThreads = 1024;

template <typename Pred>
__device__ __forceinline__ int compact_ascending(int n, int32_t *__restrict__ list, Pred pred)
{
    __shared__ int wave_count[kListThreads / kWave];
    int total = 0;
    const int lane = lane_id(), wv = threadIdx.x >> 6;
    for (int base = 0; base < n; base += kListThreads) {
        const int i = base + (int)threadIdx.x;
        const bool sel = i < n && pred(i);
        const unsigned long long mask = __ballot(sel);
        const int rank = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_count[wv] = __popcll(mask);
        __syncthreads();
        int before = 0, all = 0;
        for (int u = 0; u < kListThreads / kWave; u++) {
            const int c = wave_count[u];
            if (u < wv) before += c;
            all += c;
        }
        if (sel) list[total + before + rank] = i;
        total += all;
        __syncthreads();
    }
    return total;
}

__global__ __launch_bounds__(kListThreads) void plan_chunk_lists(const int32_t *__restrict__ off,
                                                                 const int2 *__restrict__ start, int R, int chunk,
                                                                 int nchunks, int inline_groups,
                                                                 int32_t *__restrict__ fix, int32_t *__restrict__ grp,
                                                                 int32_t *__restrict__ header)
{
    const int n_fix = compact_ascending(nchunks, fix, [&](int k) {
        const int2 a = start[k], b = start[k + 1];
        return a.x < R && b.x > a.x && a.y > off[a.x];
    });
    const int ngroups = (nchunks + kPlanGroup - 1) / kPlanGroup;
    const int n_grp = compact_ascending(ngroups, grp, [&](int g) {
        const int kend = (g + 1) * kPlanGroup;
        if (kend >= nchunks) return false;
        const int2 a = start[kend];
        if (a.x < 0 || a.x >= R || a.y <= off[a.x]) return false;
        // a cut row begins in the chunk of its first item and ends in that of its end marker
        const int64_t r = a.x;
        const int first = (int)((max(off[r], 0) + r) / chunk), last = (int)((max(off[r + 1], 0) + r) / chunk);
        return last / kPlanGroup - first / kPlanGroup > inline_groups;
    });
    if (threadIdx.x == 0) {
        header[0] = n_fix;
        header[1] = n_grp;
        header[2] = nchunks;
        header[3] = R;
    }
}

// Tiles.  tile_first[i] / tile_last[i] = column of the first / last covered entry of tile i
// (tiles of T entries).  One thread per tile finds both by bisection of the offsets: the column
// of entry p is the largest c with off[c] <= p (of several columns that share an offset, empty
// ones followed by the one that holds p, that is the last).  A column with millions of entries
// costs what any other costs.  Tiles without a covered entry keep what the arrays held.
__device__ __forceinline__ int column_of_entry(const int32_t *__restrict__ off, int V, int p)
{
    int lo = 0, hi = V;                      // largest c in [0,V) with off[c] <= p
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (off[mid] <= p) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ void plan_tile_columns(const int32_t *__restrict__ off, int V, int E, int T, int32_t *__restrict__ tile_first,
                                  int32_t *__restrict__ tile_last)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int covered = min(max(off[V], 0), E);
    const int ntiles = (covered + T - 1) / T;
    if (i >= ntiles) return;
    const int64_t first = (int64_t)i * T;
    const int last = (int)min(first + T, (int64_t)covered) - 1;
    tile_first[i] = column_of_entry(off, V, (int)first);
    tile_last[i] = column_of_entry(off, V, last);
}

int plan_chunk_for(int kind, int64_t M)
{
    if (kind == JGAMD_PLAN_GAT) return gat_chunk_for(M);
    return spmm_chunk_for(M);
}

ChunkPlanShape chunk_plan_shape(int kind, int32_t R, int64_t E)
{
    ChunkPlanShape s{};
    const int64_t M = (int64_t)R + E;
    s.chunk = plan_chunk_for(kind, M);
    s.nchunks = (int)ceil_div(M > 0 ? M : 1, s.chunk);
    s.ngroups = (int)ceil_div(s.nchunks, kPlanGroup);
    s.header_bytes = 256;
    s.start_bytes = carve_bytes((size_t)s.nchunks + 1, sizeof(int2));
    s.fix_bytes = carve_bytes((size_t)s.nchunks, 4);
    s.grp_bytes = carve_bytes((size_t)s.ngroups, 4);
    return s;
}

size_t chunk_plan_bytes(int kind, int32_t R, int64_t E)
{
    const ChunkPlanShape s = chunk_plan_shape(kind, R, E);
    return s.header_bytes + s.start_bytes + s.fix_bytes + s.grp_bytes;
}

ChunkPlan chunk_plan_view(int kind, int32_t R, int64_t E, const void *plan)
{
    const ChunkPlanShape s = chunk_plan_shape(kind, R, E);
    const char *p = static_cast<const char *>(plan);
    ChunkPlan v{};
    v.chunk = s.chunk;
    v.nchunks = s.nchunks;
    v.counts = reinterpret_cast<const int32_t *>(p);
    v.start = reinterpret_cast<const int2 *>(p + s.header_bytes);
    v.fix = reinterpret_cast<const int32_t *>(p + s.header_bytes + s.start_bytes);
    v.grp = reinterpret_cast<const int32_t *>(p + s.header_bytes + s.start_bytes + s.fix_bytes);
    return v;
}

void chunk_starts_enqueue(const int32_t *off, int32_t R, int64_t E, int chunk, int nchunks, int2 *start, hipStream_t s)
{
    // tuning aid, read once per process: the longest row kept whole, in percent of a chunk (below 100)
    static const int pct = [] {
        const char *e = getenv("JGAMD_PLAN_SNAP");
        const int v = e ? atoi(e) : 50;
        return v < 0 ? 0 : (v > 99 ? 99 : v);
    }();
    hipLaunchKernelGGL(plan_chunk_starts, dim3((unsigned)ceil_div(nchunks + 1, 256)), dim3(256), 0, s, off, R, (int)E,
                       chunk, nchunks, chunk * pct / 100, start);
}

size_t tile_plan_bytes(int64_t E)
{
    // (first, last) per tile for the two tile sizes of entry_tiles.hip
    size_t total = 0;
    for (int T : {kTileEntriesWide, kTileEntriesNarrow}) total += 2 * carve_bytes((size_t)ceil_div(E > 0 ? E : 1, T), 4);
    return total;
}

TilePlan tile_plan_view(int64_t E, int T, const void *plan)
{
    const char *p = static_cast<const char *>(plan);
    for (int t : {kTileEntriesWide, kTileEntriesNarrow}) {
        const size_t one = carve_bytes((size_t)ceil_div(E > 0 ? E : 1, t), 4);
        if (t == T) {
            TilePlan v{};
            v.tile_first = reinterpret_cast<const int32_t *>(p);
            v.tile_last = reinterpret_cast<const int32_t *>(p + one);
            return v;
        }
        p += 2 * one;
    }
    return TilePlan{};
}

void tile_columns_enqueue(const int32_t *off, int32_t V, int64_t E, int T, int32_t *tile_first, int32_t *tile_last,
                          hipStream_t s)
{
    hipLaunchKernelGGL(plan_tile_columns, dim3((unsigned)ceil_div(ceil_div(E > 0 ? E : 1, T), 256)), dim3(256), 0, s, off,
                       V, (int)E, T, tile_first, tile_last);
}

}  // namespace jg

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

static int32_t check_plan(const char *who, int32_t R, int64_t E, int32_t kind)
{
    if (R < 0 || E < 0) return fail(JGAMD_ERR_SIZE, "%s: negative size", who);
    if ((int64_t)R + E >= ((int64_t)1 << 31) - 4096)
        return fail(JGAMD_ERR_SIZE, "%s: R + E = %lld does not fit int32", who, (long long)((int64_t)R + E));
    if (kind != JGAMD_PLAN_SPMM && kind != JGAMD_PLAN_GAT && kind != JGAMD_PLAN_TILES)
        return fail(JGAMD_ERR_SIZE, "%s: kind = %d is none of JGAMD_PLAN_SPMM / _GAT / _TILES", who, kind);
    return 0;
}

JG_EXPORT int32_t jgamd_csx_plan_bytes(int32_t R, int64_t E, int32_t kind, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "csx_plan_bytes: bytes is NULL");
    if (int32_t rc = check_plan("csx_plan_bytes", R, E, kind)) return rc;
    *bytes = kind == JGAMD_PLAN_TILES ? tile_plan_bytes(E) : chunk_plan_bytes(kind, R, E);
    return 0;
}

JG_EXPORT int32_t jgamd_csx_plan(const int32_t *off, int32_t R, int64_t E, int32_t kind, void *plan, size_t plan_bytes,
                                 void *stream)
{
    if (int32_t rc = check_plan("csx_plan", R, E, kind)) return rc;
    if (!off || !plan) return fail(JGAMD_ERR_NULL, "csx_plan: off / plan is NULL");
    if (((uintptr_t)plan & 255) != 0) return fail(JGAMD_ERR_ALIGN, "csx_plan: plan not 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kind == JGAMD_PLAN_TILES) {
        const size_t need = tile_plan_bytes(E);
        if (plan_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "csx_plan: plan of %zu bytes needed, got %zu", need, plan_bytes);
        if (R == 0 || E == 0) return 0;
        for (int T : {kTileEntriesWide, kTileEntriesNarrow}) {
            const TilePlan v = tile_plan_view(E, T, plan);
            tile_columns_enqueue(off, R, E, T, const_cast<int32_t *>(v.tile_first), const_cast<int32_t *>(v.tile_last), s);
        }
        return launch_status("csx_plan");
    }
    const size_t need = chunk_plan_bytes(kind, R, E);
    if (plan_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "csx_plan: plan of %zu bytes needed, got %zu", need, plan_bytes);
    if (R == 0) return 0;
    const ChunkPlan v = chunk_plan_view(kind, R, E, plan);
    chunk_starts_enqueue(off, R, E, v.chunk, v.nchunks, const_cast<int2 *>(v.start), s);
    hipLaunchKernelGGL(plan_chunk_lists, dim3(1), dim3(kListThreads), 0, s, off, v.start, R, v.chunk, v.nchunks,
                       kind == JGAMD_PLAN_SPMM ? kSpmmInlineGroups : 0, const_cast<int32_t *>(v.fix), const_cast<int32_t *>(v.grp), const_cast<int32_t *>(v.counts));
    return launch_status("csx_plan");
}

JG_EXPORT int32_t jgamd_csx_plan_counts(const void *plan, int32_t *n_fix, int32_t *n_grp, void *stream)
{
    if (!plan || !n_fix || !n_grp) return fail(JGAMD_ERR_NULL, "csx_plan_counts: NULL argument");
    int32_t host[2] = {0, 0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(host, plan, sizeof(host), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail((int32_t)e, "csx_plan_counts: %s", hipGetErrorString(e));
    *n_fix = host[0];
    *n_grp = host[1];
    return 0;
}
