// Per-column work over fixed tiles of entries: edge softmax for H in {1, 2, 4, 8}
// heads, and the gather-sum for rows of 1, 2, 4 or 8 floats (further down).
//
// The reference (ops/cpp/edgesoftmax_op.cc:48-65, edgesoftmaxbackward_op.cc:45-51)
// walks every destination column three times.  Columns of a power-law graph
// run from one entry to millions, so here the unit of work is not a column
// but a tile of T consecutive entries of the [E,H] array:
//
//   0. tile columns : one thread per column records, for every tile, the
//                     column of its first and of its last entry (plan.hip;
//                     once per graph when the caller keeps a tile plan).
//   1. tile kernel  : a lane holds K consecutive entries (all H heads, loaded
//                     as vectors).  The tile's columns mark their first entry
//                     in a bitmap in LDS; a lane reads the K bits of its
//                     entries and never learns a column id.  Per-column totals
//                     (max, then sum of exp; or sum of y*g): runs of one column
//                     inside a lane are folded in registers, the run that
//                     reaches a lane from the lanes before it and the run that
//                     leaves it go through one segmented scan over the block's
//                     lanes and a table in LDS indexed by the position of the
//                     column's first entry, in a fixed order (no float atomics).
//                     Columns that lie inside the tile are finished from
//                     registers: x is read once, y written once.  A column
//                     that crosses a tile edge leaves a piece per tile.
//   2. merge kernel : one wavefront per column that crosses tile edges folds
//                     its pieces (tail piece of the tile it starts in, then
//                     the head pieces of the following tiles).
//   3. finish kernel: the entries of crossing columns are computed from the
//                     inputs with the merged totals.
//
// A column's slot in a tile is the position of its first entry inside the
// tile (0 for the column that began in an earlier tile), so slots are unique
// and below T.
#include "common.h"

namespace jg {

constexpr int kFlatThreads = 256;
constexpr int kFlatWaves = kFlatThreads / kWave;

template <int H> struct FlatShape {
    static constexpr int K = H <= 2 ? 8 : 4;        // entries per lane
    static constexpr int T = kFlatThreads * K;      // entries per tile
    static_assert(T == (H <= 2 ? kTileEntriesWide : kTileEntriesNarrow), "tile sizes of the tile plan");
};

struct FlatMeta {
    int head_open;   // the tile's first column began in an earlier tile
    int head_cs, head_ce;
    int tail_open;   // the tile's last column continues in the next tile
    int tail_cs, tail_ce;
    int tail_col;    // id of the tile's last column
    int pad1;
};

// The tile's T*H floats pass through LDS twice: loaded with consecutive lanes
// on consecutive 16-byte vectors (whole cache lines per instruction), read
// back as K*H consecutive floats per lane, and the other way round for the
// result.  Four floats of padding per 32 keep the per-lane reads off each
// other's banks.  The same memory then holds the per-column totals.
__host__ __device__ constexpr int flat_pad(int f) { return f + (f >> 5) * 4; }

template <int H, int T> struct FlatLds {
    unsigned bits[T / 32 + 1];      // bit p: a column begins at entry p of the tile; the last word stays zero
    int edge[4];                    // off[c_lo], off[c_lo + 1], off[c_hi], off[c_hi + 1]
    __attribute__((aligned(16))) float tot[flat_pad(T * H)];
    float carry[kFlatWaves * H];
    int wflag[kFlatWaves];
    int wmax[kFlatWaves];
};

struct OpMax {
    // The bare instruction: fmaxf() first passes each operand through a max with itself (it must
    // quiet signalling NaNs), which doubles the instructions of a pass that is nothing but
    // maxima.  Volatile so that it stays where it is written, ahead of the select that follows,
    // instead of moving into a branch of its own.  A NaN operand gives a NaN column either way.
    __device__ __forceinline__ float operator()(float a, float b) const
    {
        float r;
        asm volatile("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
        return r;
    }
};
struct OpAdd {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

// Entries the offsets cover: off[V], clamped to the length of the per-entry arrays.
__device__ __forceinline__ int covered_entries(const int32_t *__restrict__ off, int V, int E)
{
    return min(max(off[V], 0), E);
}

// A tile that holds no covered entry: no column is open in it, and (zero_out) its slots of the
// per-entry result are zero.  Returns true if the calling block has nothing else to do.
template <int H, int T>
__device__ __forceinline__ bool skip_uncovered_tile(int t0, int covered, int E, FlatMeta *meta_out, float *out)
{
    // slots past the covered entries, in this tile
    if (out) {
        const int64_t lo = (int64_t)max(t0, covered) * H, hi = (int64_t)min(t0 + T, E) * H;
        for (int64_t p = lo + threadIdx.x; p < hi; p += kFlatThreads) out[p] = 0.f;
    }
    if (t0 < covered) return false;
    if (threadIdx.x == 0) {
        FlatMeta m;
        m.head_open = m.tail_open = 0;
        m.head_cs = m.head_ce = m.tail_cs = m.tail_ce = covered;
        m.tail_col = 0;
        m.pad1 = 0;
        *meta_out = m;
    }
    return true;
}

// What a lane knows about the columns of its K entries.
template <int K> struct LaneColumns {
    unsigned starts;            // bit k: a column begins at the lane's entry k
    int first_slot, last_slot;  // slots of the columns of the lane's first and last entry
    bool ends_here;             // the column of the lane's last entry ends with that entry (or the tile does)
    unsigned closed;            // bit k: entry k is valid and its column lies inside the tile
    int tail_slot;              // slot of the tile's last column
    int closed_lo, closed_hi;   // the valid entries of columns inside the tile, relative to t0
};

// One step of an inclusive maximum scan over the wavefront (values >= 0; lanes
// without a source keep their own).
template <int CTRL, int ROWS> __device__ __forceinline__ int max_scan_step(int v)
{
    return max(v, __builtin_amdgcn_update_dpp(0, v, CTRL, ROWS, 0xf, false));
}

// The value of the lane before (wave_shr:1); lane 0 receives `first`.
__device__ __forceinline__ int from_lane_before(int v, int first)
{
    return __builtin_amdgcn_update_dpp(first, v, 0x138, 0xf, 0xf, false);
}
__device__ __forceinline__ float from_lane_before(float v, float first)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(first), __float_as_int(v), 0x138, 0xf, 0xf, false));
}

// Marks the first entries of the tile's columns [c_lo, c_hi] in L.bits and gives every lane the
// bits of its K entries and the slots of its first and last column (entries past the tile's end
// belong to the column of the tile's last entry).  Thread 0 records the tile's metadata.
// Contains barriers; L.bits and L.edge stay valid afterwards.
template <int H, int K, int T>
__device__ __forceinline__ void resolve_columns(const int32_t *__restrict__ off, int c_lo, int c_hi, int t0, int n,
                                                FlatLds<H, T> &L, LaneColumns<K> &cols, FlatMeta *meta_out)
{
    static_assert(32 % K == 0 && T / 32 + 1 <= kFlatThreads, "a lane's bits lie in one word");
    const int tid = threadIdx.x;
    if (tid <= T / 32) L.bits[tid] = 0;
    if (tid < 4) L.edge[tid] = off[tid < 2 ? c_lo + tid : c_hi + tid - 2];
    __syncthreads();
    // empty columns repeat the position of the column after them; positions outside the tile
    // (offsets that are not monotone) are left out
    for (int c = c_lo + tid; c <= c_hi; c += kFlatThreads) {
        const int pos = off[c] - t0;
        if (pos >= 0 && pos < n) atomicOr(&L.bits[pos >> 5], 1u << (pos & 31));
    }
    __syncthreads();
    const int p0 = tid * K;
    cols.starts = (L.bits[p0 >> 5] >> (p0 & 31)) & ((1u << K) - 1u);
    cols.ends_here = tid == kFlatThreads - 1 || ((L.bits[(p0 + K) >> 5] >> ((p0 + K) & 31)) & 1u);
    // slot of a lane's last column: the latest first entry at or before the lane's end
    const int own = cols.starts ? p0 + 31 - __clz((int)cols.starts) : 0;
    int incl = own;
    incl = max_scan_step<0x111, 0xf>(incl);
    incl = max_scan_step<0x112, 0xf>(incl);
    incl = max_scan_step<0x114, 0xf>(incl);
    incl = max_scan_step<0x118, 0xf>(incl);
    incl = max_scan_step<0x142, 0xa>(incl);
    incl = max_scan_step<0x143, 0xc>(incl);
    const int w = uniform(tid >> 6);
    if (lane_id() == kWave - 1) L.wmax[w] = incl;
    __syncthreads();
    int before = 0;
#pragma unroll
    for (int u = 0; u < kFlatWaves - 1; u++)
        if (u < w) before = max(before, L.wmax[u]);
    const int prev = max(before, from_lane_before(incl, 0));
    cols.first_slot = (cols.starts & 1u) ? p0 : prev;
    cols.last_slot = max(prev, own);
    const int e0 = L.edge[0], e1 = L.edge[1], e2 = L.edge[2], e3 = L.edge[3];
    const bool head_open = e0 < t0, tail_open = e3 > t0 + n;
    cols.tail_slot = min(max(e2 - t0, 0), T - 1);     // the upper clamp only matters for inconsistent offsets
    cols.closed_lo = head_open ? min(max(e1 - t0, 0), n) : 0;
    cols.closed_hi = tail_open ? min(max(e2 - t0, cols.closed_lo), n) : n;
    const int lo_k = min(max(cols.closed_lo - p0, 0), K), hi_k = min(max(cols.closed_hi - p0, 0), K);
    cols.closed = ((1u << hi_k) - 1u) & ~((1u << lo_k) - 1u);
    if (tid == 0) {
        FlatMeta m;
        m.head_cs = e0;
        m.head_ce = e1;
        m.head_open = head_open;
        m.tail_cs = e2;
        m.tail_ce = e3;
        m.tail_open = tail_open;
        m.tail_col = c_hi;
        m.pad1 = 0;
        *meta_out = m;
    }
}

// One step of an inclusive segmented scan over the wavefront: lanes that the
// move reaches and that have seen no segment start yet fold the moved value in.
// CTRL: row_shr:n = 0x110+n, row_bcast:15 = 0x142, row_bcast:31 = 0x143; lanes
// without a source (or outside ROWS) receive the identity and no flag.
template <int CTRL, int ROWS, int H, typename Op>
__device__ __forceinline__ void seg_scan_step(float (&v)[H], int &fl, Op op, float ident)
{
    const int fu = __builtin_amdgcn_update_dpp(0, fl, CTRL, ROWS, 0xf, false);
#pragma unroll
    for (int h = 0; h < H; h++) {
        const float up = __int_as_float(
            __builtin_amdgcn_update_dpp(__float_as_int(ident), __float_as_int(v[h]), CTRL, ROWS, 0xf, false));
        const float folded = op(up, v[h]);
        v[h] = fl ? v[h] : folded;
    }
    fl |= fu;
}

// The H totals of one slot.
template <int H> __device__ __forceinline__ void read_totals(const float *tot, int slot, float (&t)[H])
{
    if constexpr (H >= 4) {
#pragma unroll
        for (int q = 0; q < H / 4; q++) {
            const float4 v = *reinterpret_cast<const float4 *>(tot + slot * H + 4 * q);
            t[4 * q] = v.x;
            t[4 * q + 1] = v.y;
            t[4 * q + 2] = v.z;
            t[4 * q + 3] = v.w;
        }
    } else if constexpr (H == 2) {
        const float2 v = *reinterpret_cast<const float2 *>(tot + slot * 2);
        t[0] = v.x;
        t[1] = v.y;
    } else {
        t[0] = tot[slot];
    }
}

// tot[k] = the fold of val over the whole column of the lane's entry k, as far as the column
// lies in the tile.  Entries that do not count must hold the identity.  A run that begins and
// ends inside the lane never leaves its registers; the lane's first run (it may reach back
// into earlier lanes) and its last (it may go on in later ones) are completed by the segmented
// scan, and the lane in which a column ends publishes its total in L.tot[slot].  Afterwards
// L.tot holds the totals of every column that crosses a lane edge, the tile's first column
// (slot 0) and its last (tail_slot) among them; TABLE adds the columns inside one lane, and
// a barrier, so that L.tot can be read for any column that begins in the tile.
template <int H, int K, int T, bool TABLE = false, typename Op>
__device__ __forceinline__ void segment_totals(const float (&val)[K][H], const LaneColumns<K> &cols, FlatLds<H, T> &L,
                                               Op op, float ident, float (&tot)[K][H])
{
    const int lane = lane_id();
    const int w = uniform(threadIdx.x >> 6);
    bool st[K];
#pragma unroll
    for (int k = 0; k < K; k++) st[k] = (cols.starts >> k) & 1u;
    // a[k]: fold of the entries of k's run up to k, inside the lane
    float a[K][H];
#pragma unroll
    for (int h = 0; h < H; h++) a[0][h] = val[0][h];
#pragma unroll
    for (int k = 1; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) {
            const float folded = op(a[k - 1][h], val[k][h]);     // computed either way: a select, not a branch
            a[k][h] = st[k] ? val[k][h] : folded;
        }
    // inclusive segmented scan of the last runs: a lane in which a column begins starts a segment.
    // Rows of 16 lanes with row shifts, then lane 15 -> next row (rows 1, 3) and lane 31 -> rows
    // 2, 3: all data-parallel moves on the vector ALU (a step changes nothing once every lane
    // has seen a segment start)
    int fl = cols.starts != 0;
    float v[H];
#pragma unroll
    for (int h = 0; h < H; h++) v[h] = a[K - 1][h];
    seg_scan_step<0x111, 0xf>(v, fl, op, ident);
    seg_scan_step<0x112, 0xf>(v, fl, op, ident);
    if (__ballot(fl == 0)) {
        seg_scan_step<0x114, 0xf>(v, fl, op, ident);
        seg_scan_step<0x118, 0xf>(v, fl, op, ident);
        if (__ballot(fl == 0)) {
            seg_scan_step<0x142, 0xa>(v, fl, op, ident);
            seg_scan_step<0x143, 0xc>(v, fl, op, ident);
        }
    }
    if (lane == kWave - 1) {
#pragma unroll
        for (int h = 0; h < H; h++) L.carry[w * H + h] = v[h];
        L.wflag[w] = fl;
    }
    __syncthreads();
    float carry[H];
#pragma unroll
    for (int h = 0; h < H; h++) carry[h] = ident;
#pragma unroll
    for (int u = 0; u < kFlatWaves - 1; u++)
        if (u < w) {
            const bool cut = L.wflag[u] != 0;
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float folded = op(carry[h], L.carry[u * H + h]);
                carry[h] = cut ? L.carry[u * H + h] : folded;
            }
        }
    // the column that ends inside this lane after reaching it from the lanes before: its total is
    // what those lanes hold plus this lane's entries below its first column start
    const bool head_ends = cols.starts != 0 && !(cols.starts & 1u);
    float head_total[H];
#pragma unroll
    for (int h = 0; h < H; h++) {
        const float with_carry = op(carry[h], v[h]);
        v[h] = fl ? v[h] : with_carry;
        const float prev = from_lane_before(v[h], carry[h]);
        float hd = a[K - 1][h];
#pragma unroll
        for (int k = K - 1; k >= 1; k--) hd = st[k] ? a[k - 1][h] : hd;
        head_total[h] = op(prev, hd);
        if (head_ends) L.tot[cols.first_slot * H + h] = head_total[h];
        if (cols.ends_here) L.tot[cols.last_slot * H + h] = v[h];
    }
    __syncthreads();
    float run[H];
    read_totals<H>(L.tot, cols.last_slot, run);
    const int k0 = cols.starts ? __builtin_ctz(cols.starts) : 0;     // entries below k0: the column that ends here
#pragma unroll
    for (int k = K - 1; k >= 0; k--) {
#pragma unroll
        for (int h = 0; h < H; h++) {
            tot[k][h] = k < k0 ? head_total[h] : run[h];
            if (k >= 1) run[h] = st[k] ? a[k - 1][h] : run[h];
        }
    }
    if constexpr (TABLE) {
        // columns inside the lane (the last run is published by the lane it ends in)
        const int top = cols.starts ? 31 - __clz((int)cols.starts) : 0;
#pragma unroll
        for (int k = 0; k < K; k++)
            if (st[k] && k != top) {
#pragma unroll
                for (int h = 0; h < H; h++) L.tot[((int)threadIdx.x * K + k) * H + h] = tot[k][h];
            }
        __syncthreads();
    }
}

template <int N> struct __attribute__((aligned(N >= 4 ? 16 : 4 * N))) FloatVec {
    float f[N];
};

// Lane's K*H consecutive floats starting at entry j0: one vector access when
// the arrays are 16-byte aligned and the lane is inside the array, else
// element by element with the entry index clamped.
template <int H, int K>
__device__ __forceinline__ void load_lane(const float *__restrict__ a, bool aligned, int j0, int E, float (&v)[K][H])
{
    if (aligned && j0 + K <= E) {
        const FloatVec<K * H> t = *reinterpret_cast<const FloatVec<K * H> *>(a + (int64_t)j0 * H);
#pragma unroll
        for (int k = 0; k < K; k++)
#pragma unroll
            for (int h = 0; h < H; h++) v[k][h] = t.f[k * H + h];
    } else {
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int64_t j = min(j0 + k, E - 1);
#pragma unroll
            for (int h = 0; h < H; h++) v[k][h] = a[j * H + h];
        }
    }
}

template <int H, int K>
__device__ __forceinline__ void store_lane(float *__restrict__ a, bool aligned, int j0, unsigned mask,
                                           const float (&v)[K][H])
{
    if (aligned && mask == (1u << K) - 1) {
        FloatVec<K * H> t;
#pragma unroll
        for (int k = 0; k < K; k++)
#pragma unroll
            for (int h = 0; h < H; h++) t.f[k * H + h] = v[k][h];
        *reinterpret_cast<FloatVec<K * H> *>(a + (int64_t)j0 * H) = t;
    } else {
#pragma unroll
        for (int k = 0; k < K; k++)
            if (mask >> k & 1) {
#pragma unroll
                for (int h = 0; h < H; h++) a[(int64_t)(j0 + k) * H + h] = v[k][h];
            }
    }
}

// Tile [t0, t0+T) of a[E][H] -> v, through LDS (see FlatLds).  Needs a 16-byte
// aligned array; positions past the array's end repeat its last element.
// Ends with the lanes' reads still in flight on `buf`: a barrier must follow
// before buf is written again.
template <int H, int K>
__device__ __forceinline__ void load_tile(const float *__restrict__ a, int t0, int E, float *buf, float (&v)[K][H])
{
    constexpr int NV = K * H / 4;
    const int64_t total = (int64_t)E * H;
    float4 q[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int f = (i * kFlatThreads + threadIdx.x) * 4;
        const int64_t g = (int64_t)t0 * H + f;
        if (g + 4 <= total) {
            q[i] = *reinterpret_cast<const float4 *>(a + g);
        } else {
            q[i].x = a[min(g, total - 1)];
            q[i].y = a[min(g + 1, total - 1)];
            q[i].z = a[min(g + 2, total - 1)];
            q[i].w = a[min(g + 3, total - 1)];
        }
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int f = (i * kFlatThreads + threadIdx.x) * 4;
        *reinterpret_cast<float4 *>(buf + flat_pad(f)) = q[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const float4 t = *reinterpret_cast<const float4 *>(buf + flat_pad((int)threadIdx.x * K * H + 4 * i));
        const float c[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int j = 0; j < 4; j++) v[(4 * i + j) / H][(4 * i + j) % H] = c[j];
    }
}

// v -> out for the entries [lo, hi) of the tile (relative to t0), through LDS.
// Starts with a barrier (buf may still be read as totals).
template <int H, int K>
__device__ __forceinline__ void store_tile(float *__restrict__ out, int t0, int lo, int hi, float *buf,
                                           const float (&v)[K][H])
{
    constexpr int NV = K * H / 4;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; i++) {
        float4 t;
        t.x = v[(4 * i) / H][(4 * i) % H];
        t.y = v[(4 * i + 1) / H][(4 * i + 1) % H];
        t.z = v[(4 * i + 2) / H][(4 * i + 2) % H];
        t.w = v[(4 * i + 3) / H][(4 * i + 3) % H];
        *reinterpret_cast<float4 *>(buf + flat_pad((int)threadIdx.x * K * H + 4 * i)) = t;
    }
    __syncthreads();
    const int flo = lo * H, fhi = hi * H;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int f = (i * kFlatThreads + threadIdx.x) * 4;
        const float4 t = *reinterpret_cast<const float4 *>(buf + flat_pad(f));
        float *dst = out + (int64_t)t0 * H + f;
        if (f >= flo && f + 4 <= fhi) {
            *reinterpret_cast<float4 *>(dst) = t;
        } else {
            if (f >= flo && f < fhi) dst[0] = t.x;
            if (f + 1 >= flo && f + 1 < fhi) dst[1] = t.y;
            if (f + 2 >= flo && f + 2 < fhi) dst[2] = t.z;
            if (f + 3 >= flo && f + 3 < fhi) dst[3] = t.w;
        }
    }
}

__device__ __forceinline__ bool both_aligned(const void *a, const void *b)
{
    return (((uintptr_t)a | (uintptr_t)b) & 15) == 0;
}

// pieces: [ntiles][2][2H] floats; index 0 = head column, 1 = tail column;
// forward: H maxima then H sums (relative to those maxima); backward: H sums.
template <int H> __device__ __forceinline__ float *piece(float *pieces, int tile, int which)
{
    return pieces + ((int64_t)tile * 2 + which) * 2 * H;
}

template <int H>
__global__ __launch_bounds__(kFlatThreads) void esm_fwd_tile(const int32_t *__restrict__ off,
                                                             const float *__restrict__ x, float *__restrict__ y,
                                                             const int32_t *__restrict__ tile_first,
                                                             const int32_t *__restrict__ tile_last, int V, int E,
                                                             FlatMeta *__restrict__ meta, float *__restrict__ pieces,
                                                             int staged)
{
    constexpr int K = FlatShape<H>::K, T = FlatShape<H>::T;
    __shared__ FlatLds<H, T> L;
    const int tile = blockIdx.x;
    const int t0 = tile * T;
    const int covered = covered_entries(off, V, E);
    if (skip_uncovered_tile<H, T>(t0, covered, E, meta + tile, y)) return;
    // the clamps only matter for offsets that are not monotone
    const int c_lo = min(max(tile_first[tile], 0), V - 1);
    const int c_hi = min(max(tile_last[tile], c_lo), V - 1);
    const int n = min(T, covered - t0);
    const int j0 = t0 + threadIdx.x * K;
    const bool aligned = both_aligned(x, y);
    const bool through_lds = aligned && staged;
    float v[K][H];
    if (through_lds) load_tile<H, K>(x, t0, E, L.tot, v);
    else load_lane<H, K>(x, aligned, j0, E, v);
    LaneColumns<K> cols;
    resolve_columns<H, K, T>(off, c_lo, c_hi, t0, n, L, cols, meta + tile);
    const bool partial = n < T;      // only the last covered tile holds entries that do not count
    if (partial) {
#pragma unroll
        for (int k = 0; k < K; k++)
            if (j0 + k >= t0 + n) {
#pragma unroll
                for (int h = 0; h < H; h++) v[k][h] = -INFINITY;
            }
    }
    float t[K][H];
    segment_totals<H, K, T>(v, cols, L, OpMax(), -INFINITY, t);
    const int tail_slot = cols.tail_slot;
    if (threadIdx.x < H) {
        piece<H>(pieces, tile, 0)[threadIdx.x] = L.tot[threadIdx.x];
        piece<H>(pieces, tile, 1)[threadIdx.x] = L.tot[tail_slot * H + threadIdx.x];
    }
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) v[k][h] = __expf(v[k][h] - t[k][h]);
    if (partial) {
#pragma unroll
        for (int k = 0; k < K; k++)
            if (j0 + k >= t0 + n) {
#pragma unroll
                for (int h = 0; h < H; h++) v[k][h] = 0.f;
            }
    }
    segment_totals<H, K, T>(v, cols, L, OpAdd(), 0.f, t);
    if (threadIdx.x < H) {
        piece<H>(pieces, tile, 0)[H + threadIdx.x] = L.tot[threadIdx.x];
        piece<H>(pieces, tile, 1)[H + threadIdx.x] = L.tot[tail_slot * H + threadIdx.x];
    }
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) v[k][h] = v[k][h] * __builtin_amdgcn_rcpf(t[k][h]);
    if (through_lds) store_tile<H, K>(y, t0, cols.closed_lo, cols.closed_hi, L.tot, v);
    else store_lane<H, K>(y, aligned, j0, cols.closed, v);
}

template <int H>
__global__ __launch_bounds__(kFlatThreads) void esm_bwd_tile(const int32_t *__restrict__ off,
                                                             const float *__restrict__ y, const float *__restrict__ g,
                                                             float *__restrict__ dx,
                                                             const int32_t *__restrict__ tile_first,
                                                             const int32_t *__restrict__ tile_last, int V, int E,
                                                             FlatMeta *__restrict__ meta, float *__restrict__ pieces,
                                                             int staged)
{
    constexpr int K = FlatShape<H>::K, T = FlatShape<H>::T;
    __shared__ FlatLds<H, T> L;
    const int tile = blockIdx.x;
    const int t0 = tile * T;
    const int covered = covered_entries(off, V, E);
    if (skip_uncovered_tile<H, T>(t0, covered, E, meta + tile, dx)) return;
    // the clamps only matter for offsets that are not monotone
    const int c_lo = min(max(tile_first[tile], 0), V - 1);
    const int c_hi = min(max(tile_last[tile], c_lo), V - 1);
    const int n = min(T, covered - t0);
    const int j0 = t0 + threadIdx.x * K;
    const bool aligned = both_aligned(y, g) && ((uintptr_t)dx & 15) == 0;
    const bool through_lds = aligned && staged;
    float yv[K][H], yg[K][H];
    if (through_lds) {
        load_tile<H, K>(y, t0, E, L.tot, yv);
        __syncthreads();
        load_tile<H, K>(g, t0, E, L.tot, yg);
    } else {
        load_lane<H, K>(y, aligned, j0, E, yv);
        load_lane<H, K>(g, aligned, j0, E, yg);
    }
    LaneColumns<K> cols;
    resolve_columns<H, K, T>(off, c_lo, c_hi, t0, n, L, cols, meta + tile);
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) yg[k][h] = yv[k][h] * yg[k][h];
    if (n < T) {
#pragma unroll
        for (int k = 0; k < K; k++)
            if (j0 + k >= t0 + n) {
#pragma unroll
                for (int h = 0; h < H; h++) yg[k][h] = 0.f;
            }
    }
    float t[K][H];
    segment_totals<H, K, T>(yg, cols, L, OpAdd(), 0.f, t);
    const int tail_slot = cols.tail_slot;
    if (threadIdx.x < H) {
        piece<H>(pieces, tile, 0)[threadIdx.x] = L.tot[threadIdx.x];
        piece<H>(pieces, tile, 1)[threadIdx.x] = L.tot[tail_slot * H + threadIdx.x];
    }
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) yg[k][h] = yg[k][h] - yv[k][h] * t[k][h];
    if (through_lds) store_tile<H, K>(dx, t0, cols.closed_lo, cols.closed_hi, L.tot, yg);
    else store_lane<H, K>(dx, aligned, j0, cols.closed, yg);
}

// ---- narrow-row gather-sum on the same tiles ---------------------------------
// out[c,:] = sum over the entries j of column c of w[j] * x[idx[j],:] for rows of
// H = 1, 2, 4 or 8 floats (idx == nullptr: x[j,:], w == nullptr: weight one).  The
// wide-row kernel gives a whole wavefront to one entry; with a handful of floats
// per row that leaves most lanes idle, so here a lane gathers K entries and the
// per-column totals come from the segmented scan.  Columns inside the tile are
// written by the tile kernel, crossing ones by esm_merge.  Empty columns hold no
// entry of any tile: a tile answers for the empty ones between the previous
// tile's last column and its own last column (the last covered tile for those
// after it as well) and writes their zeros.

template <int H>
__global__ __launch_bounds__(kFlatThreads) void esm_colsum_tile(const int32_t *__restrict__ off,
                                                                const int32_t *__restrict__ idx,
                                                                const float *__restrict__ w,
                                                                const float *__restrict__ x, float *__restrict__ out,
                                                                const int32_t *__restrict__ tile_first,
                                                                const int32_t *__restrict__ tile_last, int V, int C,
                                                                int E, FlatMeta *__restrict__ meta,
                                                                float *__restrict__ pieces)
{
    constexpr int K = FlatShape<H>::K, T = FlatShape<H>::T;
    __shared__ FlatLds<H, T> L;
    const int tile = blockIdx.x;
    const int t0 = tile * T;
    const int covered = covered_entries(off, V, E);
    if (covered == 0 && tile == 0)          // no entry at all: every column is empty
        for (int64_t p = threadIdx.x; p < (int64_t)V * H; p += kFlatThreads) out[p] = 0.f;
    if (skip_uncovered_tile<H, T>(t0, covered, E, meta + tile, nullptr)) return;
    const int c_lo = min(max(tile_first[tile], 0), V - 1);
    const int c_hi = min(max(tile_last[tile], c_lo), V - 1);
    const int n = min(T, covered - t0);
    const int j0 = t0 + threadIdx.x * K;
    // gathers first: (row, weight) of the lane's K entries, then the rows themselves
    int row[K];
    float wk[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int j = min(j0 + k, E - 1);
        row[k] = idx ? idx[j] : j;
        wk[k] = w ? w[j] : 1.f;
        if (j0 + k >= t0 + n || (unsigned)row[k] >= (unsigned)C) {
            row[k] = 0;
            wk[k] = 0.f;
        }
    }
    float v[K][H];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const FloatVec<H> r = *reinterpret_cast<const FloatVec<H> *>(x + (int64_t)row[k] * H);
#pragma unroll
        for (int h = 0; h < H; h++) v[k][h] = r.f[h];
    }
    LaneColumns<K> cols;
    resolve_columns<H, K, T>(off, c_lo, c_hi, t0, n, L, cols, meta + tile);
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int h = 0; h < H; h++) v[k][h] *= wk[k];
    float t[K][H];
    segment_totals<H, K, T, true>(v, cols, L, OpAdd(), 0.f, t);
    if (threadIdx.x < H) {
        piece<H>(pieces, tile, 0)[threadIdx.x] = L.tot[threadIdx.x];
        piece<H>(pieces, tile, 1)[threadIdx.x] = L.tot[cols.tail_slot * H + threadIdx.x];
    }
    // the columns that lie inside the tile, and the empty ones this tile answers for: one thread each
    const int c_from = tile == 0 ? 0 : min(max(tile_last[tile - 1] + 1, 0), c_lo);
    const int c_to = t0 + T >= covered ? V - 1 : c_hi;
    for (int c = c_from + (int)threadIdx.x; c <= c_to; c += kFlatThreads) {
        const bool inside = c >= c_lo && c <= c_hi;
        const int cs = inside ? off[c] : 0;
        const int ce = inside ? off[c + 1] : 0;
        if (ce > cs) {
            if (cs >= t0 && ce <= t0 + n) {
                float r[H];
                read_totals<H>(L.tot, cs - t0, r);
#pragma unroll
                for (int h = 0; h < H; h++) out[(int64_t)c * H + h] = r[h];
            }
        } else {
#pragma unroll
            for (int h = 0; h < H; h++) out[(int64_t)c * H + h] = 0.f;
        }
    }
}

// Folding the pieces of a column that crosses tile edges: (max, sum relative to that max) for
// the softmax, plain sums otherwise.
template <int H, bool SOFT> struct PieceFold {
    float mx[H], sum[H];
    __device__ __forceinline__ PieceFold()
    {
#pragma unroll
        for (int h = 0; h < H; h++) {
            mx[h] = -INFINITY;
            sum[h] = 0.f;
        }
    }
    __device__ __forceinline__ void fold(int h, float m2, float s2)
    {
        if (SOFT) {
            const float mm = fmaxf(mx[h], m2);
            sum[h] = (mx[h] == -INFINITY ? 0.f : sum[h] * __expf(mx[h] - mm)) + (m2 == -INFINITY ? 0.f : s2 * __expf(m2 - mm));
            mx[h] = mm;
        } else {
            sum[h] += s2;
        }
    }
    // pieces of the tiles first..last of one column (its tail piece in the tile it begins in,
    // head pieces after that).  Most crossing columns end in the next tile: a short chain is
    // folded in order by every lane alike; a long one is dealt round-robin over the wavefront's
    // lanes, each lane keeping tile order, then folded across the lanes (fold is symmetric in
    // its operands, so every lane ends with the same bits).  The same order whoever computes it.
    __device__ __forceinline__ void chain(const float *pieces, int first, int last)
    {
        const bool chain_short = last - first < 4;
        for (int j = first + (chain_short ? 0 : lane_id()); j <= last; j += chain_short ? 1 : kWave) {
            const float *p = pieces + ((int64_t)j * 2 + (j == first ? 1 : 0)) * 2 * H;
#pragma unroll
            for (int h = 0; h < H; h++) fold(h, SOFT ? p[h] : 0.f, SOFT ? p[H + h] : p[h]);
        }
        if (chain_short) return;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float m2 = SOFT ? __shfl_xor(mx[h], o, kWave) : 0.f;
                const float s2 = __shfl_xor(sum[h], o, kWave);
                fold(h, m2, s2);
            }
        }
    }
};

// One wavefront per tile in which a crossing column begins folds the column's pieces into
// stat[tile] (forward: H maxima, H reciprocals of the sums; backward: H sums), or, for column
// sums, into the column's slot of the result.
template <int H, int T, bool FWD>
__global__ __launch_bounds__(kFlatThreads) void esm_merge(const FlatMeta *__restrict__ meta,
                                                          const float *__restrict__ pieces, float *__restrict__ stat,
                                                          int ntiles, float *__restrict__ column_out = nullptr)
{
    const int tile = blockIdx.x * kFlatWaves + (threadIdx.x >> 6);
    if (tile >= ntiles) return;
    const FlatMeta m = meta[tile];
    if (!m.tail_open || m.tail_cs < tile * T) return;
    const int last_tile = min((m.tail_ce - 1) / T, ntiles - 1);   // the clamp only matters for offsets past E
    PieceFold<H, FWD> f;
    f.chain(pieces, tile, last_tile);
    if (lane_id() == 0) {
#pragma unroll
        for (int h = 0; h < H; h++) {
            if (FWD) {
                stat[(int64_t)tile * 2 * H + h] = f.mx[h];
                stat[(int64_t)tile * 2 * H + H + h] = 1.f / f.sum[h];
            } else if (column_out) {
                column_out[(int64_t)m.tail_col * H + h] = f.sum[h];     // column sums: the total is the result
            } else {
                stat[(int64_t)tile * 2 * H + h] = f.sum[h];
            }
        }
    }
}

// Entries of crossing columns.  a = x (forward) or y (backward); b = g.  Four floats per lane and
// access where the arrays are aligned; the two ends of a range float by float.
template <int H, int T, bool FWD>
__global__ __launch_bounds__(kFlatThreads) void esm_finish(const FlatMeta *__restrict__ meta,
                                                           const float *__restrict__ stat, const float *__restrict__ a,
                                                           const float *__restrict__ b, float *__restrict__ out, int E)
{
    const int tile = blockIdx.x;
    const int t0 = tile * T;
    const int n = min(T, E - t0);
    const FlatMeta m = meta[tile];
    const bool vec = both_aligned(a, out) && (FWD || ((uintptr_t)b & 15) == 0);
#pragma unroll
    for (int part = 0; part < 2; part++) {
        int src;
        int64_t lo, hi;
        if (part == 0) {
            if (!m.head_open) continue;
            src = min(max(m.head_cs, 0) / T, tile);
            lo = (int64_t)t0 * H;
            hi = (int64_t)min(m.head_ce, t0 + n) * H;
        } else {
            if (!m.tail_open || m.tail_cs < t0) continue;
            src = tile;
            lo = (int64_t)m.tail_cs * H;
            hi = (int64_t)(t0 + n) * H;
        }
        const float *st = stat + (int64_t)src * 2 * H;
        if (vec) {
            // the heads of a lane's four floats are the same at every step (the stride is a multiple of H)
            const int64_t q0 = (lo >> 2) + threadIdx.x;
            const int hb = (int)((q0 * 4) % H);
            float s0[4], s1[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                s0[i] = st[(hb + i) % H];
                s1[i] = FWD ? st[H + (hb + i) % H] : 0.f;
            }
            auto value = [&](int i, float va, float vb) { return FWD ? __expf(va - s0[i]) * s1[i] : va * vb - va * s0[i]; };
            constexpr int kBatch = 2;
            for (int64_t qb = q0; qb * 4 < hi; qb += (int64_t)kBatch * kFlatThreads) {
                float4 va[kBatch], vb[kBatch];
                bool whole[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; u++) {
                    const int64_t p = (qb + (int64_t)u * kFlatThreads) * 4;
                    whole[u] = p >= lo && p + 4 <= hi;
                    if (whole[u]) {
                        va[u] = *reinterpret_cast<const float4 *>(a + p);
                        if (!FWD) vb[u] = *reinterpret_cast<const float4 *>(b + p);
                    }
                }
#pragma unroll
                for (int u = 0; u < kBatch; u++) {
                    const int64_t p = (qb + (int64_t)u * kFlatThreads) * 4;
                    if (whole[u]) {
                        float4 r;
                        r.x = value(0, va[u].x, FWD ? 0.f : vb[u].x);
                        r.y = value(1, va[u].y, FWD ? 0.f : vb[u].y);
                        r.z = value(2, va[u].z, FWD ? 0.f : vb[u].z);
                        r.w = value(3, va[u].w, FWD ? 0.f : vb[u].w);
                        *reinterpret_cast<float4 *>(out + p) = r;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            if (p + i >= lo && p + i < hi) out[p + i] = value(i, a[p + i], FWD ? 0.f : b[p + i]);
                    }
                }
            }
        } else {
            for (int64_t p = lo + threadIdx.x; p < hi; p += kFlatThreads) {
                const int h = (int)(p % H);
                out[p] = FWD ? __expf(a[p] - st[h]) * st[H + h] : a[p] * b[p] - a[p] * st[h];
            }
        }
    }
}

// ------------------------------------------------------------------ host ---
static int flat_tiles(int64_t E, int H)
{
    const int T = H <= 2 ? FlatShape<1>::T : FlatShape<4>::T;
    return (int)ceil_div(E, T);
}

bool edge_softmax_flat_supported(int H) { return H == 1 || H == 2 || H == 4 || H == 8; }

size_t entry_tiles_ws_bytes(int64_t E)
{
    // sized for the smallest tile and the widest pieces (H = 8)
    const size_t tiles = (size_t)ceil_div(E > 0 ? E : 1, (int64_t)FlatShape<8>::T);
    return carve_bytes(tiles, sizeof(FlatMeta)) + carve_bytes(tiles * 4 * 8, 4) + carve_bytes(tiles * 2 * 8, 4) +
           2 * carve_bytes(tiles, 4);
}

// (first, last) column per tile: from the caller's tile plan, or computed into the workspace now
static TilePlan tile_columns(const void *tiles, const int32_t *off, int32_t V, int64_t E, int T, int32_t *tile_first,
                             int32_t *tile_last, hipStream_t s)
{
    if (tiles) return tile_plan_view(E, T, tiles);
    tile_columns_enqueue(off, V, E, T, tile_first, tile_last, s);
    return TilePlan{tile_first, tile_last};
}

template <int H>
static void flat_launch(bool fwd, const int32_t *off, const float *a, const float *b, float *out, int32_t V, int64_t E,
                        void *ws, hipStream_t s, const void *tiles)
{
    constexpr int T = FlatShape<H>::T;
    const int ntiles = flat_tiles(E, H);
    Carver carve(ws);
    const size_t cap = (size_t)ceil_div(E, (int64_t)FlatShape<8>::T);
    FlatMeta *meta = carve.take<FlatMeta>(cap);
    float *pieces = carve.take<float>(cap * 4 * 8);
    float *stat = carve.take<float>(cap * 2 * 8);
    const TilePlan tp = tile_columns(tiles, off, V, E, T, carve.take<int32_t>(cap), carve.take<int32_t>(cap), s);
    const int32_t *tile_first = tp.tile_first, *tile_last = tp.tile_last;
    // Through LDS pays once a lane's K*H floats span 64 bytes or more (measured:
    // 1 head 42 vs 44 us direct, 8 heads 390 vs 319 us); JGAMD_SOFTMAX_STAGE=0/1 overrides.
    const char *env = getenv("JGAMD_SOFTMAX_STAGE");
    const int staged = env ? atoi(env) : (H >= 2 ? 1 : 0);
    if (fwd) {
        hipLaunchKernelGGL(esm_fwd_tile<H>, dim3(ntiles), dim3(kFlatThreads), 0, s, off, a, out, tile_first, tile_last,
                           V, (int)E, meta, pieces, staged);
        hipLaunchKernelGGL((esm_merge<H, T, true>), dim3((unsigned)ceil_div(ntiles, kFlatWaves)), dim3(kFlatThreads), 0, s,
                           meta, pieces, stat, ntiles);
        hipLaunchKernelGGL((esm_finish<H, T, true>), dim3(ntiles), dim3(kFlatThreads), 0, s, meta, stat, a, a, out,
                           (int)E);
    } else {
        hipLaunchKernelGGL(esm_bwd_tile<H>, dim3(ntiles), dim3(kFlatThreads), 0, s, off, a, b, out, tile_first,
                           tile_last, V, (int)E, meta, pieces, staged);
        hipLaunchKernelGGL((esm_merge<H, T, false>), dim3((unsigned)ceil_div(ntiles, kFlatWaves)), dim3(kFlatThreads), 0,
                           s, meta, pieces, stat, ntiles);
        hipLaunchKernelGGL((esm_finish<H, T, false>), dim3(ntiles), dim3(kFlatThreads), 0, s, meta, stat, a, b, out,
                           (int)E);
    }
}

template <int H>
static void colsum_launch(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, int32_t R,
                          int32_t C, int64_t E, void *ws, hipStream_t s, const void *tiles)
{
    constexpr int T = FlatShape<H>::T;
    const int ntiles = flat_tiles(E, H);
    Carver carve(ws);
    const size_t cap = (size_t)ceil_div(E, (int64_t)FlatShape<8>::T);
    FlatMeta *meta = carve.take<FlatMeta>(cap);
    float *pieces = carve.take<float>(cap * 4 * 8);
    carve.take<float>(cap * 2 * 8);      // the softmax kernels' merged totals: not used here
    const TilePlan tp = tile_columns(tiles, off, R, E, T, carve.take<int32_t>(cap), carve.take<int32_t>(cap), s);
    const int32_t *tile_first = tp.tile_first, *tile_last = tp.tile_last;
    hipLaunchKernelGGL(esm_colsum_tile<H>, dim3(ntiles), dim3(kFlatThreads), 0, s, off, idx, w, x, out, tile_first,
                       tile_last, R, C, (int)E, meta, pieces);
    hipLaunchKernelGGL((esm_merge<H, T, false>), dim3((unsigned)ceil_div(ntiles, kFlatWaves)), dim3(kFlatThreads), 0, s,
                       meta, pieces, (float *)nullptr, ntiles, out);
}

// out[r,:] = sum_j w[j] * x[idx[j],:] for rows of F = 1, 2, 4 or 8 floats.  Needs R > 0,
// E > 0, off[0] == 0, off[R] == E, x rows aligned to min(16, 4F) bytes.
bool narrow_spmm_supported(int F, const void *x)
{
    if (!(F == 1 || F == 2 || F == 4 || F == 8)) return false;
    return ((uintptr_t)x & (uintptr_t)((F >= 4 ? 16 : 4 * F) - 1)) == 0;
}

void narrow_spmm_enqueue(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, int32_t R,
                         int32_t C, int64_t E, int32_t F, void *ws, hipStream_t s, const void *tiles)
{
    switch (F) {
    case 1: colsum_launch<1>(off, idx, w, x, out, R, C, E, ws, s, tiles); break;
    case 2: colsum_launch<2>(off, idx, w, x, out, R, C, E, ws, s, tiles); break;
    case 4: colsum_launch<4>(off, idx, w, x, out, R, C, E, ws, s, tiles); break;
    default: colsum_launch<8>(off, idx, w, x, out, R, C, E, ws, s, tiles); break;
    }
}

// fwd: a = x, b unused; bwd: a = y, b = g.  V > 0, E > 0, off[V] == E.
void edge_softmax_flat_enqueue(bool fwd, const int32_t *off, const float *a, const float *b, float *out, int32_t V,
                               int64_t E, int32_t H, void *ws, hipStream_t s, const void *tiles)
{
    switch (H) {
    case 1: flat_launch<1>(fwd, off, a, b, out, V, E, ws, s, tiles); break;
    case 2: flat_launch<2>(fwd, off, a, b, out, V, E, ws, s, tiles); break;
    case 4: flat_launch<4>(fwd, off, a, b, out, V, E, ws, s, tiles); break;
    default: flat_launch<8>(fwd, off, a, b, out, V, E, ws, s, tiles); break;
    }
}

}  // namespace jg
