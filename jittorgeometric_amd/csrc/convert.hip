// COO -> CSR/CSC as a stable two-level counting sort.
//
// The reference (ops/cpp/cootocsr_op.cc:35-53, cootocsc_op.cc:33-51) is a
// sequential counting sort: histogram of the key, prefix sum, then a scatter
// in input order, so edges of one row keep their input order.  Atomics on a
// GPU cannot give that order (and 10^7 global atomics write through to
// memory), so the sort is two stable partitions that rank their items with
// wave-level match + popcount and count only in LDS:
//
//   1. bucket histogram : per block of 8192 edges, LDS counts per BUCKET
//                         (bucket = key >> shift, <= 2048 buckets).
//   2. scan             : the (bucket, block) table -> each block's write
//                         cursor in each bucket (and every bucket's extent).
//   3. partition        : every block re-reads its edges, sorts its tile by
//                         bucket inside LDS and writes one record per edge,
//                         one contiguous run per (block, bucket), in input
//                         order.  A record is packed into 8 bytes (12 with the
//                         permutation) when a node id and the key bits left for
//                         the second level fit one word, else it is the plain
//                         12/16-byte (key, other, weight[, position]).
//   4. sub-block plan   : buckets are cut into sub-blocks of <= 8192 records
//                         (one tile), so a hub's bucket is many blocks' work.
//   5. sub-block count  : LDS counts per key of the bucket (<= 2048 keys).
//   6. bucket offsets   : per bucket, prefix over its sub-blocks and keys ->
//                         the final offsets array and every sub-block's
//                         first output slot per key.
//   7. sub-block scatter: the tile is sorted by key inside LDS and leaves as
//                         one contiguous run per (sub-block, key).
//
// Both scatters go through LDS because lanes that store 64 unrelated
// addresses leave partly written cache lines behind: with ~1000 bins times
// ~500 resident blocks the write frontier does not fit in L2 and every short
// store is written back on its own (2.7-3x the bytes on the counters).
//
// Two levels of at most 2048 bins each cover V <= 2^22 vertices.  Above that
// the records are sorted by plain LSD passes of the same stable partition
// (11-bit digits, least significant first), the offsets are read off the
// sorted keys, and the records are unpacked.
#include <type_traits>

#include "common.h"

namespace jg {

constexpr int kPartThreads = 512;                 // 8 waves
constexpr int kPartWaves = kPartThreads / kWave;
constexpr int kItems = 16;                        // items per thread
constexpr int kTile = kPartThreads * kItems;      // 8192 items per block tile
constexpr int kWaveSpan = kWave * kItems;         // 1024 consecutive items per wave
constexpr int kMaxBins = 2048;
constexpr int kMaxBinBits = 11;

struct Rec3 {
    int32_t key, other;
    uint32_t w;
};
struct __attribute__((aligned(16))) Rec4 {
    int32_t key, other;
    uint32_t w;
    int32_t id;
};

// Between the two levels a record is packed: inside a bucket only the low `shift` bits of the
// key matter, so a = (key low bits << obits) | other endpoint and b = the weight's bits.  An
// endpoint that does not fit the obits = 32 - shift bits left (never the case for node ids
// below V, whatever the graph) is replaced by the all-ones field and b by the edge's position
// in the input; the last step then fetches endpoint and weight from the input arrays.  With
// out_perm the record carries the edge's position as a third word.
struct __attribute__((aligned(8))) Pack2 {
    uint32_t a, b;
};
struct Pack3 {
    uint32_t a, b;
    int32_t id;
};
template <bool PERM> struct PackOf { using type = Pack2; };
template <> struct PackOf<true> { using type = Pack3; };
__device__ __forceinline__ int32_t get_id(const Pack2 &) { return 0; }
__device__ __forceinline__ int32_t get_id(const Pack3 &r) { return r.id; }
struct PackRule {
    int shift;          // low key bits kept in a record
    int obits;          // bits of the endpoint field (32 - shift)
    uint32_t omask;     // all ones in that field = "look the edge up"
};
__device__ __forceinline__ uint32_t key_low_of(uint32_t a, const PackRule &p) { return p.shift ? a >> p.obits : 0u; }
__device__ __forceinline__ Pack2 pack(const Rec3 &r, const PackRule &p)
{
    // an endpoint that does not fit was replaced by -1 when the record was loaded, with its
    // edge's position in the weight word
    Pack2 q;
    q.a = ((uint32_t)r.other >= p.omask ? p.omask : (uint32_t)r.other) | (p.shift ? ((uint32_t)r.key << p.obits) : 0u);
    q.b = r.w;
    return q;
}
__device__ __forceinline__ Pack3 pack(const Rec4 &r, const PackRule &p)
{
    Pack3 q;
    q.a = ((uint32_t)r.other >= p.omask ? p.omask : (uint32_t)r.other) | (p.shift ? ((uint32_t)r.key << p.obits) : 0u);
    q.b = r.w;
    q.id = r.id;
    return q;
}

// How the second level reads a record of either form.
struct PackedView {
    PackRule rule;
    template <typename R> __device__ __forceinline__ int key_low(const R &q) const { return (int)key_low_of(q.a, rule); }
    template <bool PERM, typename R>
    __device__ __forceinline__ void unpack(const R &q, const int32_t *others_in, const uint32_t *w_in, int32_t &other,
                                           uint32_t &wv, int32_t &id) const
    {
        uint32_t o = rule.shift ? (q.a & rule.omask) : q.a;
        wv = q.b;
        id = get_id(q);
        if (o == rule.omask) {       // endpoint kept in the input arrays
            if (!PERM) id = (int32_t)wv;
            o = (uint32_t)others_in[id];
            wv = w_in ? w_in[id] : 0u;
        }
        other = (int32_t)o;
    }
};
struct PlainView {
    int mask;
    template <typename R> __device__ __forceinline__ int key_low(const R &q) const { return q.key & mask; }
    template <bool PERM, typename R>
    __device__ __forceinline__ void unpack(const R &q, const int32_t *, const uint32_t *, int32_t &other, uint32_t &wv,
                                           int32_t &id) const
    {
        other = q.other;
        wv = q.w;
        id = get_id(q);
    }
};

// A record out of an array, field by field for the 16-byte kind: copied as one aligned block, a
// lane's sixteen of them stayed in scratch memory (272 bytes per lane) instead of registers.  The
// kernels take the same time either way (more registers, fewer wavefronts); without scratch
// memory no launch of this library makes the runtime set any aside.
template <typename Rec> __device__ __forceinline__ Rec read_rec(const Rec *p) { return *p; }
template <> __device__ __forceinline__ Rec4 read_rec<Rec4>(const Rec4 *p)
{
    const uint4 q = *reinterpret_cast<const uint4 *>(p);
    Rec4 r;
    r.key = (int32_t)q.x;
    r.other = (int32_t)q.y;
    r.w = q.z;
    r.id = (int32_t)q.w;
    return r;
}

template <typename Rec> __device__ __forceinline__ void write_rec(Rec *p, const Rec &r) { *p = r; }
template <> __device__ __forceinline__ void write_rec<Rec4>(Rec4 *p, const Rec4 &r)
{
    *reinterpret_cast<uint4 *>(p) = make_uint4((uint32_t)r.key, (uint32_t)r.other, r.w, (uint32_t)r.id);
}

template <bool PERM> struct RecOf { using type = Rec3; };
template <> struct RecOf<true> { using type = Rec4; };

__device__ __forceinline__ void set_id(Rec3 &, int32_t) {}
__device__ __forceinline__ void set_id(Rec4 &r, int32_t id) { r.id = id; }
__device__ __forceinline__ int32_t get_id(const Rec3 &) { return 0; }
__device__ __forceinline__ int32_t get_id(const Rec4 &r) { return r.id; }

// Tile a workgroup of the histogram and of the partition takes.  Workgroup b runs on XCD b % 8;
// every XCD gets a contiguous range of tiles, so that what neighbouring tiles write side by side
// (their counts in the table, the runs they append to a bucket) meets in one L2 before it is
// written back (V = 2.45M, E = 126M: 3.54 -> 2.73 ms).  The grid is rounded up to a
// multiple of 8; workgroups past the last tile return.
__device__ __forceinline__ int tile_of_workgroup(int nblocks)
{
    const int per = (nblocks + 7) / 8;
    const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    return ((int)(blockIdx.x >> 3) < per && t < nblocks) ? t : -1;
}

// bins[b] += unit for every lane with b >= 0, one LDS atomic per run of equal b over consecutive
// lanes of a row of 16.  Keys that arrive sorted (an edge list ordered by source) put whole
// wavefronts on one counter, and 64 atomics on one LDS address take 64 turns; a run costs one.
// The neighbour's value comes from a row shift on the vector ALU (runs are cut at rows of 16
// lanes, which the shift does not cross), so unsorted keys pay a few ALU instructions, no LDS trip.
__device__ __forceinline__ void count_runs(uint32_t *bins, int b, uint32_t unit)
{
    const int l15 = lane_id() & 15;
    const int prev = __builtin_amdgcn_update_dpp(b, b, 0x111 /* row_shr:1 */, 0xf, 0xf, false);
    const bool start = l15 == 0 || b != prev;
    const uint64_t starts = __ballot(start);
    if (start && b >= 0) {
        // the starts of this row of 16 lanes after this lane; none: the run goes to the row's end
        const uint32_t row = (uint32_t)(starts >> (lane_id() & 48)) & 0xffffu;
        const uint32_t later = row >> (l15 + 1);
        const uint32_t len = min(later ? (uint32_t)__builtin_ctz(later) : 31u, (uint32_t)(15 - l15)) + 1u;
        atomicAdd(&bins[b], len * unit);
    }
}

// ---------------------------------------------------------------- step 1 ---
// keys: the key row of edge_index.  Items with key outside [0,V) are ignored
// here and in every later step.  table is [nbins][nblocks] (+1 trailing zero).
__global__ __launch_bounds__(kPartThreads) void csx_bucket_histogram(const int32_t *__restrict__ keys, int64_t E,
                                                                     int32_t V, int shift, int nbins,
                                                                     int32_t *__restrict__ table, int nblocks)
{
    __shared__ uint32_t bins[kMaxBins];
    const int blk = tile_of_workgroup(nblocks);
    if (blk < 0) return;
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) bins[b] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blk * kTile;
    // all loads first (index clamped instead of predicated), then the counting
    int32_t k[kItems];
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int64_t e = base + (int64_t)i * kPartThreads + threadIdx.x;
        k[i] = keys[e < E ? e : E - 1];
    }
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int64_t e = base + (int64_t)i * kPartThreads + threadIdx.x;
        count_runs(bins, (e < E && (uint32_t)k[i] < (uint32_t)V) ? (k[i] >> shift) : -1, 1u);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) table[(int64_t)b * nblocks + blk] = (int32_t)bins[b];
    if (blk == 0 && threadIdx.x == 0) table[(int64_t)nbins * nblocks] = 0;
}

// ------------------------------------------------------- stable tile sort ---
// The block's tile is kTile consecutive items; wave w owns the kWaveSpan
// consecutive items starting at w*kWaveSpan and visits them in rounds of 64
// (lane l = item r*64 + l), so (wave, round, lane) is the input order.
//
// tile_sort gives every item its position in the tile sorted stably by bin:
//   start[bin] + (items of that bin in earlier waves)
//              + (same wave, earlier rounds) + (same round, lower lanes).
// Per-wave counters are 16 bits wide (a wave holds 1024 items, a tile 8192
// positions), two waves to a word.  tile_emit then moves the records through
// an LDS window of kStage records so that consecutive lanes hold consecutive
// sorted records, and hands each one to `emit` with its global position
// gbase(bin) + (position - start[bin]).  The window takes what is left of
// kTileLdsBytes after the per-bin arrays, so two blocks fit a CU's 160 KB.
constexpr size_t kTileLdsBytes = 78 * 1024;

struct TileLds {
    uint32_t *cnt;    // [kPartWaves / 2][nbins]
    int *start;       // [nbins] tile-local first position of the bin
    int *delta;       // [nbins] global minus tile-local position
    int *misc;        // [kPartWaves] wave totals, [kPartWaves] tile total
    uint32_t *stage;  // stage_n records
    int stage_n;
};
constexpr int kTileMisc = 16;
inline size_t tile_bins_bytes(int nbins) { return ((size_t)(kPartWaves / 2 + 2) * nbins + kTileMisc) * 4; }
// records per trip through LDS: a multiple of the block size, at most a tile
inline int tile_stage_records(int nbins, size_t rec_bytes)
{
    size_t n = (kTileLdsBytes - tile_bins_bytes(nbins)) / rec_bytes;
    n = n / kPartThreads * kPartThreads;
    return (int)(n > (size_t)kTile ? (size_t)kTile : n);
}
inline size_t tile_lds_bytes(int nbins, size_t rec_bytes)
{
    return tile_bins_bytes(nbins) + (size_t)tile_stage_records(nbins, rec_bytes) * rec_bytes;
}
// the stage area also holds a byte per (wavefront, bin) while the items are ranked
constexpr bool tile_stage_holds_tags(size_t rec_bytes)
{
    return ((kTileLdsBytes - ((size_t)(kPartWaves / 2 + 2) * kMaxBins + kTileMisc) * 4) / rec_bytes / kPartThreads *
            kPartThreads) * rec_bytes >= (size_t)kPartWaves * kMaxBins;
}
static_assert(tile_stage_holds_tags(8) && tile_stage_holds_tags(12) && tile_stage_holds_tags(16),
              "stage area too small for the tag table at the largest number of bins");
template <typename Rec, typename Base>
__device__ __forceinline__ int tile_sort(uint32_t *raw, int stage_n, TileLds &L, int nbins,
                                         const int (&bin)[kItems], int (&lp)[kItems], Base gbase)
{
    L.stage = raw;
    L.stage_n = stage_n;
    L.cnt = raw + stage_n * (sizeof(Rec) / 4);
    L.start = reinterpret_cast<int *>(L.cnt + (kPartWaves / 2) * nbins);
    L.delta = L.start + nbins;
    L.misc = L.delta + nbins;

    const int w = threadIdx.x >> 6;
    const int lane = lane_id();
    const int half = (w & 1) * 16;
    uint32_t *mine = L.cnt + (w >> 1) * nbins;
    for (int i = threadIdx.x; i < (kPartWaves / 2) * nbins; i += kPartThreads) L.cnt[i] = 0;
    // bins b0 .. b0+K-1 belong to this thread in the per-bin phase; their
    // global bases are fetched now so the latency hides behind the counting
    constexpr int kMaxK = kMaxBins / kPartThreads;
    const int K = (nbins + kPartThreads - 1) / kPartThreads;
    const int b0 = threadIdx.x * K;
    int gb[kMaxK];
#pragma unroll
    for (int i = 0; i < kMaxK; i++) gb[i] = (i < K && b0 + i < nbins) ? gbase(b0 + i) : 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kItems; r++) count_runs(mine, bin[r], 1u << half);
    __syncthreads();
    uint32_t pk[kMaxK][kPartWaves / 2];
    int tot[kMaxK];
    int mysum = 0;
#pragma unroll
    for (int i = 0; i < kMaxK; i++) {
        tot[i] = 0;
        if (i < K && b0 + i < nbins) {
            int run = 0;
#pragma unroll
            for (int v = 0; v < kPartWaves / 2; v++) {
                const uint32_t c = L.cnt[v * nbins + b0 + i];
                const int lo = c & 0xffff, hi = c >> 16;
                pk[i][v] = (uint32_t)run | ((uint32_t)(run + lo) << 16);
                run += lo + hi;
            }
            tot[i] = run;
            mysum += run;
        }
    }
    int inc = mysum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int t = __shfl_up(inc, d, kWave);
        if (lane >= d) inc += t;
    }
    if (lane == kWave - 1) L.misc[w] = inc;
    __syncthreads();
    int base = inc - mysum;
    for (int v = 0; v < w; v++) base += L.misc[v];
#pragma unroll
    for (int i = 0; i < kMaxK; i++)
        if (i < K && b0 + i < nbins) {
            L.start[b0 + i] = base;
            L.delta[b0 + i] = gb[i] - base;
            const uint32_t both = (uint32_t)base | ((uint32_t)base << 16);
#pragma unroll
            for (int v = 0; v < kPartWaves / 2; v++) L.cnt[v * nbins + b0 + i] = pk[i][v] + both;
            base += tot[i];
        }
    if (threadIdx.x == kPartThreads - 1) L.misc[kPartWaves] = base;
    __syncthreads();
    // Lanes of one round with the same bin.  Comparing the bins themselves takes one vote per bit
    // of the bin (9 to 11); instead every lane leaves its number in a table indexed by bin (the
    // stage area is idle until the records move) and reads the slot back: lanes of one bin read the
    // same number, whichever of them wrote last, and telling those numbers apart takes 6 votes.
    // The LDS executes a wavefront's accesses in order, so the read sees every lane's write.
    uint8_t *tags = reinterpret_cast<uint8_t *>(L.stage) + w * nbins;
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        const int b = bin[r];
        const bool valid = b >= 0;
        if (valid) tags[b] = (uint8_t)lane;
        asm volatile("" ::: "memory");      // the slot is read back from LDS, not from the value just stored
        const int tag = valid ? tags[b] : 0;
        // peers: valid lanes of this round with the same bin as this lane, kept as two halves;
        // m is all ones where the tag's bit is set, so ~(vote ^ m) keeps the lanes that voted alike
        const uint64_t voters = __ballot(valid);
        uint32_t plo = (uint32_t)voters, phi = (uint32_t)(voters >> 32);
#pragma unroll
        for (int t = 0; t < 6; t++) {
            const int m = (tag << (31 - t)) >> 31;
            const uint64_t vote = __ballot(m != 0);
            plo &= ~((uint32_t)vote ^ (uint32_t)m);
            phi &= ~((uint32_t)(vote >> 32) ^ (uint32_t)m);
        }
        const int rank = (int)__builtin_amdgcn_mbcnt_hi(phi, __builtin_amdgcn_mbcnt_lo(plo, 0u));    // peers in lower lanes
        // the lane whose number the group read adds the group's size to the bin's counter
        uint32_t old = 0;
        if (valid && lane == tag) old = atomicAdd(&mine[b], (uint32_t)(__popc(plo) + __popc(phi)) << half);
        old = __shfl(old, tag, kWave);
        lp[r] = (int)((old >> half) & 0xffff) + rank;
    }
    __syncthreads();      // the stage area is the records' from here on
    return L.misc[kPartWaves];
}

template <typename Rec, typename BinOfRec, typename Emit>
__device__ __forceinline__ void tile_emit(const TileLds &L, int total, BinOfRec bin_of_rec, const Rec (&rec)[kItems],
                                          const int (&bin)[kItems], const int (&lp)[kItems], Emit emit)
{
    Rec *stage = reinterpret_cast<Rec *>(L.stage);
    for (int h0 = 0; h0 < total; h0 += L.stage_n) {
#pragma unroll
        for (int r = 0; r < kItems; r++)
            if (bin[r] >= 0 && (unsigned)(lp[r] - h0) < (unsigned)L.stage_n) write_rec(stage + (lp[r] - h0), rec[r]);
        __syncthreads();
        const int n = min(total - h0, L.stage_n);
#pragma unroll 4
        for (int j = threadIdx.x; j < n; j += kPartThreads) {
            const Rec q = read_rec(stage + j);
            emit(L.delta[bin_of_rec(q)] + h0 + j, q);
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- step 3 ---
// Loader for the first partition: items come from the COO arrays.
__device__ __forceinline__ void keep_position(Rec3 &r, int32_t c) { r.w = (uint32_t)c; }
__device__ __forceinline__ void keep_position(Rec4 &, int32_t) {}      // has it already (id)
template <typename Rec> struct CooLoader {
    const int32_t *keys;
    const int32_t *others;
    const uint32_t *w;
    int64_t n;
    int32_t V;
    uint32_t omask;     // endpoints from this value up do not pack (0: nothing is packed, LSD passes)
    // Branch-free: the index is clamped, validity is judged afterwards.  INSIDE: the caller knows
    // e < n (a tile that ends before the list does), so the addresses are the lane's base plus a constant.
    template <bool INSIDE = false> __device__ __forceinline__ void load(int64_t e, Rec &r) const
    {
        const int64_t c = (INSIDE || e < n) ? e : n - 1;
        r.key = keys[c];
        r.other = others[c];
        r.w = w ? w[c] : 0u;
        set_id(r, (int32_t)c);
        // an endpoint that does not pack is looked up again from its position at the end; no
        // lane of a wavefront has one in any graph whose node ids are below V
        if (omask && __ballot((uint32_t)r.other >= omask) != 0ull) {
            if ((uint32_t)r.other >= omask) {
                r.other = -1;
                keep_position(r, (int32_t)c);
            }
        }
    }
    template <bool INSIDE = false> __device__ __forceinline__ bool valid(int64_t e, const Rec &r) const
    {
        return (INSIDE || e < n) && (uint32_t)r.key < (uint32_t)V;
    }
};
// Loader for the later LSD passes: items are records; only the first *count
// slots hold records (edges with out-of-range keys were dropped by pass 0).
template <typename Rec> struct RecLoader {
    const Rec *recs;
    const int32_t *count;
    int64_t cap;      // upper bound of *count (> 0)
    __device__ __forceinline__ void load(int64_t e, Rec &r) const { r = read_rec(recs + (e < cap ? e : cap - 1)); }
    __device__ __forceinline__ bool valid(int64_t e, const Rec &) const { return e < (int64_t)*count; }
};

// Per-block counts of one digit ((key >> shift) & mask) for any loader.
template <typename Rec, typename Loader>
__global__ __launch_bounds__(kPartThreads) void csx_digit_histogram(Loader in, int shift, int mask, int nbins,
                                                                    int32_t *__restrict__ table, int nblocks)
{
    __shared__ uint32_t bins[kMaxBins];
    const int blk = tile_of_workgroup(nblocks);
    if (blk < 0) return;
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) bins[b] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blk * kTile;
    Rec rec[kItems];
#pragma unroll
    for (int i = 0; i < kItems; i++) in.load(base + (int64_t)i * kPartThreads + threadIdx.x, rec[i]);
#pragma unroll
    for (int i = 0; i < kItems; i++)
        count_runs(bins, in.valid(base + (int64_t)i * kPartThreads + threadIdx.x, rec[i]) ? ((rec[i].key >> shift) & mask) : -1,
                   1u);
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) table[(int64_t)b * nblocks + blk] = (int32_t)bins[b];
    if (blk == 0 && threadIdx.x == 0) table[(int64_t)nbins * nblocks] = 0;
}

__global__ void csx_save_count(const int32_t *__restrict__ table_end, int32_t *__restrict__ count)
{
    *count = *table_end;
}

// Records sorted by key -> offsets (off[k] = first position whose key is >= k)
// and the unpacked output arrays.  One thread per position 0..cap (inclusive).
template <typename Rec, bool PERM>
__global__ void csx_unpack_sorted(const Rec *__restrict__ recs, const int32_t *__restrict__ count, int64_t cap,
                                  int32_t V, int32_t *__restrict__ off, int32_t *__restrict__ out_idx,
                                  uint32_t *__restrict__ out_w, int32_t *__restrict__ out_perm)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t n = *count;
    if (p > n || p > cap) return;
    const int64_t prev = p > 0 ? recs[p - 1].key : -1;
    const int64_t cur = p < n ? recs[p].key : (int64_t)V;
    for (int64_t k = prev + 1; k <= cur; k++) off[k] = (int32_t)p;
    if (p < n) {
        const Rec r = recs[p];
        out_idx[p] = r.other;
        if (out_w) out_w[p] = r.w;
        if (PERM) out_perm[p] = get_id(r);
    }
}

template <typename Rec, typename Loader>
__global__ __launch_bounds__(kPartThreads) void csx_partition(Loader in, int shift, int mask, int nbins,
                                                              const int32_t *__restrict__ table,
                                                              int nblocks, Rec *__restrict__ out, int stage_n)
{
    extern __shared__ uint32_t lds_raw[];
    const int w = threadIdx.x >> 6;
    const int blk = tile_of_workgroup(nblocks);
    if (blk < 0) return;
    const int64_t base = (int64_t)blk * kTile + (int64_t)w * kWaveSpan + lane_id();
    Rec rec[kItems];
    int bin[kItems], lp[kItems];
#pragma unroll
    for (int r = 0; r < kItems; r++) in.load(base + (int64_t)r * kWave, rec[r]);
#pragma unroll
    for (int r = 0; r < kItems; r++)
        bin[r] = in.valid(base + (int64_t)r * kWave, rec[r]) ? ((rec[r].key >> shift) & mask) : -1;

    TileLds L;
    const int total = tile_sort<Rec>(lds_raw, stage_n, L, nbins, bin, lp,
                                     [&](int b) { return table[(int64_t)b * nblocks + blk]; });
    tile_emit(L, total, [&](const Rec &q) { return (q.key >> shift) & mask; }, rec, bin, lp,
              [&](int pos, const Rec &q) { write_rec(out + pos, q); });
}

// The first partition of the two-level path: same tile sort, the records leave packed.
template <typename Rec, typename Out>
__global__ __launch_bounds__(kPartThreads) void csx_partition_pack(CooLoader<Rec> in, PackRule rule, int nbins,
                                                                   const int32_t *__restrict__ table, int nblocks,
                                                                   Out *__restrict__ out, int stage_n)
{
    extern __shared__ uint32_t lds_raw[];
    const int w = threadIdx.x >> 6;
    const int blk = tile_of_workgroup(nblocks);
    if (blk < 0) return;
    const int64_t base = (int64_t)blk * kTile + (int64_t)w * kWaveSpan + lane_id();
    Rec rec[kItems];
    int bin[kItems], lp[kItems];
    if ((int64_t)(blk + 1) * kTile <= in.n) {
#pragma unroll
        for (int r = 0; r < kItems; r++) in.template load<true>(base + r * kWave, rec[r]);
#pragma unroll
        for (int r = 0; r < kItems; r++)
            bin[r] = in.template valid<true>(base + r * kWave, rec[r]) ? (rec[r].key >> rule.shift) : -1;
    } else {
#pragma unroll
        for (int r = 0; r < kItems; r++) in.load(base + (int64_t)r * kWave, rec[r]);
#pragma unroll
        for (int r = 0; r < kItems; r++)
            bin[r] = in.valid(base + (int64_t)r * kWave, rec[r]) ? (rec[r].key >> rule.shift) : -1;
    }

    TileLds L;
    const int total = tile_sort<Rec>(lds_raw, stage_n, L, nbins, bin, lp,
                                     [&](int b) { return table[(int64_t)b * nblocks + blk]; });
    tile_emit(L, total, [&](const Rec &q) { return q.key >> rule.shift; }, rec, bin, lp,
              [&](int pos, const Rec &q) { out[pos] = pack(q, rule); });
}

// ---------------------------------------------------------------- step 4 ---
// After the scan, bucket b holds records [table[b*nblocks], table[(b+1)*nblocks]).
// Cuts every bucket into sub-blocks of at most kSubRecords records (at least
// one per bucket): sub_first[b] = first sub-block of b, sub_bucket[s] = bucket
// of sub-block s (-1 for the unused tail of the max_sub launch slots).
constexpr int kSubRecords = kTile;

__global__ __launch_bounds__(1024) void csx_plan_subblocks(const int32_t *__restrict__ table, int nblocks,
                                                           int nbuckets, int max_sub,
                                                           int32_t *__restrict__ sub_bucket,
                                                           int32_t *__restrict__ sub_first)
{
    __shared__ int first[kMaxBins + 1];
    __shared__ int wave_tot[16];
    // thread t owns buckets 2t and 2t+1
    int n[2], mysum = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int b = 2 * threadIdx.x + i;
        n[i] = 0;
        if (b < nbuckets) {
            const int size = table[(int64_t)(b + 1) * nblocks] - table[(int64_t)b * nblocks];
            n[i] = size <= kSubRecords ? 1 : (size + kSubRecords - 1) / kSubRecords;
        }
        mysum += n[i];
    }
    int inc = mysum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int t = __shfl_up(inc, d, kWave);
        if (lane_id() >= d) inc += t;
    }
    const int w = threadIdx.x >> 6;
    if (lane_id() == kWave - 1) wave_tot[w] = inc;
    __syncthreads();
    int run = inc - mysum;
    for (int v = 0; v < w; v++) run += wave_tot[v];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int b = 2 * threadIdx.x + i;
        if (b < nbuckets) first[b] = run;
        run += n[i];
    }
    if (threadIdx.x == 1023) first[nbuckets] = run;   // buckets past the last count 0: the total
    __syncthreads();
    for (int b = threadIdx.x; b <= nbuckets; b += 1024) sub_first[b] = first[b];
    for (int b = threadIdx.x; b < nbuckets; b += 1024)
        for (int s = first[b]; s < first[b + 1] && s < max_sub; s++) sub_bucket[s] = b;
    for (int s = first[nbuckets] + threadIdx.x; s < max_sub; s += 1024) sub_bucket[s] = -1;
}

struct SubRange {
    int bucket, begin, end;
};
__device__ __forceinline__ SubRange sub_range(const int32_t *table, int nblocks, const int32_t *sub_bucket,
                                              const int32_t *sub_first, int s)
{
    SubRange r;
    r.bucket = sub_bucket[s];
    if (r.bucket < 0) {
        r.begin = r.end = 0;
        return r;
    }
    const int b0 = table[(int64_t)r.bucket * nblocks], b1 = table[(int64_t)(r.bucket + 1) * nblocks];
    r.begin = b0 + (s - sub_first[r.bucket]) * kSubRecords;
    r.end = min(b1, r.begin + kSubRecords);
    return r;
}

// ---------------------------------------------------------------- step 5 ---
// cnt2[s][key] = records of sub-block s whose low key bits are `key`.
template <typename Rec, typename View>
__global__ __launch_bounds__(kPartThreads) void csx_sub_count(const Rec *__restrict__ recs,
                                                              const int32_t *__restrict__ table, int nblocks,
                                                              const int32_t *__restrict__ sub_bucket,
                                                              const int32_t *__restrict__ sub_first, View view, int shift,
                                                              int32_t *__restrict__ cnt2)
{
    __shared__ uint32_t bins[kMaxBins];
    const SubRange r = sub_range(table, nblocks, sub_bucket, sub_first, blockIdx.x);
    if (r.bucket < 0) return;
    const int nkeys = 1 << shift;
    for (int k = threadIdx.x; k < nkeys; k += kPartThreads) bins[k] = 0;
    __syncthreads();
    constexpr int kBatch = 8;
    // every wavefront makes the same number of trips, so that count_runs sees whole wavefronts
    for (int e0 = r.begin + threadIdx.x; e0 - (int)threadIdx.x < r.end; e0 += kBatch * kPartThreads) {
        int k[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; i++) k[i] = view.key_low(recs[max(min(e0 + i * kPartThreads, r.end - 1), r.begin)]);
#pragma unroll
        for (int i = 0; i < kBatch; i++) count_runs(bins, e0 + i * kPartThreads < r.end ? k[i] : -1, 1u);
    }
    __syncthreads();
    for (int k = threadIdx.x; k < nkeys; k += kPartThreads) cnt2[(int64_t)blockIdx.x * nkeys + k] = (int32_t)bins[k];
}

// ---------------------------------------------------------------- step 6 ---
// One block per bucket.  For every key of the bucket: exclusive prefix of its
// counts over the bucket's sub-blocks, then an exclusive prefix over the keys
// (+ the bucket's first slot) = off[key]; cnt2[s][key] becomes the first
// output slot of sub-block s for that key.
__global__ __launch_bounds__(kPartThreads) void csx_bucket_offsets(const int32_t *__restrict__ table, int nblocks,
                                                                   int nbuckets,
                                                                   const int32_t *__restrict__ sub_first, int shift,
                                                                   int32_t V, int32_t *__restrict__ cnt2,
                                                                   int32_t *__restrict__ off, int64_t E,
                                                                   int32_t *__restrict__ out_idx,
                                                                   uint32_t *__restrict__ out_w,
                                                                   int32_t *__restrict__ out_perm)
{
    __shared__ int wave_tot[kPartWaves];
    __shared__ int carry;
    const int b = blockIdx.x;
    const int nkeys = 1 << shift;
    const int s0 = sub_first[b], s1 = sub_first[b + 1];
    const int64_t k0 = (int64_t)b << shift;
    if (threadIdx.x == 0) carry = table[(int64_t)b * nblocks];
    __syncthreads();
    // a bucket of up to kKeep sub-blocks keeps a key's counts in registers between the two loops
    // (all loads in flight together, the table read once)
    constexpr int kKeep = 16;
    const int ns = s1 - s0;
    for (int kb = 0; kb < nkeys; kb += kPartThreads) {
        const int k = kb + threadIdx.x;
        int total = 0;
        int kept[kKeep];
        if (k < nkeys) {
            if (ns <= kKeep) {
#pragma unroll
                for (int i = 0; i < kKeep; i++) kept[i] = cnt2[(int64_t)(s0 + min(i, ns - 1)) * nkeys + k];
#pragma unroll
                for (int i = 0; i < kKeep; i++)
                    if (i < ns) total += kept[i];
            } else {
#pragma unroll 8
                for (int s = s0; s < s1; s++) total += cnt2[(int64_t)s * nkeys + k];
            }
        }
        // block-exclusive scan of `total` in key order
        int inc = total;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const int t = __shfl_up(inc, d, kWave);
            if (lane_id() >= d) inc += t;
        }
        const int w = threadIdx.x >> 6;
        if (lane_id() == kWave - 1) wave_tot[w] = inc;
        __syncthreads();
        int before = carry;
        for (int v = 0; v < w; v++) before += wave_tot[v];
        const int key_base = before + inc - total;
        if (k < nkeys) {
            if (k0 + k < V) off[k0 + k] = key_base;
            int run = key_base;
            if (ns <= kKeep) {
#pragma unroll
                for (int i = 0; i < kKeep; i++)
                    if (i < ns) {
                        cnt2[(int64_t)(s0 + i) * nkeys + k] = run;
                        run += kept[i];
                    }
            } else {
#pragma unroll 8
                for (int s = s0; s < s1; s++) {
                    const int c = cnt2[(int64_t)s * nkeys + k];
                    cnt2[(int64_t)s * nkeys + k] = run;
                    run += c;
                }
            }
        }
        __syncthreads();
        if (threadIdx.x == kPartThreads - 1) carry = key_base + total;
        __syncthreads();
    }
    const int64_t covered = table[(int64_t)nbuckets * nblocks];
    if (b == nbuckets - 1 && threadIdx.x == 0) off[V] = (int32_t)covered;
    // Edges with a key outside [0,V) were dropped, so off[V] may be below E: the slots past off[V]
    // are zeroed (the reference hands zero-filled arrays to the op, ops/cootocsr.py:30-32).
    // Nothing to do in the usual case.
    for (int64_t i = covered + (int64_t)b * kPartThreads + threadIdx.x; i < E; i += (int64_t)gridDim.x * kPartThreads) {
        out_idx[i] = 0;
        if (out_w) out_w[i] = 0u;
        if (out_perm) out_perm[i] = 0;
    }
}

// ---------------------------------------------------------------- step 7 ---
// One block per sub-block (one tile of records): sorted by key inside LDS,
// then every key's run goes to cnt2[sub][key] onwards, unpacked.
template <typename Rec, bool PERM, typename View>
__global__ __launch_bounds__(kPartThreads) void csx_sub_scatter(const Rec *__restrict__ recs,
                                                                const int32_t *__restrict__ table, int nblocks,
                                                                const int32_t *__restrict__ sub_bucket,
                                                                const int32_t *__restrict__ sub_first,
                                                                const int32_t *__restrict__ cnt2, View view, int shift,
                                                                const int32_t *__restrict__ others_in,
                                                                const uint32_t *__restrict__ w_in,
                                                                int32_t *__restrict__ out_idx,
                                                                uint32_t *__restrict__ out_w,
                                                                int32_t *__restrict__ out_perm, int stage_n,
                                                                int nbuckets, int max_sub)
{
    extern __shared__ uint32_t lds_raw[];
    // Workgroup b runs on XCD b % 8.  The sub-blocks of one bucket write interleaved runs into the
    // bucket's output region (a few hundred KB): handing every XCD a contiguous range of
    // sub-blocks lets those runs meet in one L2 before they are written back.
    const int nsub = min(sub_first[nbuckets], max_sub);      // the grid holds 8 * ceil(max_sub / 8) workgroups
    const int per = (nsub + 7) / 8;
    const int sub = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per || sub >= nsub) return;
    const SubRange sr = sub_range(table, nblocks, sub_bucket, sub_first, sub);
    if (sr.bucket < 0) return;
    const int nkeys = 1 << shift;
    const int base = sr.begin + (threadIdx.x >> 6) * kWaveSpan + lane_id();
    Rec rec[kItems];
    int bin[kItems], lp[kItems];
#pragma unroll
    for (int r = 0; r < kItems; r++) rec[r] = read_rec(recs + min(base + r * kWave, sr.end - 1));
#pragma unroll
    for (int r = 0; r < kItems; r++) bin[r] = base + r * kWave < sr.end ? view.key_low(rec[r]) : -1;
    TileLds L;
    const int total = tile_sort<Rec>(lds_raw, stage_n, L, nkeys, bin, lp,
                                     [&](int k) { return cnt2[(int64_t)sub * nkeys + k]; });
    tile_emit(L, total, [&](const Rec &q) { return view.key_low(q); }, rec, bin, lp, [&](int pos, const Rec &q) {
        int32_t other, id;
        uint32_t wv;
        view.template unpack<PERM>(q, others_in, w_in, other, wv, id);
        out_idx[pos] = other;
        if (out_w) out_w[pos] = wv;
        if (PERM) out_perm[pos] = id;
    });
}

// Expands compressed offsets into one row id per entry (for the transpose).  A block takes a tile
// of kTileEntriesNarrow entries; the rows of its first and last entry come from the tile -> row
// map (plan.hip), their offsets are staged in LDS, a thread finds the row of its first entry by
// bisection there and walks on from it, and stores its four row ids as 16 bytes.  (One wavefront
// per row, the first form of this kernel, wrote 0.3 TB/s on rows of a few dozen entries.)
// Entries past off[R] belong to no row and get row 0.
constexpr int kExpandSlots = 4;
__global__ __launch_bounds__(256) void csx_expand_rows(const int32_t *__restrict__ off,
                                                       const int32_t *__restrict__ tile_first,
                                                       const int32_t *__restrict__ tile_last, int32_t R, int64_t E,
                                                       int32_t *__restrict__ rows)
{
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    constexpr int T = kTileEntriesNarrow;
    static_assert(T == 256 * kExpandSlots, "one tile per block");
    __shared__ int s_off[T + 2];
    const int tile = blockIdx.x;
    const int64_t t0 = (int64_t)tile * T;
    const int covered = min(max(off[R], 0), (int)E);
    const int64_t j0 = t0 + (int64_t)threadIdx.x * kExpandSlots;
    if (t0 >= covered) {
        for (int k = 0; k < kExpandSlots; k++)
            if (j0 + k < E) rows[j0 + k] = 0;
        return;
    }
    const int c_lo = min(max(tile_first[tile], 0), R - 1);
    const int c_hi = min(max(tile_last[tile], c_lo), R - 1);
    const int ncol = c_hi - c_lo + 1;
    const bool staged = ncol + 1 <= T + 2;
    if (staged)
        for (int i = threadIdx.x; i <= ncol; i += 256) s_off[i] = off[c_lo + i];
    __syncthreads();
    auto offv = [&](int c) { return staged ? s_off[c - c_lo] : off[c]; };
    const int last = covered - 1;
    const int jc = (int)min(j0, (int64_t)last);
    int lo = c_lo, hi = c_hi;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (offv(mid) <= jc) lo = mid;
        else hi = mid - 1;
    }
    int c = lo, ce = offv(c + 1);
    i32x4 r;
#pragma unroll
    for (int k = 0; k < kExpandSlots; k++) {
        const int64_t j = j0 + k;
        while (ce <= j && c < c_hi) {
            c++;
            ce = offv(c + 1);
        }
        r[k] = j > last ? 0 : c;
    }
    if (j0 + kExpandSlots <= E) {
        *reinterpret_cast<i32x4 *>(rows + j0) = r;      // rows is carved 256-byte aligned, j0 a multiple of 4
    } else {
#pragma unroll
        for (int k = 0; k < kExpandSlots; k++)
            if (j0 + k < E) rows[j0 + k] = r[k];
    }
}

// inv[perm[i]] = i; entries of perm outside [0,n) are skipped.
__global__ void csx_invert_permutation(const int32_t *__restrict__ perm, int64_t n, int32_t *__restrict__ inv)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int32_t p = perm[i];
    if ((uint64_t)p < (uint64_t)n) inv[p] = (int32_t)i;
}

__global__ void fill_i32(int32_t *p, int64_t n, int32_t v)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Edges with a key outside [0,V) were dropped, so off[V] may be below E: the slots past
// off[V] are zeroed (the reference hands zero-filled arrays to the op, ops/cootocsr.py:30-32).
// Nothing to do in the usual case, which costs one read of off[V] per thread.
__global__ void csx_zero_tail(const int32_t *__restrict__ off_end, int64_t E, int32_t *__restrict__ out_idx,
                              uint32_t *__restrict__ out_w, int32_t *__restrict__ out_perm)
{
    const int64_t first = *off_end;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < E; i += step) {
        out_idx[i] = 0;
        if (out_w) out_w[i] = 0u;
        if (out_perm) out_perm[i] = 0;
    }
}

static void zero_tail(const int32_t *out_off, int32_t V, int64_t E, int32_t *out_idx, float *out_w,
                      int32_t *out_perm, hipStream_t s)
{
    const unsigned blocks = (unsigned)(ceil_div(E, 256) < 1024 ? ceil_div(E, 256) : 1024);
    hipLaunchKernelGGL(csx_zero_tail, dim3(blocks), dim3(256), 0, s, out_off + V, E, out_idx,
                       reinterpret_cast<uint32_t *>(out_w), out_perm);
}

// ------------------------------------------------------------------ host ---
struct ConvPlan {
    int shift;        // low key bits handled inside a bucket
    int nbuckets;     // bins of the partition
    int64_t nblocks;  // tiles of kTile edges
    int max_sub;      // upper bound on the number of sub-blocks
    int digits;       // > 0: V above 2^22, plain LSD passes of 11 bits each
};

static ConvPlan make_plan(int64_t E, int32_t V)
{
    ConvPlan p{};
    int bits = 0;
    while (bits < 31 && ((int64_t)1 << bits) < (int64_t)V) bits++;   // keys < 2^bits
    p.nblocks = ceil_div(E > 0 ? E : 1, kTile);
    if (bits > 2 * kMaxBinBits) {
        p.digits = (bits + kMaxBinBits - 1) / kMaxBinBits;
        p.shift = 0;
        p.nbuckets = kMaxBins;
        p.max_sub = 1;
        return p;
    }
    // about 512 buckets (swept 128 .. 2048 on V = 1M / E = 17M and V = 233k / E = 115M: 256 .. 512 is
    // fastest; fewer buckets make the first level's runs longer and the second level's shorter)
    p.shift = bits > 9 ? bits - 9 : 0;
    if (p.shift > kMaxBinBits) p.shift = kMaxBinBits;
    p.nbuckets = (int)ceil_div(V > 0 ? V : 1, (int64_t)1 << p.shift);
    p.max_sub = (int)(E / kSubRecords) + p.nbuckets;
    return p;
}

static size_t conv_ws_bytes(int64_t E, int32_t V, bool perm)
{
    ConvPlan p = make_plan(E, V);
    const size_t table_n = (size_t)p.nbuckets * (size_t)p.nblocks + 1;
    size_t b = 0;
    b += carve_bytes(table_n, 4);
    b += carve_bytes(scan_ws_ints((int64_t)table_n), 4);
    // LSD passes keep two buffers of unpacked records; the two-level path one of packed records
    // (the array is carved at the unpacked size either way, which the LSD fallback needs)
    b += carve_bytes((size_t)E, perm ? sizeof(Rec4) : sizeof(Rec3)) * (p.digits > 0 ? 2 : 1);
    b += carve_bytes((size_t)p.max_sub, 4);
    b += carve_bytes((size_t)p.nbuckets + 1, 4);
    b += carve_bytes((size_t)p.max_sub << p.shift, 4);
    return b;
}

template <typename K> static void allow_lds(K kernel, size_t bytes)
{
    if (bytes > 48 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <bool PERM>
static int32_t convert(const int32_t *keys, const int32_t *others, const float *w, int64_t E, int32_t V,
                       int32_t *out_idx, int32_t *out_off, float *out_w, int32_t *out_perm, void *ws,
                       hipStream_t s)
{
    using Rec = typename RecOf<PERM>::type;
    const ConvPlan p = make_plan(E, V);
    Carver carve(ws);
    const size_t table_n = (size_t)p.nbuckets * (size_t)p.nblocks + 1;
    int32_t *table = carve.take<int32_t>(table_n);
    int32_t *sums = carve.take<int32_t>(scan_ws_ints((int64_t)table_n));
    Rec *recs = carve.take<Rec>((size_t)E);
    int32_t *sub_bucket = carve.take<int32_t>((size_t)p.max_sub);
    int32_t *sub_first = carve.take<int32_t>((size_t)p.nbuckets + 1);
    int32_t *cnt2 = carve.take<int32_t>((size_t)p.max_sub << p.shift);
    const unsigned nb = (unsigned)p.nblocks;
    const int nblk = (int)nb;
    int32_t rc;

    if (E == 0) {
        hipLaunchKernelGGL(fill_i32, dim3((unsigned)ceil_div((int64_t)V + 1, 256)), dim3(256), 0, s, out_off,
                           (int64_t)V + 1, 0);
        return launch_status("coo_to_csx(fill)");
    }

    if (p.digits > 0) {
        // V > 2^22: LSD passes over 11-bit digits; sub_first doubles as the record count
        Rec *bufs[2] = {recs, carve.take<Rec>((size_t)E)};
        int32_t *count = sub_first;
        const size_t lds = tile_lds_bytes(kMaxBins, sizeof(Rec));
        const int stage_n = tile_stage_records(kMaxBins, sizeof(Rec));
        for (int d = 0; d < p.digits; d++) {
            const int shift = d * kMaxBinBits;
            Rec *dst = bufs[d & 1];
            if (d == 0) {
                CooLoader<Rec> in{keys, others, reinterpret_cast<const uint32_t *>(w), E, V, 0u};
                hipLaunchKernelGGL((csx_digit_histogram<Rec, CooLoader<Rec>>), dim3((nb + 7) / 8 * 8), dim3(kPartThreads), 0, s, in,
                                   shift, kMaxBins - 1, kMaxBins, table, nblk);
                if ((rc = exclusive_scan_i32(table, table, (int64_t)table_n, sums, s))) return rc;
                hipLaunchKernelGGL(csx_save_count, dim3(1), dim3(1), 0, s, table + (table_n - 1), count);
                auto part = csx_partition<Rec, CooLoader<Rec>>;
                allow_lds(part, lds);
                hipLaunchKernelGGL(part, dim3((nb + 7) / 8 * 8), dim3(kPartThreads), lds, s, in, shift, kMaxBins - 1, kMaxBins,
                                   table, nblk, dst, stage_n);
            } else {
                RecLoader<Rec> in{bufs[(d - 1) & 1], count, E};
                hipLaunchKernelGGL((csx_digit_histogram<Rec, RecLoader<Rec>>), dim3((nb + 7) / 8 * 8), dim3(kPartThreads), 0, s, in,
                                   shift, kMaxBins - 1, kMaxBins, table, nblk);
                if ((rc = exclusive_scan_i32(table, table, (int64_t)table_n, sums, s))) return rc;
                auto part = csx_partition<Rec, RecLoader<Rec>>;
                allow_lds(part, lds);
                hipLaunchKernelGGL(part, dim3((nb + 7) / 8 * 8), dim3(kPartThreads), lds, s, in, shift, kMaxBins - 1, kMaxBins,
                                   table, nblk, dst, stage_n);
            }
        }
        hipLaunchKernelGGL((csx_unpack_sorted<Rec, PERM>), dim3((unsigned)ceil_div(E + 1, 256)), dim3(256), 0, s,
                           bufs[(p.digits - 1) & 1], count, E, V, out_off, out_idx,
                           reinterpret_cast<uint32_t *>(out_w), out_perm);
        zero_tail(out_off, V, E, out_idx, out_w, out_perm, s);
        return launch_status("coo_to_csx(lsd)");
    }

    hipLaunchKernelGGL(csx_bucket_histogram, dim3((nb + 7) / 8 * 8), dim3(kPartThreads), 0, s, keys, E, V, p.shift, p.nbuckets,
                       table, nblk);
    if ((rc = exclusive_scan_i32(table, table, (int64_t)table_n, sums, s))) return rc;

    const uint32_t *wbits = reinterpret_cast<const uint32_t *>(w);
    const int nkeys = 1 << p.shift;
    int kbits = 0;
    while (((int64_t)1 << kbits) < (int64_t)V) kbits++;
    // Packed records need a node id and the low key bits in one word.  Where they do not fit
    // (V above 2^21 with 2048 keys to a bucket) the records stay unpacked: a seventh of the
    // endpoints would otherwise be fetched again one by one.
    const bool packed_ok = kbits + p.shift <= 32;
    auto level2 = [&](auto *records, auto view) {
        using R = typename std::remove_pointer<decltype(records)>::type;
        hipLaunchKernelGGL(csx_plan_subblocks, dim3(1), dim3(1024), 0, s, table, nblk, p.nbuckets, p.max_sub, sub_bucket,
                           sub_first);
        hipLaunchKernelGGL((csx_sub_count<R, decltype(view)>), dim3((unsigned)p.max_sub), dim3(kPartThreads), 0, s,
                           records, table, nblk, sub_bucket, sub_first, view, p.shift, cnt2);
        hipLaunchKernelGGL(csx_bucket_offsets, dim3((unsigned)p.nbuckets), dim3(kPartThreads), 0, s, table, nblk,
                           p.nbuckets, sub_first, p.shift, V, cnt2, out_off, E, out_idx,
                           reinterpret_cast<uint32_t *>(out_w), out_perm);
        auto scat = csx_sub_scatter<R, PERM, decltype(view)>;
        const size_t scat_lds = tile_lds_bytes(nkeys, sizeof(R));
        allow_lds(scat, scat_lds);
        hipLaunchKernelGGL(scat, dim3((unsigned)((p.max_sub + 7) / 8 * 8)), dim3(kPartThreads), scat_lds, s, records, table, nblk,
                           sub_bucket, sub_first, cnt2, view, p.shift, others, wbits, out_idx,
                           reinterpret_cast<uint32_t *>(out_w), out_perm, tile_stage_records(nkeys, sizeof(R)),
                           p.nbuckets, p.max_sub);
    };
    const size_t part_lds = tile_lds_bytes(p.nbuckets, sizeof(Rec));
    if (packed_ok) {
        using Packed = typename PackOf<PERM>::type;
        Packed *packed = reinterpret_cast<Packed *>(recs);
        PackRule rule;
        rule.shift = p.shift;
        rule.obits = 32 - p.shift;
        rule.omask = p.shift ? (((uint32_t)1 << rule.obits) - 1u) : 0xffffffffu;
        CooLoader<Rec> in{keys, others, wbits, E, V, rule.omask};
        auto part = csx_partition_pack<Rec, Packed>;
        allow_lds(part, part_lds);
        hipLaunchKernelGGL(part, dim3((nb + 7) / 8 * 8), dim3(kPartThreads), part_lds, s, in, rule, p.nbuckets, table, nblk, packed,
                           tile_stage_records(p.nbuckets, sizeof(Rec)));
        level2(packed, PackedView{rule});
    } else {
        CooLoader<Rec> in{keys, others, wbits, E, V, 0u};
        auto part = csx_partition<Rec, CooLoader<Rec>>;
        allow_lds(part, part_lds);
        hipLaunchKernelGGL(part, dim3((nb + 7) / 8 * 8), dim3(kPartThreads), part_lds, s, in, p.shift, 0x7fffffff, p.nbuckets,
                           table, nblk, recs, tile_stage_records(p.nbuckets, sizeof(Rec)));
        level2(recs, PlainView{nkeys - 1});
    }
    return launch_status("coo_to_csx");
}

}  // namespace jg

using namespace jg;

static int32_t check_conv_sizes(const char *who, int64_t E, int32_t V)
{
    if (E < 0 || V < 0) return fail(JGAMD_ERR_SIZE, "%s: negative size (E=%lld, V=%d)", who, (long long)E, V);
    if (E >= ((int64_t)1 << 31) - ((int64_t)1 << 20))
        return fail(JGAMD_ERR_SIZE, "%s: E=%lld does not fit int32 offsets", who, (long long)E);
    if (V == INT32_MAX) return fail(JGAMD_ERR_SIZE, "%s: V too large", who);
    return 0;
}

static int32_t check_ws(const char *who, const void *ws, size_t have, size_t need)
{
    if (need == 0) return 0;
    if (!ws || have < need)
        return fail(JGAMD_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws ? have : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "%s: workspace not 256-byte aligned", who);
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_coo_to_csx_workspace(int64_t E, int32_t V, int32_t with_perm, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "coo_to_csx_workspace: bytes is NULL");
    if (int32_t rc = check_conv_sizes("coo_to_csx", E, V)) return rc;
    *bytes = conv_ws_bytes(E, V, with_perm != 0);
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_coo_to_csx(const int32_t *edge_index, const float *edge_weight, int64_t E, int32_t V,
                                    int32_t key_row, int32_t *out_idx, int32_t *out_off, float *out_w,
                                    int32_t *out_perm, void *ws, size_t ws_bytes, void *stream)
{
    if (int32_t rc = check_conv_sizes("coo_to_csx", E, V)) return rc;
    if (key_row != 0 && key_row != 1) return fail(JGAMD_ERR_SIZE, "coo_to_csx: key_row must be 0 or 1");
    if (!out_off) return fail(JGAMD_ERR_NULL, "coo_to_csx: out_off is NULL");
    if (E > 0 && (!edge_index || !edge_weight || !out_idx || !out_w))
        return fail(JGAMD_ERR_NULL, "coo_to_csx: NULL array with E > 0");
    if (int32_t rc = check_ws("coo_to_csx", ws, ws_bytes, conv_ws_bytes(E, V, out_perm != nullptr))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int32_t *keys = edge_index + (key_row ? E : 0);
    const int32_t *others = edge_index + (key_row ? 0 : E);
    return out_perm ? convert<true>(keys, others, edge_weight, E, V, out_idx, out_off, out_w, out_perm, ws, s)
                    : convert<false>(keys, others, edge_weight, E, V, out_idx, out_off, out_w, out_perm, ws, s);
}

static size_t transpose_ws_bytes(int64_t E, int32_t C)
{
    // row of every entry, the tile -> row map it is made from, the conversion's own scratch
    return carve_bytes((size_t)E, 4) + 2 * carve_bytes((size_t)ceil_div(E > 0 ? E : 1, kTileEntriesNarrow), 4) +
           conv_ws_bytes(E, C, true);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_csx_transpose_workspace(int64_t E, int32_t R, int32_t C, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "csx_transpose_workspace: bytes is NULL");
    if (R < 0) return fail(JGAMD_ERR_SIZE, "csx_transpose: negative R");
    if (int32_t rc = check_conv_sizes("csx_transpose", E, C)) return rc;
    *bytes = transpose_ws_bytes(E, C);
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_csx_transpose(const int32_t *off, const int32_t *idx, const float *w, int32_t R, int32_t C,
                                       int64_t E, int32_t *out_off, int32_t *out_idx, float *out_w,
                                       int32_t *out_perm, void *ws, size_t ws_bytes, void *stream)
{
    if (R < 0) return fail(JGAMD_ERR_SIZE, "csx_transpose: negative R");
    if (int32_t rc = check_conv_sizes("csx_transpose", E, C)) return rc;
    if (!off || !out_off) return fail(JGAMD_ERR_NULL, "csx_transpose: off/out_off is NULL");
    if (E > 0 && (!idx || !out_idx)) return fail(JGAMD_ERR_NULL, "csx_transpose: NULL array with E > 0");
    if (out_w && !w) return fail(JGAMD_ERR_NULL, "csx_transpose: out_w given without w");
    if (int32_t rc = check_ws("csx_transpose", ws, ws_bytes, transpose_ws_bytes(E, C))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Carver carve(ws);
    int32_t *rows = carve.take<int32_t>((size_t)E);
    const size_t ntiles = (size_t)ceil_div(E > 0 ? E : 1, kTileEntriesNarrow);
    int32_t *tile_first = carve.take<int32_t>(ntiles), *tile_last = carve.take<int32_t>(ntiles);
    void *inner = carve.base + carve.used;
    if (E > 0 && R > 0) {
        tile_columns_enqueue(off, R, E, kTileEntriesNarrow, tile_first, tile_last, s);
        hipLaunchKernelGGL(csx_expand_rows, dim3((unsigned)ntiles), dim3(256), 0, s, off, tile_first, tile_last, R, E,
                           rows);
    }
    return out_perm ? convert<true>(idx, rows, w, E, C, out_idx, out_off, out_w, out_perm, inner, s)
                    : convert<false>(idx, rows, w, E, C, out_idx, out_off, out_w, out_perm, inner, s);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_invert_permutation(const int32_t *perm, int64_t n, int32_t *inv, void *stream)
{
    if (n < 0 || n >= ((int64_t)1 << 31)) return fail(JGAMD_ERR_SIZE, "invert_permutation: n=%lld out of range", (long long)n);
    if (n == 0) return 0;
    if (!perm || !inv) return fail(JGAMD_ERR_NULL, "invert_permutation: NULL array");
    hipLaunchKernelGGL(csx_invert_permutation, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), perm, n, inv);
    return launch_status("invert_permutation");
}
