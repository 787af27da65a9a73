// COO -> CSR/CSC as a stable two-level counting sort.
//
// The reference (ops/cpp/cootocsr_op.cc:35-53, cootocsc_op.cc:33-51) is a
// sequential counting sort: histogram of the key, prefix sum, then a scatter
// in input order, so edges of one row keep their input order.  Atomics on a
// GPU cannot give that order, so the scatter is done as two stable
// partitions, each ranking its items with wave-level match + popcount:
//
//   1. histogram   : off[key] += 1 (global atomics) and, per block, a count of
//                    the block's items per BUCKET (bucket = key >> shift,
//                    at most 2048 buckets).
//   2. scans       : off -> exclusive prefix (the final offsets); the
//                    (bucket, block) count table -> exclusive prefix, which
//                    is each block's write cursor in each bucket.
//   3. partition   : every block re-reads its items and writes them, as
//                    12/16-byte records, to their bucket in input order.
//   4. bucket sort : one block per bucket walks the bucket's records in
//                    order and places each at off[key] + (rank among equal
//                    keys so far); the bucket's output window is a few
//                    hundred KB, so these scattered writes combine in L2.
//
// Two levels of at most 2048 bins each cover V <= 2^22 vertices.
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

template <bool PERM> struct RecOf { using type = Rec3; };
template <> struct RecOf<true> { using type = Rec4; };

__device__ __forceinline__ void set_id(Rec3 &, int32_t) {}
__device__ __forceinline__ void set_id(Rec4 &r, int32_t id) { r.id = id; }
__device__ __forceinline__ int32_t get_id(const Rec3 &) { return 0; }
__device__ __forceinline__ int32_t get_id(const Rec4 &r) { return r.id; }

// ---------------------------------------------------------------- step 1 ---
// keys: the key row of edge_index.  Items with key outside [0,V) are ignored
// here and in every later step.
__global__ __launch_bounds__(kPartThreads) void csx_histogram(const int32_t *__restrict__ keys, int64_t E,
                                                              int32_t V, int shift, int nbins,
                                                              int32_t *__restrict__ off_counts,
                                                              int32_t *__restrict__ table, int nblocks)
{
    __shared__ int bins[kMaxBins];
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) bins[b] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * kTile;
#pragma unroll 4
    for (int i = 0; i < kItems; i++) {
        int64_t e = base + (int64_t)i * kPartThreads + threadIdx.x;
        if (e < E) {
            int32_t k = keys[e];
            if ((uint32_t)k < (uint32_t)V) {
                atomicAdd(&off_counts[k], 1);
                atomicAdd(&bins[k >> shift], 1);
            }
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += kPartThreads)
        table[(int64_t)b * nblocks + blockIdx.x] = bins[b];
}

// ------------------------------------------------------- stable tile rank ---
// The block's tile is kTile consecutive items; wave w owns the kWaveSpan
// consecutive items starting at w*kWaveSpan and visits them in rounds of 64
// (lane l = item r*64 + l), so (wave, round, lane) is the input order.
// cnt is [kPartWaves][nbins] in LDS.  On entry cnt is undefined; `cursor(b)`
// gives the position of the first item of bin b in this tile.  On exit
// pos[r] is the destination of this thread's item of round r (bin[r] < 0:
// item absent).  `after(b, end)` is called once per bin with the position
// one past the tile's last item of bin b.
template <typename Cursor, typename After>
__device__ __forceinline__ void tile_rank(int *cnt, int nbins, int nbits, const int (&bin)[kItems],
                                          int (&pos)[kItems], Cursor cursor, After after)
{
    const int w = threadIdx.x >> 6;
    const int lane = lane_id();
    int *mine = cnt + w * nbins;
    for (int b = threadIdx.x; b < nbins * kPartWaves; b += kPartThreads) cnt[b] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kItems; r++)
        if (bin[r] >= 0) atomicAdd(&mine[bin[r]], 1);
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += kPartThreads) {
        int run = cursor(b);
#pragma unroll
        for (int v = 0; v < kPartWaves; v++) {
            int c = cnt[v * nbins + b];
            cnt[v * nbins + b] = run;
            run += c;
        }
        after(b, run);
    }
    __syncthreads();
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (kWave - lane));
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        const int b = bin[r];
        const bool valid = b >= 0;
        uint64_t peers = __ballot(valid);
        for (int t = 0; t < nbits; t++) {
            const bool bit = (b >> t) & 1;
            const uint64_t vote = __ballot(bit);
            peers &= bit ? vote : ~vote;
        }
        // peers: valid lanes of this round with the same bin as this lane
        const int leader = __ffsll((unsigned long long)peers) - 1;
        const int rank = __popcll(peers & below);
        int start = 0;
        if (valid && lane == leader) start = atomicAdd(&mine[b], __popcll(peers));
        start = __shfl(start, leader < 0 ? 0 : leader, kWave);
        pos[r] = start + rank;
    }
}

// ---------------------------------------------------------------- step 3 ---
// Loader for the first partition: items come from the COO arrays.
template <typename Rec> struct CooLoader {
    const int32_t *keys;
    const int32_t *others;
    const uint32_t *w;
    int64_t n;
    int32_t V;
    __device__ __forceinline__ bool load(int64_t e, Rec &r) const
    {
        if (e >= n) return false;
        r.key = keys[e];
        r.other = others[e];
        r.w = w ? w[e] : 0u;
        set_id(r, (int32_t)e);
        return (uint32_t)r.key < (uint32_t)V;
    }
};
template <typename Rec, typename Loader>
__global__ __launch_bounds__(kPartThreads) void csx_partition(Loader in, int shift, int mask, int nbins,
                                                              int nbits, const int32_t *__restrict__ table,
                                                              int nblocks, Rec *__restrict__ out)
{
    extern __shared__ int cnt[];
    const int w = threadIdx.x >> 6;
    const int64_t base = (int64_t)blockIdx.x * kTile + (int64_t)w * kWaveSpan + lane_id();
    Rec rec[kItems];
    int bin[kItems], pos[kItems];
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        bool ok = in.load(base + (int64_t)r * kWave, rec[r]);
        bin[r] = ok ? ((rec[r].key >> shift) & mask) : -1;
    }
    const int blk = blockIdx.x;
    tile_rank(
        cnt, nbins, nbits, bin, pos, [&](int b) { return table[(int64_t)b * nblocks + blk]; },
        [](int, int) {});
#pragma unroll
    for (int r = 0; r < kItems; r++)
        if (bin[r] >= 0) out[pos[r]] = rec[r];
}

// ---------------------------------------------------------------- step 4 ---
// One block per bucket: keys [b << shift, (b+1) << shift) and the records
// recs[off[first key] .. off[last key + 1]).  Chunks of kTile records are
// ranked in order; cursor[] (LDS) carries each key's next free slot from one
// chunk to the next.
template <typename Rec, bool PERM>
__global__ __launch_bounds__(kPartThreads) void csx_bucket_sort(const Rec *__restrict__ recs,
                                                                const int32_t *__restrict__ off, int32_t V,
                                                                int shift, int nbits,
                                                                int32_t *__restrict__ out_idx,
                                                                uint32_t *__restrict__ out_w,
                                                                int32_t *__restrict__ out_perm)
{
    extern __shared__ int lds[];
    const int nkeys = 1 << shift;
    int *cursor = lds;               // [nkeys]
    int *cnt = lds + nkeys;          // [kPartWaves][nkeys]
    const int64_t k0 = (int64_t)blockIdx.x << shift;
    const int64_t k1 = min((int64_t)V, k0 + nkeys);
    const int begin = off[k0], end = off[k1];
    for (int k = threadIdx.x; k < nkeys; k += kPartThreads)
        cursor[k] = k0 + k < V ? off[k0 + k] : end;
    __syncthreads();
    const int w = threadIdx.x >> 6;
    const int mask = nkeys - 1;
    for (int chunk = begin; chunk < end; chunk += kTile) {
        const int base = chunk + w * kWaveSpan + lane_id();
        Rec rec[kItems];
        int bin[kItems], pos[kItems];
#pragma unroll
        for (int r = 0; r < kItems; r++) {
            int e = base + r * kWave;
            bool ok = e < end;
            if (ok) rec[r] = recs[e];
            bin[r] = ok ? (rec[r].key & mask) : -1;
        }
        tile_rank(
            cnt, nkeys, nbits, bin, pos, [&](int b) { return cursor[b]; },
            [&](int b, int next) { cursor[b] = next; });
#pragma unroll
        for (int r = 0; r < kItems; r++)
            if (bin[r] >= 0) {
                out_idx[pos[r]] = rec[r].other;
                if (out_w) out_w[pos[r]] = rec[r].w;
                if (PERM) out_perm[pos[r]] = get_id(rec[r]);
            }
        __syncthreads();
    }
}

// Expands compressed offsets into one row id per entry (for the transpose).
__global__ void csx_expand_rows(const int32_t *__restrict__ off, int32_t R, int32_t *__restrict__ rows)
{
    // one wave per row keeps long rows coalesced; short rows cost one store
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * (blockDim.x >> 6);
    for (int r = wave; r < R; r += nwaves) {
        const int s = off[r], e = off[r + 1];
        for (int j = s + lane_id(); j < e; j += kWave) rows[j] = r;
    }
}

__global__ void fill_i32(int32_t *p, int64_t n, int32_t v)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ------------------------------------------------------------------ host ---
struct ConvPlan {
    int shift;        // low key bits handled by the bucket sort
    int nbuckets;     // bins of the partition
    int64_t nblocks;  // tiles of kTile items
};

static ConvPlan make_plan(int64_t E, int32_t V)
{
    ConvPlan p{};
    int bits = 0;
    while (bits < 31 && ((int64_t)1 << bits) < (int64_t)V) bits++;   // keys < 2^bits
    p.nblocks = ceil_div(E > 0 ? E : 1, kTile);
    p.shift = bits > 10 ? bits - 10 : 0;
    if (p.shift > kMaxBinBits) p.shift = kMaxBinBits;
    p.nbuckets = (int)ceil_div(V > 0 ? V : 1, (int64_t)1 << p.shift);
    return p;
}

static int64_t scan_len(const ConvPlan &p, int32_t V)
{
    int64_t table = (int64_t)p.nbuckets * p.nblocks;
    return table > (int64_t)V + 1 ? table : (int64_t)V + 1;
}

static size_t conv_ws_bytes(int64_t E, int32_t V, bool perm)
{
    ConvPlan p = make_plan(E, V);
    size_t b = 0;
    b += carve_bytes((size_t)p.nbuckets * (size_t)p.nblocks, 4);
    b += carve_bytes(scan_ws_ints(scan_len(p, V)), 4);
    b += carve_bytes((size_t)E, perm ? sizeof(Rec4) : sizeof(Rec3));
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
    const size_t table_n = (size_t)p.nbuckets * (size_t)p.nblocks;
    int32_t *table = carve.take<int32_t>(table_n);
    int32_t *sums = carve.take<int32_t>(scan_ws_ints(scan_len(p, V)));
    Rec *recs = carve.take<Rec>((size_t)E);
    const unsigned nb = (unsigned)p.nblocks;
    int32_t rc;

    hipLaunchKernelGGL(fill_i32, dim3((unsigned)ceil_div((int64_t)V + 1, 256)), dim3(256), 0, s, out_off,
                       (int64_t)V + 1, 0);
    if (E == 0) return launch_status("coo_to_csx(fill)");

    int bbits = 0;
    while ((1 << bbits) < p.nbuckets) bbits++;
    hipLaunchKernelGGL(csx_histogram, dim3(nb), dim3(kPartThreads), 0, s, keys, E, V, p.shift, p.nbuckets, out_off,
                       table, (int)nb);
    if ((rc = exclusive_scan_i32(out_off, out_off, (int64_t)V + 1, sums, s))) return rc;
    if ((rc = exclusive_scan_i32(table, table, (int64_t)table_n, sums, s))) return rc;

    CooLoader<Rec> in{keys, others, reinterpret_cast<const uint32_t *>(w), E, V};
    auto part = csx_partition<Rec, CooLoader<Rec>>;
    const size_t part_lds = (size_t)kPartWaves * p.nbuckets * sizeof(int);
    allow_lds(part, part_lds);
    hipLaunchKernelGGL(part, dim3(nb), dim3(kPartThreads), part_lds, s, in, p.shift, 0x7fffffff, p.nbuckets, bbits,
                       table, (int)nb, recs);

    const int nkeys = 1 << p.shift;
    auto sort = csx_bucket_sort<Rec, PERM>;
    const size_t sort_lds = (size_t)(kPartWaves + 1) * nkeys * sizeof(int);
    allow_lds(sort, sort_lds);
    hipLaunchKernelGGL(sort, dim3((unsigned)p.nbuckets), dim3(kPartThreads), sort_lds, s, recs, out_off, V, p.shift,
                       p.shift, out_idx, reinterpret_cast<uint32_t *>(out_w), out_perm);
    return launch_status("coo_to_csx");
}

}  // namespace jg

using namespace jg;

static int32_t check_conv_sizes(const char *who, int64_t E, int32_t V)
{
    if (E < 0 || V < 0) return fail(JGAMD_ERR_SIZE, "%s: negative size (E=%lld, V=%d)", who, (long long)E, V);
    if (E >= ((int64_t)1 << 31) - ((int64_t)1 << 20))
        return fail(JGAMD_ERR_SIZE, "%s: E=%lld does not fit int32 offsets", who, (long long)E);
    if ((int64_t)V > ((int64_t)1 << (2 * kMaxBinBits)))
        return fail(JGAMD_ERR_UNSUPPORTED, "%s: V=%d above 2^22 is not supported", who, V);
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
    return carve_bytes((size_t)E, 4) + conv_ws_bytes(E, C, true);
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
    void *inner = carve.base + carve.used;
    if (E > 0 && R > 0) {
        int blocks = (int)(ceil_div(R, 4) < 65536 ? ceil_div(R, 4) : 65536);
        hipLaunchKernelGGL(csx_expand_rows, dim3(blocks), dim3(256), 0, s, off, R, rows);
    }
    return out_perm ? convert<true>(idx, rows, w, E, C, out_idx, out_off, out_w, out_perm, inner, s)
                    : convert<false>(idx, rows, w, E, C, out_idx, out_off, out_w, out_perm, inner, s);
}
