// Graph preprocessing in front of the conversion: self-loop handling and the
// degree normalisation of the edge weights.
//
// add_remaining_self_loops (utils/loop.py:98-136 of the reference): the
// self-loops of the input are dropped, the other edges keep their order, and
// one loop per node is appended; a node's loop takes the weight of its dropped
// loop (the last one in input order, which is what the reference's indexed
// assignment leaves), every other loop the fill value.  Here: per-block counts
// of the kept edges, a scan of the counts, and a scatter in which each block
// ranks its own kept edges by a block scan, so the order is the input order
// without any atomic.  The "last loop of node v" is an integer atomicMax of
// the edge id, which is order-independent.
//
// sym/mean normalisation (nn/conv/gcn_conv.py:33-37, nn/conv/sage_conv.py:36-40):
// w'[e] = a[row[e]] * w[e] * b[col[e]] with a, b = deg^p (inf -> 0); the degree
// itself is the column sum computed through the conversion.
#include "common.h"

namespace jg {

constexpr int kLoopThreads = 256;
constexpr int kLoopItems = 8;                        // edges per thread
constexpr int kLoopTile = kLoopThreads * kLoopItems; // edges per block

__global__ void norm_fill_i32(int32_t *p, int64_t n, int32_t v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// counts[b] = edges of tile b with row != col; last_loop[v] = max id of a self-loop (v, v)
__global__ __launch_bounds__(kLoopThreads) void loops_count(const int32_t *__restrict__ row,
                                                            const int32_t *__restrict__ col, int64_t E, int32_t N,
                                                            int32_t *__restrict__ counts,
                                                            int32_t *__restrict__ last_loop)
{
    __shared__ int wave_sum[kLoopThreads / kWave];
    const int64_t base = (int64_t)blockIdx.x * kLoopTile;
    int kept = 0;
#pragma unroll
    for (int i = 0; i < kLoopItems; i++) {
        const int64_t e = base + (int64_t)i * kLoopThreads + threadIdx.x;
        if (e < E) {
            const int r = row[e], c = col[e];
            if (r != c) kept++;
            else if ((unsigned)r < (unsigned)N) atomicMax(&last_loop[r], (int32_t)e);
        }
    }
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) kept += __shfl_xor(kept, o, kWave);
    if (lane_id() == 0) wave_sum[threadIdx.x >> 6] = kept;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int v = 0; v < kLoopThreads / kWave; v++) t += wave_sum[v];
        counts[blockIdx.x] = t;
    }
}

// Kept edges of tile b go to positions base[b] + (rank inside the tile, input order).
// Edge (round i, thread t) = base + i*256 + t, so loads and stores of a round are coalesced; its
// rank = kept edges of earlier rounds + of earlier wavefronts in the round + of lower lanes.
__global__ __launch_bounds__(kLoopThreads) void loops_scatter(const int32_t *__restrict__ row,
                                                              const int32_t *__restrict__ col,
                                                              const float *__restrict__ w, int64_t E,
                                                              const int32_t *__restrict__ base,
                                                              const int32_t *__restrict__ total_kept, int32_t N,
                                                              int32_t *__restrict__ out_index,
                                                              float *__restrict__ out_w)
{
    constexpr int kWaves = kLoopThreads / kWave;
    __shared__ int cnt[kLoopItems][kWaves];
    const int64_t first = (int64_t)blockIdx.x * kLoopTile + threadIdx.x;
    const int wv = threadIdx.x >> 6, lane = lane_id();
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (kWave - lane));
    int r[kLoopItems], c[kLoopItems], rank[kLoopItems];
    float ww[kLoopItems];
#pragma unroll
    for (int i = 0; i < kLoopItems; i++) {
        const int64_t e = first + (int64_t)i * kLoopThreads;
        const int64_t ec = e < E ? e : E - 1;
        r[i] = row[ec];
        c[i] = col[ec];
        ww[i] = w ? w[ec] : 1.f;
        if (e >= E) r[i] = c[i];        // past the end: treated as dropped
    }
#pragma unroll
    for (int i = 0; i < kLoopItems; i++) {
        const uint64_t keep = __ballot(r[i] != c[i]);
        rank[i] = __popcll(keep & below);
        if (lane == 0) cnt[i][wv] = __popcll(keep);
    }
    __syncthreads();
    const int64_t out_E = (int64_t)*total_kept + N;     // row 1 of out_index starts here
    int64_t pos = base[blockIdx.x];
#pragma unroll
    for (int i = 0; i < kLoopItems; i++) {
        int before = 0, round_total = 0;
#pragma unroll
        for (int v = 0; v < kWaves; v++) {
            const int n = cnt[i][v];
            before += v < wv ? n : 0;
            round_total += n;
        }
        if (r[i] != c[i]) {
            const int64_t p = pos + before + rank[i];
            out_index[p] = r[i];
            out_index[out_E + p] = c[i];
            out_w[p] = ww[i];
        }
        pos += round_total;
    }
}

__global__ void loops_append(const float *__restrict__ w, const int32_t *__restrict__ last_loop,
                             const int32_t *__restrict__ total_kept, int32_t N, float fill,
                             int32_t *__restrict__ out_index, float *__restrict__ out_w)
{
    const int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= N) return;
    const int64_t kept = *total_kept;
    const int64_t out_E = kept + N;
    out_index[kept + v] = v;
    out_index[out_E + kept + v] = v;
    const int32_t e = last_loop[v];
    out_w[kept + v] = (w && e >= 0) ? w[e] : fill;
}

// a[v] = deg[v]^power with inf -> 0 (power -0.5: 1/sqrt, -1: 1/x, as the reference's pow gives)
__global__ void degree_power(const float *__restrict__ deg, int32_t N, float power, float *__restrict__ out)
{
    const int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= N) return;
    const float p = powf(deg[v], power);
    out[v] = isinf(p) ? 0.f : p;
}

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4n __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float scaled(float w, const float *a, const float *b, int r, int c, int N)
{
    float v = w;
    if (a) v = ((unsigned)r < (unsigned)N ? a[r] : 0.f) * v;
    if (b) v = v * ((unsigned)c < (unsigned)N ? b[c] : 0.f);
    return v;
}

// One edge per thread.  The time goes into the two reads at random places of the factor arrays
// (4 MB each at a million nodes: L2 request rate, not bytes); four edges per thread with
// streamed (non-temporal) 16-byte accesses for the edge arrays was slower, 297 against 211 us
// on 17M edges.
__global__ __launch_bounds__(256) void scale_edge_weights(const int32_t *__restrict__ row, const int32_t *__restrict__ col,
                                                          const float *__restrict__ w, const float *__restrict__ a,
                                                          const float *__restrict__ b, int64_t E, int32_t N,
                                                          float *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    out[e] = scaled(w[e], a, b, row[e], col[e], N);
}

// The same product for weights that sit in compressed (slot) order: slot j of column c holds the
// edge (idx[j] -> c), so out[j] = a[idx[j]] * w[j] * b[c], the expression above term for term.
// A block takes one tile of kTileEntriesNarrow slots; the columns of its first and last slot
// come from the tile -> column map, their offsets are staged in LDS, every thread finds the
// column of its first slot by bisection there and walks on from it.
constexpr int kScaleSlots = 4;      // slots per thread
__global__ __launch_bounds__(256) void scale_csx_weights(const int32_t *__restrict__ off,
                                                         const int32_t *__restrict__ idx, const float *__restrict__ w,
                                                         const float *__restrict__ a, const float *__restrict__ b,
                                                         const int32_t *__restrict__ tile_first,
                                                         const int32_t *__restrict__ tile_last, int32_t V, int64_t E,
                                                         int32_t N, float *__restrict__ out, int vectors)
{
    constexpr int T = kTileEntriesNarrow;
    static_assert(T == 256 * kScaleSlots, "one tile per block");
    __shared__ int s_off[T + 2];
    const int tile = blockIdx.x;
    const int64_t t0 = (int64_t)tile * T;
    const int covered = min(max(off[V], 0), (int)E);
    // slots past off[V] hold no edge (a conversion that dropped keys left zeros there)
    if (t0 >= covered) {
        for (int64_t j = t0 + threadIdx.x; j < E && j < t0 + T; j += 256) out[j] = 0.f;
        return;
    }
    const int c_lo = min(max(tile_first[tile], 0), V - 1);
    const int c_hi = min(max(tile_last[tile], c_lo), V - 1);
    const int ncol = c_hi - c_lo + 1;
    const bool staged = ncol + 1 <= T + 2;
    if (staged)
        for (int i = threadIdx.x; i <= ncol; i += 256) s_off[i] = off[c_lo + i];
    __syncthreads();
    auto offv = [&](int c) { return staged ? s_off[c - c_lo] : off[c]; };
    const int64_t j0 = t0 + (int64_t)threadIdx.x * kScaleSlots;
    const int last = covered - 1;
    const int jc = (int)min(j0, (int64_t)last);
    int lo = c_lo, hi = c_hi;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (offv(mid) <= jc) lo = mid;
        else hi = mid - 1;
    }
    int c = lo, ce = offv(c + 1);
    if (vectors && j0 + kScaleSlots <= E) {
        // the thread's four slots as one 16-byte access per array, the four factor reads in flight together
        const i32x4 iv = *reinterpret_cast<const i32x4 *>(idx + j0);
        const f32x4n wv = *reinterpret_cast<const f32x4n *>(w + j0);
        float av[kScaleSlots];
#pragma unroll
        for (int k = 0; k < kScaleSlots; k++) av[k] = (a && (unsigned)iv[k] < (unsigned)N) ? a[iv[k]] : 0.f;
        f32x4n o;
#pragma unroll
        for (int k = 0; k < kScaleSlots; k++) {
            const int64_t j = j0 + k;
            while (ce <= j && c < c_hi) {
                c++;
                ce = offv(c + 1);
            }
            float v = wv[k];
            if (a) v = av[k] * v;
            if (b) v = v * ((unsigned)c < (unsigned)N ? b[c] : 0.f);
            o[k] = j > last ? 0.f : v;
        }
        *reinterpret_cast<f32x4n *>(out + j0) = o;
        return;
    }
#pragma unroll
    for (int k = 0; k < kScaleSlots; k++) {
        const int64_t j = j0 + k;
        if (j >= E) break;
        if (j > last) {
            out[j] = 0.f;
            continue;
        }
        while (ce <= j && c < c_hi) {
            c++;
            ce = offv(c + 1);
        }
        out[j] = scaled(w[j], a, b, idx[j], c, N);
    }
}

__global__ void scale_copy_kept(const int32_t *__restrict__ total, int32_t *__restrict__ out) { *out = *total; }

static int64_t loop_blocks(int64_t E) { return ceil_div(E > 0 ? E : 1, kLoopTile); }
static size_t loops_ws_bytes(int64_t E, int32_t N)
{
    const int64_t nb = loop_blocks(E) + 1;
    return carve_bytes((size_t)nb, 4) + carve_bytes(scan_ws_ints(nb), 4) + carve_bytes((size_t)(N > 0 ? N : 1), 4);
}

}  // namespace jg

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

JG_EXPORT int32_t jgamd_add_remaining_self_loops_workspace(int64_t E, int32_t N, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "add_remaining_self_loops_workspace: bytes is NULL");
    if (E < 0 || N < 0) return fail(JGAMD_ERR_SIZE, "add_remaining_self_loops: negative size");
    *bytes = loops_ws_bytes(E, N);
    return 0;
}

JG_EXPORT int32_t jgamd_add_remaining_self_loops(const int32_t *edge_index, const float *edge_weight, int64_t E,
                                                 int32_t N, float fill, int32_t *out_index, float *out_weight,
                                                 int32_t *out_kept, void *ws, size_t ws_bytes, void *stream)
{
    if (E < 0 || N < 0) return fail(JGAMD_ERR_SIZE, "add_remaining_self_loops: negative size");
    if (E + N >= ((int64_t)1 << 31)) return fail(JGAMD_ERR_SIZE, "add_remaining_self_loops: E + N does not fit int32");
    if (!out_index || !out_weight || !out_kept) return fail(JGAMD_ERR_NULL, "add_remaining_self_loops: NULL output");
    if (E > 0 && !edge_index) return fail(JGAMD_ERR_NULL, "add_remaining_self_loops: edge_index is NULL");
    const size_t need = loops_ws_bytes(E, N);
    if (!ws || ws_bytes < need)
        return fail(JGAMD_ERR_WORKSPACE, "add_remaining_self_loops: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "add_remaining_self_loops: workspace not 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t nb = loop_blocks(E);
    Carver carve(ws);
    int32_t *counts = carve.take<int32_t>((size_t)nb + 1);
    int32_t *sums = carve.take<int32_t>(scan_ws_ints(nb + 1));
    int32_t *last_loop = carve.take<int32_t>((size_t)(N > 0 ? N : 1));
    const int32_t *row = edge_index, *col = edge_index + E;
    if (N > 0)
        hipLaunchKernelGGL(norm_fill_i32, dim3((unsigned)ceil_div(N, 256)), dim3(256), 0, s, last_loop, (int64_t)N, -1);
    // counts[nb] = 0 so that the exclusive scan leaves the total there
    hipLaunchKernelGGL(norm_fill_i32, dim3(1), dim3(1), 0, s, counts + nb, (int64_t)1, 0);
    if (E > 0)
        hipLaunchKernelGGL(loops_count, dim3((unsigned)nb), dim3(kLoopThreads), 0, s, row, col, E, N, counts, last_loop);
    else
        hipLaunchKernelGGL(norm_fill_i32, dim3(1), dim3(1), 0, s, counts, (int64_t)1, 0);
    if (int32_t rc = exclusive_scan_i32(counts, counts, nb + 1, sums, s)) return rc;
    if (E > 0)
        hipLaunchKernelGGL(loops_scatter, dim3((unsigned)nb), dim3(kLoopThreads), 0, s, row, col, edge_weight, E, counts,
                           counts + nb, N, out_index, out_weight);
    if (N > 0)
        hipLaunchKernelGGL(loops_append, dim3((unsigned)ceil_div(N, 256)), dim3(256), 0, s, edge_weight, last_loop,
                           counts + nb, N, fill, out_index, out_weight);
    hipLaunchKernelGGL(scale_copy_kept, dim3(1), dim3(1), 0, s, counts + nb, out_kept);
    return launch_status("add_remaining_self_loops");
}

JG_EXPORT int32_t jgamd_degree_power(const float *deg, int32_t N, float power, float *out, void *stream)
{
    if (N < 0) return fail(JGAMD_ERR_SIZE, "degree_power: negative size");
    if (N == 0) return 0;
    if (!deg || !out) return fail(JGAMD_ERR_NULL, "degree_power: NULL array");
    hipLaunchKernelGGL(degree_power, dim3((unsigned)ceil_div(N, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       deg, N, power, out);
    return launch_status("degree_power");
}

JG_EXPORT int32_t jgamd_scale_edge_weights(const int32_t *edge_index, const float *edge_weight, const float *by_row,
                                           const float *by_col, int64_t E, int32_t N, float *out, void *stream)
{
    if (E < 0 || N < 0) return fail(JGAMD_ERR_SIZE, "scale_edge_weights: negative size");
    if (E == 0) return 0;
    if (!edge_index || !edge_weight || !out) return fail(JGAMD_ERR_NULL, "scale_edge_weights: NULL array");
    hipLaunchKernelGGL(scale_edge_weights, dim3((unsigned)ceil_div(E, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), edge_index, edge_index + E, edge_weight, by_row, by_col, E, N,
                       out);
    return launch_status("scale_edge_weights");
}

JG_EXPORT int32_t jgamd_scale_csx_weights_workspace(int64_t E, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "scale_csx_weights_workspace: bytes is NULL");
    if (E < 0) return fail(JGAMD_ERR_SIZE, "scale_csx_weights: negative size");
    *bytes = 2 * carve_bytes((size_t)ceil_div(E > 0 ? E : 1, kTileEntriesNarrow), 4);
    return 0;
}

JG_EXPORT int32_t jgamd_scale_csx_weights(const int32_t *off, const int32_t *idx, const float *w, const float *by_idx,
                                          const float *by_seg, int32_t V, int64_t E, int32_t N, float *out, void *ws,
                                          size_t ws_bytes, void *stream)
{
    if (E < 0 || V < 0 || N < 0) return fail(JGAMD_ERR_SIZE, "scale_csx_weights: negative size");
    if (E >= ((int64_t)1 << 31) - ((int64_t)1 << 20)) return fail(JGAMD_ERR_SIZE, "scale_csx_weights: E does not fit int32");
    if (E == 0) return 0;
    if (V == 0) return fail(JGAMD_ERR_SIZE, "scale_csx_weights: E > 0 with V = 0");
    if (!off || !idx || !w || !out) return fail(JGAMD_ERR_NULL, "scale_csx_weights: NULL array");
    size_t need = 0;
    (void)jgamd_scale_csx_weights_workspace(E, &need);
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "scale_csx_weights: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "scale_csx_weights: workspace not 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Carver carve(ws);
    const size_t ntiles = (size_t)ceil_div(E, kTileEntriesNarrow);
    int32_t *tile_first = carve.take<int32_t>(ntiles);
    int32_t *tile_last = carve.take<int32_t>(ntiles);
    tile_columns_enqueue(off, V, E, kTileEntriesNarrow, tile_first, tile_last, s);
    const int vectors = (((uintptr_t)idx | (uintptr_t)w | (uintptr_t)out) & 15) == 0;
    hipLaunchKernelGGL(scale_csx_weights, dim3((unsigned)ntiles), dim3(256), 0, s, off, idx, w, by_idx, by_seg,
                       tile_first, tile_last, V, E, N, out, vectors);
    return launch_status("scale_csx_weights");
}
