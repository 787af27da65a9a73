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

__global__ void scale_edge_weights(const int32_t *__restrict__ row, const int32_t *__restrict__ col,
                                   const float *__restrict__ w, const float *__restrict__ a,
                                   const float *__restrict__ b, int64_t E, int32_t N, float *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    float v = w[e];
    if (a) {
        const int r = row[e];
        v = ((unsigned)r < (unsigned)N ? a[r] : 0.f) * v;
    }
    if (b) {
        const int c = col[e];
        v = v * ((unsigned)c < (unsigned)N ? b[c] : 0.f);
    }
    out[e] = v;
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
