// Neighbour sampling for one layer of a sampled subgraph.
//
// The reference (ops/cpp/sampleprocessing_op.cc:47-84 on the CPU, :88-160 on the
// GPU) copies all neighbours of a destination when it has at most `fanout` of
// them and otherwise draws `fanout` distinct ones with rand() / a curand state
// seeded from clock64(), so two runs never agree.  Here the draw is a pure
// function of (seed, destination id): Floyd's algorithm picks a uniform
// k-subset of {0..deg-1} with k draws, each draw a 64-bit mix of (seed,
// destination, step).  Work per destination is O(k^2) whatever its degree, the
// picks are stored in the output slots themselves, sorted, and then replaced
// by the neighbour ids, so a destination's sampled neighbours keep the order
// they have in the global arrays.
#include "common.h"

namespace jg {

__device__ __forceinline__ uint32_t sample_mix(uint64_t seed, uint32_t node, uint32_t step)
{
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (((uint64_t)node << 32) | step);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint32_t)(z >> 32);
}

__global__ void sample_neighbors_k(const int32_t *__restrict__ dst, const int32_t *__restrict__ layer_off,
                                   const int32_t *__restrict__ g_off, const int32_t *__restrict__ g_idx, int n_dst,
                                   int g_nodes, int fanout, int64_t out_len, uint64_t seed, int32_t *__restrict__ out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_dst) return;
    const int64_t pos = layer_off[i];
    const int64_t cap = (int64_t)layer_off[i + 1] - pos;
    if (pos < 0 || cap <= 0 || pos + cap > out_len) return;
    const int node = dst[i];
    if ((unsigned)node >= (unsigned)g_nodes) return;
    const int start = g_off[node];
    const int deg = g_off[node + 1] - start;
    if (deg <= 0) return;
    int32_t *mine = out + pos;
    if (fanout < 0 || deg <= fanout) {
        const int n = (int)min((int64_t)deg, cap);
        for (int j = 0; j < n; j++) mine[j] = g_idx[start + j];
        return;
    }
    const int k = (int)min((int64_t)fanout, cap);
    // Floyd: for j = deg-k .. deg-1 draw t in [0, j]; take t unless it was taken, then take j
    int have = 0;
    for (int j = deg - k; j < deg; j++) {
        const uint32_t r = sample_mix(seed, (uint32_t)node, (uint32_t)(j - (deg - k)));
        int t = (int)(((uint64_t)r * (uint64_t)(j + 1)) >> 32);
        bool taken = false;
        for (int q = 0; q < have; q++) taken |= mine[q] == t;
        if (taken) t = j;
        // insert keeping mine[0..have) ascending
        int q = have;
        while (q > 0 && mine[q - 1] > t) {
            mine[q] = mine[q - 1];
            q--;
        }
        mine[q] = t;
        have++;
    }
    for (int q = 0; q < k; q++) mine[q] = g_idx[start + mine[q]];
}

// ---- per-destination list lengths and their offsets -------------------------
// length of dst[i]'s list = min(size of column dst[i] of the global arrays, cap), 0 for a
// destination outside [0, g_nodes).  lead = 1: counts[0] = 0 and the lengths follow from slot 1
// (the layout the sampling script scans); lead = 0: lengths from slot 0 and a zero in slot
// n_dst, ready for an exclusive scan over n_dst + 1 slots.
__global__ void layer_column_counts(const int32_t *__restrict__ dst, const int32_t *__restrict__ g_off, int n_dst,
                                    int g_nodes, int cap, int lead, int32_t *__restrict__ counts)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) counts[lead ? 0 : n_dst] = 0;
    if (i >= n_dst) return;
    const int node = dst[i];
    int c = 0;
    if ((unsigned)node < (unsigned)g_nodes) c = min(g_off[node + 1] - g_off[node], cap);
    counts[i + lead] = c;
}

// ---- symmetric-normalisation weights of a layer -----------------------------
__global__ void getweight_zero(int32_t *__restrict__ ins, int32_t *__restrict__ outs, int vtx)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < vtx) {
        ins[i] = 0;
        outs[i] = 0;
    }
}

// ins[dst[i]] += size of column i (integer atomics: the sum does not depend on the order)
__global__ void getweight_in_degrees(const int32_t *__restrict__ dst, const int32_t *__restrict__ off, int n_dst,
                                     int vtx, int32_t *__restrict__ ins)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_dst) return;
    const int node = dst[i];
    const int size = off[i + 1] - off[i];
    if ((unsigned)node < (unsigned)vtx && size > 0) atomicAdd(&ins[node], size);
}

// outs[row[j]] += 1 for every entry below off[n_dst]
__global__ void getweight_out_degrees(const int32_t *__restrict__ row, const int32_t *__restrict__ off, int n_dst,
                                      int64_t E, int vtx, int32_t *__restrict__ outs)
{
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t covered = min((int64_t)max(off[n_dst], 0), E);
    if (j >= covered) return;
    const int src = row[j];
    if ((unsigned)src < (unsigned)vtx) atomicAdd(&outs[src], 1);
}

// w[j] = 1 / (sqrtf(outs[row[j]]) * sqrtf(ins[dst[column of j]])); the column of an entry is
// found by a search in the offsets, so a column of any size is spread over many lanes.
__global__ void getweight_weights(const int32_t *__restrict__ dst, const int32_t *__restrict__ off,
                                  const int32_t *__restrict__ row, int n_dst, int64_t E, int vtx,
                                  const int32_t *__restrict__ ins, const int32_t *__restrict__ outs,
                                  float *__restrict__ w)
{
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= E) return;
    const int64_t covered = min((int64_t)max(off[n_dst], 0), E);
    float r = 0.0f;
    if (j < covered) {
        int lo = 0, hi = n_dst;              // last column i with off[i] <= j
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if ((int64_t)off[mid] <= j) lo = mid; else hi = mid;
        }
        const int node = dst[lo];
        const int src = row[j];
        if ((unsigned)node < (unsigned)vtx && (unsigned)src < (unsigned)vtx)
            r = 1.0f / (sqrtf((float)outs[src]) * sqrtf((float)ins[node]));      // correctly rounded sqrt and divide
    }
    w[j] = r;
}

}  // namespace jg

using namespace jg;

extern "C" __attribute__((visibility("default"))) int32_t jgamd_sample_neighbors(
    const int32_t *dst, const int32_t *layer_off, const int32_t *g_off, const int32_t *g_idx, int32_t n_dst,
    int32_t g_nodes, int32_t fanout, int64_t out_len, uint64_t seed, int32_t *out, void *stream)
{
    if (n_dst < 0 || g_nodes < 0 || out_len < 0) return fail(JGAMD_ERR_SIZE, "sample_neighbors: negative size");
    if (fanout > 1024) return fail(JGAMD_ERR_UNSUPPORTED, "sample_neighbors: fanout %d above 1024", fanout);
    if (n_dst == 0 || out_len == 0) return 0;
    if (!dst || !layer_off || !g_off || !g_idx || !out) return fail(JGAMD_ERR_NULL, "sample_neighbors: NULL array");
    hipLaunchKernelGGL(sample_neighbors_k, dim3((unsigned)ceil_div(n_dst, 128)), dim3(128), 0,
                       static_cast<hipStream_t>(stream), dst, layer_off, g_off, g_idx, n_dst, g_nodes, fanout, out_len,
                       seed, out);
    return launch_status("sample_neighbors");
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_layer_column_counts(
    const int32_t *dst, const int32_t *g_off, int32_t n_dst, int32_t g_nodes, int32_t cap, int32_t *counts,
    void *stream)
{
    if (n_dst < 0 || g_nodes < 0) return fail(JGAMD_ERR_SIZE, "layer_column_counts: negative size");
    if (!counts || (n_dst > 0 && (!dst || !g_off))) return fail(JGAMD_ERR_NULL, "layer_column_counts: NULL array");
    hipLaunchKernelGGL(layer_column_counts, dim3((unsigned)ceil_div(n_dst + 1, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), dst, g_off, n_dst, g_nodes, cap, 1, counts);
    return launch_status("layer_column_counts");
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_layer_column_offsets_workspace(int32_t n_dst,
                                                                                               size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "layer_column_offsets_workspace: NULL result");
    if (n_dst < 0) return fail(JGAMD_ERR_SIZE, "layer_column_offsets_workspace: negative size");
    *bytes = carve_bytes((size_t)n_dst + 1, sizeof(int32_t)) + carve_bytes(scan_ws_ints((int64_t)n_dst + 1), sizeof(int32_t));
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_layer_column_offsets(
    const int32_t *dst, const int32_t *g_off, int32_t n_dst, int32_t g_nodes, int32_t cap, int32_t *offsets, void *ws,
    size_t ws_bytes, void *stream)
{
    size_t need = 0;
    if (int32_t rc = jgamd_layer_column_offsets_workspace(n_dst, &need)) return rc;
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "layer_column_offsets: workspace of %zu bytes needed", need);
    if (n_dst > 0 && (!dst || !g_off)) return fail(JGAMD_ERR_NULL, "layer_column_offsets: NULL array");
    if (!offsets) return fail(JGAMD_ERR_NULL, "layer_column_offsets: NULL result");
    Carver c{static_cast<char *>(ws)};
    int32_t *counts = c.take<int32_t>((size_t)n_dst + 1);
    int32_t *sums = c.take<int32_t>(scan_ws_ints((int64_t)n_dst + 1));
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(layer_column_counts, dim3((unsigned)ceil_div(n_dst + 1, 256)), dim3(256), 0, s, dst, g_off, n_dst,
                       g_nodes, cap, 0, counts);
    return exclusive_scan_i32(counts, offsets, (int64_t)n_dst + 1, sums, s);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_getweight_workspace(int32_t vtx_size, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "getweight_workspace: NULL result");
    if (vtx_size < 0) return fail(JGAMD_ERR_SIZE, "getweight_workspace: negative size");
    *bytes = 2 * carve_bytes((size_t)vtx_size, sizeof(int32_t));
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_getweight(
    const int32_t *dst, const int32_t *off, const int32_t *row, int32_t n_dst, int32_t vtx_size, int64_t E, float *w,
    void *ws, size_t ws_bytes, void *stream)
{
    if (n_dst < 0 || vtx_size < 0 || E < 0) return fail(JGAMD_ERR_SIZE, "getweight: negative size");
    if (E >= (int64_t)1 << 31) return fail(JGAMD_ERR_SIZE, "getweight: E above 2^31-1");
    if (E == 0) return 0;
    if (!dst || !off || !row || !w) return fail(JGAMD_ERR_NULL, "getweight: NULL array");
    size_t need = 0;
    if (int32_t rc = jgamd_getweight_workspace(vtx_size, &need)) return rc;
    if (need && (!ws || ws_bytes < need)) return fail(JGAMD_ERR_WORKSPACE, "getweight: workspace of %zu bytes needed", need);
    hipStream_t s = static_cast<hipStream_t>(stream);
    Carver c{static_cast<char *>(ws)};
    int32_t *ins = c.take<int32_t>((size_t)vtx_size);
    int32_t *outs = c.take<int32_t>((size_t)vtx_size);
    const unsigned eb = (unsigned)ceil_div(E, (int64_t)256);
    if (vtx_size > 0)
        hipLaunchKernelGGL(getweight_zero, dim3((unsigned)ceil_div(vtx_size, 256)), dim3(256), 0, s, ins, outs, vtx_size);
    if (n_dst > 0)
        hipLaunchKernelGGL(getweight_in_degrees, dim3((unsigned)ceil_div(n_dst, 256)), dim3(256), 0, s, dst, off, n_dst,
                           vtx_size, ins);
    hipLaunchKernelGGL(getweight_out_degrees, dim3(eb), dim3(256), 0, s, row, off, n_dst, E, vtx_size, outs);
    hipLaunchKernelGGL(getweight_weights, dim3(eb), dim3(256), 0, s, dst, off, row, n_dst, E, vtx_size, ins, outs, w);
    return launch_status("getweight");
}
