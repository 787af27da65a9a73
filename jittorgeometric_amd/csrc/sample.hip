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
