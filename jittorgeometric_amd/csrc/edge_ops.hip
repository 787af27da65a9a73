// Per-edge operators over the CSC arrays: edge softmax forward/backward and
// the vertex -> edge copy.
//
// Edge softmax: the values of one destination column are contiguous
// ([off[c]*H, off[c+1]*H) in an [E,H] array).  A group of G lanes (G a power
// of two, H | G) owns one column; lane l of the group always sees head l % H,
// so the three passes (max, sum of exp, normalise) need only xor-shuffles
// between lanes H, 2H, ... apart.  G is picked from the mean column length so
// that short columns do not idle a whole wavefront.
#include "common.h"

namespace jg {

constexpr int kEdgeThreads = 256;

template <int G, typename Op> __device__ __forceinline__ float group_reduce(float v, int H, Op op)
{
    for (int o = H; o < G; o <<= 1) v = op(v, __shfl_xor(v, o, kWave));
    return v;
}

// x -> y = exp(x - max) / sum exp(x - max) per (column, head);
// ops/cpp/edgesoftmax_op.cc:48-65 with the three loops kept as three passes.
template <int G>
__global__ __launch_bounds__(kEdgeThreads) void edge_softmax_fwd_k(const int32_t *__restrict__ off,
                                                                   const float *__restrict__ x, float *__restrict__ y,
                                                                   int V, int H)
{
    const int gl = threadIdx.x % G;
    const int64_t ngroups = (int64_t)gridDim.x * (kEdgeThreads / G);
    for (int64_t c = (int64_t)blockIdx.x * (kEdgeThreads / G) + threadIdx.x / G; c < V; c += ngroups) {
        const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
        float m = -INFINITY;
        for (int64_t p = s + gl; p < e; p += G) m = fmaxf(m, x[p]);
        m = group_reduce<G>(m, H, [](float a, float b) { return fmaxf(a, b); });
        float t = 0.f;
        for (int64_t p = s + gl; p < e; p += G) t += expf(x[p] - m);
        t = group_reduce<G>(t, H, [](float a, float b) { return a + b; });
        for (int64_t p = s + gl; p < e; p += G) y[p] = expf(x[p] - m) / t;
    }
}

// dx = y*g - y*sum(y*g) per (column, head); ops/cpp/edgesoftmaxbackward_op.cc:45-51.
template <int G>
__global__ __launch_bounds__(kEdgeThreads) void edge_softmax_bwd_k(const int32_t *__restrict__ off,
                                                                   const float *__restrict__ y,
                                                                   const float *__restrict__ g, float *__restrict__ dx,
                                                                   int V, int H)
{
    const int gl = threadIdx.x % G;
    const int64_t ngroups = (int64_t)gridDim.x * (kEdgeThreads / G);
    for (int64_t c = (int64_t)blockIdx.x * (kEdgeThreads / G) + threadIdx.x / G; c < V; c += ngroups) {
        const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
        float dot = 0.f;
        for (int64_t p = s + gl; p < e; p += G) dot += y[p] * g[p];
        dot = group_reduce<G>(dot, H, [](float a, float b) { return a + b; });
        for (int64_t p = s + gl; p < e; p += G) dx[p] = y[p] * g[p] - y[p] * dot;
    }
}

// Any H (not a power of two, or above 64): one thread per (column, head).
__global__ void edge_softmax_fwd_any(const int32_t *__restrict__ off, const float *__restrict__ x,
                                     float *__restrict__ y, int V, int H)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)V * H) return;
    const int c = (int)(i / H), h = (int)(i % H);
    const int s = off[c], e = off[c + 1];
    float m = -INFINITY;
    for (int j = s; j < e; j++) m = fmaxf(m, x[(int64_t)j * H + h]);
    float t = 0.f;
    for (int j = s; j < e; j++) t += expf(x[(int64_t)j * H + h] - m);
    for (int j = s; j < e; j++) y[(int64_t)j * H + h] = expf(x[(int64_t)j * H + h] - m) / t;
}

__global__ void edge_softmax_bwd_any(const int32_t *__restrict__ off, const float *__restrict__ y,
                                     const float *__restrict__ g, float *__restrict__ dx, int V, int H)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)V * H) return;
    const int c = (int)(i / H), h = (int)(i % H);
    const int s = off[c], e = off[c + 1];
    float dot = 0.f;
    for (int j = s; j < e; j++) dot += y[(int64_t)j * H + h] * g[(int64_t)j * H + h];
    for (int j = s; j < e; j++) {
        const int64_t p = (int64_t)j * H + h;
        dx[p] = y[p] * g[p] - y[p] * dot;
    }
}

// out[e,:] = x[idx[e],:]  (flag 0)   or   x[column of e,:]  (flag 1).
// Each wavefront takes 64 consecutive edges; for flag 1 every lane finds the
// column of its own edge by binary search in off, then the rows are copied
// one edge at a time with the row index broadcast from its lane.
__global__ __launch_bounds__(kEdgeThreads) void scatter_to_edge_k(const int32_t *__restrict__ off,
                                                                  const int32_t *__restrict__ idx,
                                                                  const float *__restrict__ x, float *__restrict__ out,
                                                                  int V, int64_t E, int F, int flag)
{
    const int64_t e0 = ((int64_t)blockIdx.x * (kEdgeThreads / kWave) + wave_in_block()) * kWave;
    if (e0 >= E) return;
    const int lane = lane_id();
    const int64_t me = e0 + lane;
    int node = 0;
    if (me < E) {
        if (flag == 0) {
            node = idx[me];
        } else {
            // largest c with off[c] <= me
            int lo = 0, hi = V;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if ((int64_t)off[mid] <= me) lo = mid; else hi = mid;
            }
            node = lo;
        }
        if ((unsigned)node >= (unsigned)V) node = -1;
    }
    const int n = (int)min((int64_t)kWave, E - e0);
    for (int i = 0; i < n; i++) {
        const int c = bcast_i(node, i);
        float *dst = out + (e0 + i) * F;
        if (c < 0) {
            for (int f = lane; f < F; f += kWave) dst[f] = 0.f;
        } else {
            const float *src = x + (int64_t)c * F;
            for (int f = lane; f < F; f += kWave) dst[f] = src[f];
        }
    }
}

static int pick_group(int64_t E, int V, int H)
{
    const int64_t mean = V > 0 ? (E * H) / V : 0;   // values per column
    int g = mean <= 8 ? 4 : mean <= 32 ? 8 : mean <= 128 ? 16 : mean <= 512 ? 32 : 64;
    return g < H ? H : g;
}

static bool pow2_upto64(int H) { return H >= 1 && H <= 64 && (H & (H - 1)) == 0; }

}  // namespace jg

using namespace jg;

#define JG_EXPORT extern "C" __attribute__((visibility("default")))

static int32_t check_softmax(const char *who, const void *off, const void *a, const void *b, int32_t V, int64_t E,
                             int32_t H)
{
    if (V < 0 || E < 0 || H < 1) return fail(JGAMD_ERR_SIZE, "%s: bad size (V=%d, E=%lld, H=%d)", who, V, (long long)E, H);
    if (E >= ((int64_t)1 << 31)) return fail(JGAMD_ERR_SIZE, "%s: E does not fit int32 offsets", who);
    if (!off) return fail(JGAMD_ERR_NULL, "%s: off is NULL", who);
    if (E > 0 && (!a || !b)) return fail(JGAMD_ERR_NULL, "%s: NULL array with E > 0", who);
    return 0;
}

template <typename K, typename... A> static void launch_groups(K k, int G, int V, hipStream_t s, A... a)
{
    const int per_block = kEdgeThreads / G;
    int64_t blocks = ceil_div(V, per_block);
    if (blocks > 65536 * 8) blocks = 65536 * 8;
    hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(kEdgeThreads), 0, s, a...);
}

JG_EXPORT int32_t jgamd_edge_softmax_fwd(const int32_t *off, const float *x, float *y, int32_t V, int64_t E,
                                         int32_t H, void *stream)
{
    if (int32_t rc = check_softmax("edge_softmax_fwd", off, x, y, V, E, H)) return rc;
    if (V == 0 || E == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!pow2_upto64(H)) {
        hipLaunchKernelGGL(edge_softmax_fwd_any, dim3((unsigned)ceil_div((int64_t)V * H, 256)), dim3(256), 0, s, off, x,
                           y, V, H);
        return launch_status("edge_softmax_fwd");
    }
    switch (pick_group(E, V, H)) {
    case 1: case 2: case 4: launch_groups(edge_softmax_fwd_k<4>, 4, V, s, off, x, y, V, H); break;
    case 8: launch_groups(edge_softmax_fwd_k<8>, 8, V, s, off, x, y, V, H); break;
    case 16: launch_groups(edge_softmax_fwd_k<16>, 16, V, s, off, x, y, V, H); break;
    case 32: launch_groups(edge_softmax_fwd_k<32>, 32, V, s, off, x, y, V, H); break;
    default: launch_groups(edge_softmax_fwd_k<64>, 64, V, s, off, x, y, V, H); break;
    }
    return launch_status("edge_softmax_fwd");
}

JG_EXPORT int32_t jgamd_edge_softmax_bwd(const int32_t *off, const float *y, const float *g, float *dx, int32_t V,
                                         int64_t E, int32_t H, void *stream)
{
    if (int32_t rc = check_softmax("edge_softmax_bwd", off, y, dx, V, E, H)) return rc;
    if (E > 0 && !g) return fail(JGAMD_ERR_NULL, "edge_softmax_bwd: g is NULL");
    if (V == 0 || E == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!pow2_upto64(H)) {
        hipLaunchKernelGGL(edge_softmax_bwd_any, dim3((unsigned)ceil_div((int64_t)V * H, 256)), dim3(256), 0, s, off, y,
                           g, dx, V, H);
        return launch_status("edge_softmax_bwd");
    }
    switch (pick_group(E, V, H)) {
    case 1: case 2: case 4: launch_groups(edge_softmax_bwd_k<4>, 4, V, s, off, y, g, dx, V, H); break;
    case 8: launch_groups(edge_softmax_bwd_k<8>, 8, V, s, off, y, g, dx, V, H); break;
    case 16: launch_groups(edge_softmax_bwd_k<16>, 16, V, s, off, y, g, dx, V, H); break;
    case 32: launch_groups(edge_softmax_bwd_k<32>, 32, V, s, off, y, g, dx, V, H); break;
    default: launch_groups(edge_softmax_bwd_k<64>, 64, V, s, off, y, g, dx, V, H); break;
    }
    return launch_status("edge_softmax_bwd");
}

JG_EXPORT int32_t jgamd_scatter_to_edge(const int32_t *off, const int32_t *idx, const float *x, float *out, int32_t V,
                                        int64_t E, int32_t F, int32_t flag, void *stream)
{
    if (V < 0 || E < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "scatter_to_edge: negative size");
    if (flag != 0 && flag != 1) return fail(JGAMD_ERR_SIZE, "scatter_to_edge: flag must be 0 or 1");
    if (E == 0 || F == 0) return 0;
    if (!x || !out) return fail(JGAMD_ERR_NULL, "scatter_to_edge: x/out is NULL");
    if (flag == 0 && !idx) return fail(JGAMD_ERR_NULL, "scatter_to_edge: idx is NULL for flag 0");
    if (flag == 1 && !off) return fail(JGAMD_ERR_NULL, "scatter_to_edge: off is NULL for flag 1");
    if (V == 0) return fail(JGAMD_ERR_SIZE, "scatter_to_edge: E > 0 with V = 0");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t waves = ceil_div(E, kWave);
    hipLaunchKernelGGL(scatter_to_edge_k, dim3((unsigned)ceil_div(waves, kEdgeThreads / kWave)), dim3(kEdgeThreads), 0,
                       s, off, idx, x, out, V, E, F, flag);
    return launch_status("scatter_to_edge");
}
