// Per-edge operators over the CSC arrays: edge softmax forward/backward and
// the vertex -> edge copy.
//
// Edge softmax: the values of one destination column are contiguous
// ([off[c]*H, off[c+1]*H) in an [E,H] array).  A group of G lanes (G a power
// of two, H | G) owns one column; lane l of the group always sees head l % H,
// so the three passes (max, sum of exp, normalise) need only xor-shuffles
// between lanes H, 2H, ... apart.  G is picked from the mean column length so
// that short columns do not idle a whole wavefront.  Columns longer than
// kLongColumn entries (hubs) are skipped by the group kernel, collected into a
// list, and each handled by a whole 1024-thread block with LDS reductions.
#include "common.h"

namespace jg {

constexpr int kEdgeThreads = 256;
constexpr int kLongColumn = 512;   // entries; longer columns get a block each
constexpr int kRegItems = 8;       // values per lane held in registers on the short-column path

template <int G, typename Op> __device__ __forceinline__ float group_reduce(float v, int H, Op op)
{
    for (int o = H; o < G; o <<= 1) v = op(v, __shfl_xor(v, o, kWave));
    return v;
}

// Walks positions first, first+G, ... below e, kRegItems at a time: the loads of a batch are
// issued together (index clamped, not predicated), then f(position, a[p], b[p]) runs on the
// positions inside the range.
template <int G, typename F>
__device__ __forceinline__ void group_walk(const float *__restrict__ a, const float *__restrict__ b, int64_t first,
                                           int64_t e, F f)
{
    for (int64_t p0 = first; p0 < e; p0 += (int64_t)kRegItems * G) {
        float va[kRegItems], vb[kRegItems];
#pragma unroll
        for (int i = 0; i < kRegItems; i++) {
            const int64_t p = min(p0 + (int64_t)i * G, e - 1);
            va[i] = a[p];
            vb[i] = b[p];
        }
#pragma unroll
        for (int i = 0; i < kRegItems; i++)
            if (p0 + (int64_t)i * G < e) f(p0 + (int64_t)i * G, va[i], vb[i]);
    }
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
        if (off[c + 1] - off[c] > kLongColumn) continue;   // left to the block-per-column kernel
        const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
        if (e <= s) continue;
        if (e - s <= (int64_t)kRegItems * G) {
            // the whole column fits in kRegItems values per lane: one trip to memory, all loads
            // issued together (index clamped, not predicated), the three passes run on registers
            float v[kRegItems];
#pragma unroll
            for (int i = 0; i < kRegItems; i++) v[i] = x[min(s + gl + (int64_t)i * G, e - 1)];
            float m = -INFINITY;
#pragma unroll
            for (int i = 0; i < kRegItems; i++)
                if (s + gl + (int64_t)i * G < e) m = fmaxf(m, v[i]);
            m = group_reduce<G>(m, H, [](float a, float b) { return fmaxf(a, b); });
            float t = 0.f;
#pragma unroll
            for (int i = 0; i < kRegItems; i++) {
                v[i] = expf(v[i] - m);
                if (s + gl + (int64_t)i * G < e) t += v[i];
            }
            t = group_reduce<G>(t, H, [](float a, float b) { return a + b; });
#pragma unroll
            for (int i = 0; i < kRegItems; i++)
                if (s + gl + (int64_t)i * G < e) y[s + gl + (int64_t)i * G] = v[i] / t;
            continue;
        }
        // longer columns: the same three passes, kRegItems loads in flight per lane
        float m = -INFINITY;
        group_walk<G>(x, x, s + gl, e, [&](int64_t, float v, float) { m = fmaxf(m, v); });
        m = group_reduce<G>(m, H, [](float a, float b) { return fmaxf(a, b); });
        float t = 0.f;
        group_walk<G>(x, x, s + gl, e, [&](int64_t, float v, float) { t += expf(v - m); });
        t = group_reduce<G>(t, H, [](float a, float b) { return a + b; });
        group_walk<G>(x, x, s + gl, e, [&](int64_t p, float v, float) { y[p] = expf(v - m) / t; });
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
        if (off[c + 1] - off[c] > kLongColumn) continue;
        const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
        if (e <= s) continue;
        if (e - s <= (int64_t)kRegItems * G) {
            float yv[kRegItems], gv[kRegItems];
#pragma unroll
            for (int i = 0; i < kRegItems; i++) {
                const int64_t p = min(s + gl + (int64_t)i * G, e - 1);
                yv[i] = y[p];
                gv[i] = g[p];
            }
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < kRegItems; i++)
                if (s + gl + (int64_t)i * G < e) dot += yv[i] * gv[i];
            dot = group_reduce<G>(dot, H, [](float a, float b) { return a + b; });
#pragma unroll
            for (int i = 0; i < kRegItems; i++)
                if (s + gl + (int64_t)i * G < e) dx[s + gl + (int64_t)i * G] = yv[i] * gv[i] - yv[i] * dot;
            continue;
        }
        float dot = 0.f;
        group_walk<G>(y, g, s + gl, e, [&](int64_t, float yv, float gv) { dot += yv * gv; });
        dot = group_reduce<G>(dot, H, [](float a, float b) { return a + b; });
        group_walk<G>(y, g, s + gl, e, [&](int64_t p, float yv, float gv) { dx[p] = yv * gv - yv * dot; });
    }
}

// ---- hub columns ------------------------------------------------------------
__global__ void edge_zero_counter(int32_t *counter) { *counter = 0; }

// list[0..*counter) = columns with more than kLongColumn entries (any order:
// each is processed independently).
__global__ void edge_list_long(const int32_t *__restrict__ off, int V, int32_t *__restrict__ counter,
                               int32_t *__restrict__ list, int capacity)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= V) return;
    if (off[c + 1] - off[c] > kLongColumn) {
        const int slot = atomicAdd(counter, 1);
        if (slot < capacity) list[slot] = c;
    }
}

// Per-head reduction over the block: thread t holds head t % H (kLongThreads % H == 0),
// so folding halves of at least H keeps heads apart.  Result for head h in red[h].
constexpr int kLongThreads = 1024;
constexpr int kLongBatch = 8;      // values per thread fetched together

template <typename Op> __device__ __forceinline__ float block_head_reduce(float v, int H, float *red, Op op)
{
    __syncthreads();
    red[threadIdx.x] = v;
    __syncthreads();
    for (int o = kLongThreads / 2; o >= H; o >>= 1) {
        if ((int)threadIdx.x < o) red[threadIdx.x] = op(red[threadIdx.x], red[threadIdx.x + o]);
        __syncthreads();
    }
    return red[threadIdx.x % H];
}

// Walks this thread's values of [s,e) (stride kLongThreads) kLongBatch at a time: the loads of a
// batch are issued together (index clamped, not predicated), then `f(position, value...)` runs on
// the ones inside the range.
template <typename F> __device__ __forceinline__ void long_walk1(const float *__restrict__ a, int64_t s, int64_t e, F f)
{
    for (int64_t p0 = s + threadIdx.x; p0 < e; p0 += (int64_t)kLongBatch * kLongThreads) {
        float v[kLongBatch];
#pragma unroll
        for (int i = 0; i < kLongBatch; i++) v[i] = a[min(p0 + (int64_t)i * kLongThreads, e - 1)];
#pragma unroll
        for (int i = 0; i < kLongBatch; i++)
            if (p0 + (int64_t)i * kLongThreads < e) f(p0 + (int64_t)i * kLongThreads, v[i]);
    }
}
template <typename F>
__device__ __forceinline__ void long_walk2(const float *__restrict__ a, const float *__restrict__ b, int64_t s,
                                           int64_t e, F f)
{
    for (int64_t p0 = s + threadIdx.x; p0 < e; p0 += (int64_t)kLongBatch * kLongThreads) {
        float va[kLongBatch], vb[kLongBatch];
#pragma unroll
        for (int i = 0; i < kLongBatch; i++) {
            const int64_t p = min(p0 + (int64_t)i * kLongThreads, e - 1);
            va[i] = a[p];
            vb[i] = b[p];
        }
#pragma unroll
        for (int i = 0; i < kLongBatch; i++)
            if (p0 + (int64_t)i * kLongThreads < e) f(p0 + (int64_t)i * kLongThreads, va[i], vb[i]);
    }
}

__global__ __launch_bounds__(kLongThreads) void edge_softmax_fwd_long(const int32_t *__restrict__ off,
                                                                      const float *__restrict__ x,
                                                                      float *__restrict__ y, int H,
                                                                      const int32_t *__restrict__ counter,
                                                                      const int32_t *__restrict__ list)
{
    __shared__ float red[kLongThreads];
    if ((int)blockIdx.x >= *counter) return;
    const int c = list[blockIdx.x];
    const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
    float m = -INFINITY;
    long_walk1(x, s, e, [&](int64_t, float v) { m = fmaxf(m, v); });
    m = block_head_reduce(m, H, red, [](float a, float b) { return fmaxf(a, b); });
    float t = 0.f;
    long_walk1(x, s, e, [&](int64_t, float v) { t += expf(v - m); });
    t = block_head_reduce(t, H, red, [](float a, float b) { return a + b; });
    long_walk1(x, s, e, [&](int64_t p, float v) { y[p] = expf(v - m) / t; });
}

__global__ __launch_bounds__(kLongThreads) void edge_softmax_bwd_long(const int32_t *__restrict__ off,
                                                                      const float *__restrict__ y,
                                                                      const float *__restrict__ g,
                                                                      float *__restrict__ dx, int H,
                                                                      const int32_t *__restrict__ counter,
                                                                      const int32_t *__restrict__ list)
{
    __shared__ float red[kLongThreads];
    if ((int)blockIdx.x >= *counter) return;
    const int c = list[blockIdx.x];
    const int64_t s = (int64_t)off[c] * H, e = (int64_t)off[c + 1] * H;
    float dot = 0.f;
    long_walk2(y, g, s, e, [&](int64_t, float yv, float gv) { dot += yv * gv; });
    dot = block_head_reduce(dot, H, red, [](float a, float b) { return a + b; });
    long_walk2(y, g, s, e, [&](int64_t p, float yv, float gv) { dx[p] = yv * gv - yv * dot; });
}

// Any H (not a power of two, or above 64): one thread per (column, head).  The thread adds a
// column's terms one after the other, as the reference's loop does, but in double: a column of
// 10^4 entries would otherwise be 10^4 roundings away from the sum the tile kernels compute.
__global__ void edge_softmax_fwd_any(const int32_t *__restrict__ off, const float *__restrict__ x,
                                     float *__restrict__ y, int V, int H)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)V * H) return;
    const int c = (int)(i / H), h = (int)(i % H);
    const int s = off[c], e = off[c + 1];
    float m = -INFINITY;
    for (int j = s; j < e; j++) m = fmaxf(m, x[(int64_t)j * H + h]);
    double sum = 0.0;
    for (int j = s; j < e; j++) sum += (double)expf(x[(int64_t)j * H + h] - m);
    const float t = (float)sum;
    for (int j = s; j < e; j++) y[(int64_t)j * H + h] = expf(x[(int64_t)j * H + h] - m) / t;
}

__global__ void edge_softmax_bwd_any(const int32_t *__restrict__ off, const float *__restrict__ y,
                                     const float *__restrict__ g, float *__restrict__ dx, int V, int H)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)V * H) return;
    const int c = (int)(i / H), h = (int)(i % H);
    const int s = off[c], e = off[c + 1];
    double sum = 0.0;
    for (int j = s; j < e; j++) sum += (double)y[(int64_t)j * H + h] * (double)g[(int64_t)j * H + h];
    const float dot = (float)sum;
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

// Scratch of the hub-column path: a counter and the list of long columns
// (at most E / kLongColumn of them).
static int long_capacity(int32_t V, int64_t E)
{
    const int64_t c = E / kLongColumn + 1;
    return (int)(c < (int64_t)V ? c : (int64_t)V);
}
static size_t group_ws_bytes(int32_t V, int64_t E) { return 256 + carve_bytes((size_t)long_capacity(V, E), 4); }
static size_t softmax_ws_bytes(int32_t V, int64_t E) { return group_ws_bytes(V, E) + entry_tiles_ws_bytes(E); }
// JGAMD_SOFTMAX=groups keeps the lane-group-per-column kernels for 1-8 heads too
static bool use_flat(int H)
{
    const char *e = getenv("JGAMD_SOFTMAX");
    return edge_softmax_flat_supported(H) && !(e && strcmp(e, "groups") == 0);
}

static int32_t check_softmax_ws(const char *who, const void *ws, size_t have, int32_t V, int64_t E)
{
    const size_t need = softmax_ws_bytes(V, E);
    if (!ws || have < need) return fail(JGAMD_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws ? have : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "%s: workspace not 256-byte aligned", who);
    return 0;
}

JG_EXPORT int32_t jgamd_edge_softmax_workspace(int32_t V, int64_t E, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "edge_softmax_workspace: bytes is NULL");
    if (V < 0 || E < 0) return fail(JGAMD_ERR_SIZE, "edge_softmax_workspace: negative size");
    *bytes = (V == 0 || E == 0) ? 0 : softmax_ws_bytes(V, E);
    return 0;
}

// Fills list/counter with the hub columns; returns the launch bound for the block-per-column kernel.
static int list_long_columns(const int32_t *off, int32_t V, int64_t E, void *ws, int32_t **counter, int32_t **list,
                             hipStream_t s)
{
    Carver carve(ws);
    *counter = carve.take<int32_t>(1);
    const int cap = long_capacity(V, E);
    *list = carve.take<int32_t>((size_t)cap);
    hipLaunchKernelGGL(edge_zero_counter, dim3(1), dim3(1), 0, s, *counter);
    hipLaunchKernelGGL(edge_list_long, dim3((unsigned)ceil_div(V, 256)), dim3(256), 0, s, off, V, *counter, *list, cap);
    return cap;
}

// tiles: the tile plan of `off` (jgamd_csx_plan, JGAMD_PLAN_TILES) or NULL
static int32_t softmax_fwd(const void *tiles, const int32_t *off, const float *x, float *y, int32_t V, int64_t E,
                           int32_t H, void *ws, size_t ws_bytes, void *stream)
{
    if (int32_t rc = check_softmax("edge_softmax_fwd", off, x, y, V, E, H)) return rc;
    if (V == 0 || E == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!pow2_upto64(H)) {
        hipLaunchKernelGGL(edge_softmax_fwd_any, dim3((unsigned)ceil_div((int64_t)V * H, 256)), dim3(256), 0, s, off, x,
                           y, V, H);
        return launch_status("edge_softmax_fwd");
    }
    if (int32_t rc = check_softmax_ws("edge_softmax_fwd", ws, ws_bytes, V, E)) return rc;
    if (use_flat(H)) {
        edge_softmax_flat_enqueue(true, off, x, nullptr, y, V, E, H, static_cast<char *>(ws) + group_ws_bytes(V, E), s,
                                  tiles);
        return launch_status("edge_softmax_fwd");
    }
    switch (pick_group(E, V, H)) {
    case 1: case 2: case 4: launch_groups(edge_softmax_fwd_k<4>, 4, V, s, off, x, y, V, H); break;
    case 8: launch_groups(edge_softmax_fwd_k<8>, 8, V, s, off, x, y, V, H); break;
    case 16: launch_groups(edge_softmax_fwd_k<16>, 16, V, s, off, x, y, V, H); break;
    case 32: launch_groups(edge_softmax_fwd_k<32>, 32, V, s, off, x, y, V, H); break;
    default: launch_groups(edge_softmax_fwd_k<64>, 64, V, s, off, x, y, V, H); break;
    }
    int32_t *counter, *list;
    const int cap = list_long_columns(off, V, E, ws, &counter, &list, s);
    hipLaunchKernelGGL(edge_softmax_fwd_long, dim3((unsigned)cap), dim3(kLongThreads), 0, s, off, x, y, H, counter, list);
    return launch_status("edge_softmax_fwd");
}

JG_EXPORT int32_t jgamd_edge_softmax_fwd(const int32_t *off, const float *x, float *y, int32_t V, int64_t E,
                                         int32_t H, void *ws, size_t ws_bytes, void *stream)
{
    return softmax_fwd(nullptr, off, x, y, V, E, H, ws, ws_bytes, stream);
}

static int32_t check_tiles(const char *who, const void *tiles)
{
    if (!tiles) return fail(JGAMD_ERR_NULL, "%s: tiles is NULL", who);
    if (((uintptr_t)tiles & 255) != 0) return fail(JGAMD_ERR_ALIGN, "%s: tiles not 256-byte aligned", who);
    return 0;
}

JG_EXPORT int32_t jgamd_edge_softmax_fwd_planned(const void *tiles, const int32_t *off, const float *x, float *y,
                                                 int32_t V, int64_t E, int32_t H, void *ws, size_t ws_bytes,
                                                 void *stream)
{
    if (int32_t rc = check_tiles("edge_softmax_fwd_planned", tiles)) return rc;
    return softmax_fwd(tiles, off, x, y, V, E, H, ws, ws_bytes, stream);
}

static int32_t softmax_bwd(const void *tiles, const int32_t *off, const float *y, const float *g, float *dx, int32_t V,
                           int64_t E, int32_t H, void *ws, size_t ws_bytes, void *stream)
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
    if (int32_t rc = check_softmax_ws("edge_softmax_bwd", ws, ws_bytes, V, E)) return rc;
    if (use_flat(H)) {
        edge_softmax_flat_enqueue(false, off, y, g, dx, V, E, H, static_cast<char *>(ws) + group_ws_bytes(V, E), s,
                                  tiles);
        return launch_status("edge_softmax_bwd");
    }
    switch (pick_group(E, V, H)) {
    case 1: case 2: case 4: launch_groups(edge_softmax_bwd_k<4>, 4, V, s, off, y, g, dx, V, H); break;
    case 8: launch_groups(edge_softmax_bwd_k<8>, 8, V, s, off, y, g, dx, V, H); break;
    case 16: launch_groups(edge_softmax_bwd_k<16>, 16, V, s, off, y, g, dx, V, H); break;
    case 32: launch_groups(edge_softmax_bwd_k<32>, 32, V, s, off, y, g, dx, V, H); break;
    default: launch_groups(edge_softmax_bwd_k<64>, 64, V, s, off, y, g, dx, V, H); break;
    }
    int32_t *counter, *list;
    const int cap = list_long_columns(off, V, E, ws, &counter, &list, s);
    hipLaunchKernelGGL(edge_softmax_bwd_long, dim3((unsigned)cap), dim3(kLongThreads), 0, s, off, y, g, dx, H, counter,
                       list);
    return launch_status("edge_softmax_bwd");
}

JG_EXPORT int32_t jgamd_edge_softmax_bwd(const int32_t *off, const float *y, const float *g, float *dx, int32_t V,
                                         int64_t E, int32_t H, void *ws, size_t ws_bytes, void *stream)
{
    return softmax_bwd(nullptr, off, y, g, dx, V, E, H, ws, ws_bytes, stream);
}

JG_EXPORT int32_t jgamd_edge_softmax_bwd_planned(const void *tiles, const int32_t *off, const float *y, const float *g,
                                                 float *dx, int32_t V, int64_t E, int32_t H, void *ws,
                                                 size_t ws_bytes, void *stream)
{
    if (int32_t rc = check_tiles("edge_softmax_bwd_planned", tiles)) return rc;
    return softmax_bwd(tiles, off, y, g, dx, V, E, H, ws, ws_bytes, stream);
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
