// Mean cross-entropy of row-major logits [V,C] against integer labels, and its gradient: the
// loss at the end of the full-graph training step (nn.cross_entropy_loss(pred, label) in
// examples/gcn_example.py:113; nn.log_softmax + nn.nll_loss in examples/sage_example.py:69,83).
//
//     lse[i]  = max_c x[i,c] + log sum_c exp(x[i,c] - max_c x[i,c])
//     loss    = mean over the rows with a label in [0,C) of (lse[i] - x[i, label[i]])
//     grad    = g / count * (exp(x[i,c] - lse[i]) - [c == label[i]])      (0 for the other rows)
//
// With millions of rows and a few dozen classes a row is shorter than a wavefront: G lanes
// (a power of two, about C / 4) share a row, so that consecutive lanes read consecutive floats
// of consecutive rows, and the row's maximum and sum fold with xor-shuffles inside the group.
// The mean is reduced in two fixed-order stages (per-block partial sums in double, then one
// block), so the result does not change from run to run.
//
// The gradient's probabilities are exp(x - lse) with lse kept as one float per row, so they
// carry lse's rounding: a relative error of about ulp(lse) / 2, which is 5e-7 while |lse| stays
// under 8 and reaches 8e-6 at |lse| near 170 (logits scaled far beyond what a trained classifier
// produces).
#include <math.h>

#include "common.h"

namespace jg {

constexpr int kCeThreads = 256;
constexpr int kCeRows = 2048;      // rows per block, at most
constexpr int kCeMinRows = 32;     // and at least (one pass of the narrowest lane group)

// Rows per block: as many as keep the per-block partial sums few, but never so many that a small
// matrix leaves most of the 256 compute units without a block (2,708 rows of 7 classes at 2048
// rows per block were two blocks and 56 us; at 32 rows per block 85 blocks and a few us).
static int ce_rows_per_block(int64_t V)
{
    int rows = kCeRows;
    while (rows > kCeMinRows && V / rows < 1024) rows >>= 1;
    return rows;
}

__device__ __forceinline__ int64_t label_at(const int32_t *y32, const int64_t *y64, int64_t row)
{
    return y64 ? y64[row] : (int64_t)y32[row];
}

// REG: the row fits four floats per lane (C <= 4 G); a group of lanes then takes kCeUnroll rows per
// pass, all loads first, so that enough bytes are in flight.  Otherwise the row is read twice.
constexpr int kCeUnroll = 4;

template <int G, bool REG>
__global__ __launch_bounds__(kCeThreads) void ce_rows(const float *__restrict__ x, const int32_t *__restrict__ y32,
                                                      const int64_t *__restrict__ y64, int64_t V, int C,
                                                      int rows_per_block, int log_probs,
                                                      float *__restrict__ lse_out,
                                                      double *__restrict__ block_sum, int32_t *__restrict__ block_cnt)
{
    constexpr int RP = kCeThreads / G;      // row groups per pass
    __shared__ double s_sum[RP];
    __shared__ int s_cnt[RP];
    const int g = threadIdx.x % G, lr = threadIdx.x / G;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < V ? r0 + rows_per_block : V;
    double acc = 0.0;
    int cnt = 0;
    auto finish = [&](int64_t row, const float *p, float m, float s) {
        // rows of log-probabilities (nll_loss): the loss is -row[label] and the gradient has no
        // softmax term, which an infinite lse switches off in the backward kernels (exp(-inf) = 0)
        const float l = log_probs ? 0.f : m + logf(s);
        lse_out[row] = log_probs ? INFINITY : l;
        const int64_t lab = label_at(y32, y64, row);
        if (lab >= 0 && lab < C) {
            acc += (double)(l - p[lab]);
            cnt++;
        }
    };
    if (REG) {
        for (int64_t rb = r0; rb < r1; rb += RP * kCeUnroll) {
            float v[kCeUnroll][4];
            const float *p[kCeUnroll];
#pragma unroll
            for (int u = 0; u < kCeUnroll; u++) {
                const int64_t row = rb + u * RP + lr;
                p[u] = x + (row < r1 ? row : r1 - 1) * (int64_t)C;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int c = g + i * G;
                    v[u][i] = p[u][c < C ? c : 0];
                }
            }
#pragma unroll
            for (int u = 0; u < kCeUnroll; u++) {
                float m = -INFINITY, s = 0.f;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (g + i * G < C) m = fmaxf(m, v[u][i]);
#pragma unroll
                for (int o = G / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, G));
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (g + i * G < C) s += expf(v[u][i] - m);
#pragma unroll
                for (int o = G / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, G);
                const int64_t row = rb + u * RP + lr;
                if (g == 0 && row < r1) finish(row, p[u], m, s);
            }
        }
    } else {
        for (int64_t rb = r0; rb < r1; rb += RP) {
            const int64_t row = rb + lr;
            const bool ok = row < r1;
            const float *p = x + (ok ? row : r1 - 1) * (int64_t)C;
            float m = -INFINITY, s = 0.f;
            for (int c = g; c < C; c += G) m = fmaxf(m, p[c]);
#pragma unroll
            for (int o = G / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, G));
            for (int c = g; c < C; c += G) s += expf(p[c] - m);
#pragma unroll
            for (int o = G / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, G);
            if (g == 0 && ok) finish(row, p, m, s);
        }
    }
    if (g == 0) {
        s_sum[lr] = acc;
        s_cnt[lr] = cnt;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        int n = 0;
        for (int i = 0; i < RP; i++) {
            t += s_sum[i];
            n += s_cnt[i];
        }
        block_sum[blockIdx.x] = t;
        block_cnt[blockIdx.x] = n;
    }
}

// loss[0] = sum / count (0 / 0 = NaN when no row has a label in range), count[0] = rows counted
__global__ __launch_bounds__(kCeThreads) void ce_final(const double *__restrict__ block_sum,
                                                       const int32_t *__restrict__ block_cnt, int nblocks,
                                                       float *__restrict__ loss, int32_t *__restrict__ count)
{
    __shared__ double s_sum[kCeThreads];
    __shared__ long long s_cnt[kCeThreads];
    double t = 0.0;
    long long n = 0;
    for (int b = threadIdx.x; b < nblocks; b += kCeThreads) {
        t += block_sum[b];
        n += block_cnt[b];
    }
    s_sum[threadIdx.x] = t;
    s_cnt[threadIdx.x] = n;
    __syncthreads();
    if (threadIdx.x == 0) {
        double tt = 0.0;
        long long nn = 0;
        const int used = nblocks < kCeThreads ? nblocks : kCeThreads;     // the other threads hold zeros
        for (int i = 0; i < used; i++) {
            tt += s_sum[i];
            nn += s_cnt[i];
        }
        loss[0] = (float)(tt / (double)nn);
        count[0] = (int32_t)(nn > 0x7fffffffLL ? 0x7fffffffLL : nn);
    }
}

template <int G>
__global__ __launch_bounds__(kCeThreads) void ce_grad(const float *__restrict__ x, const int32_t *__restrict__ y32,
                                                      const int64_t *__restrict__ y64, const float *__restrict__ lse,
                                                      const int32_t *__restrict__ count,
                                                      const float *__restrict__ grad_loss, int64_t V, int C,
                                                      int rows_per_block, float *__restrict__ grad)
{
    constexpr int RP = kCeThreads / G;
    const int g = threadIdx.x % G, lr = threadIdx.x / G;
    const int n = count[0];
    const float scale = (grad_loss ? grad_loss[0] : 1.f) / (float)n;      // n == 0: no row is counted below
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < V ? r0 + rows_per_block : V;
    for (int64_t row = r0 + lr; row < r1; row += RP) {
        const int64_t lab = label_at(y32, y64, row);
        const bool counted = lab >= 0 && lab < C;
        const float l = lse[row];
        const float *p = x + row * (int64_t)C;
        float *q = grad + row * (int64_t)C;
        for (int c = g; c < C; c += G)
            q[c] = counted ? scale * (expf(p[c] - l) - (c == lab ? 1.f : 0.f)) : 0.f;
    }
}

// The same gradient with the matrix taken as one run of V * C floats: a lane owns four
// consecutive floats (one 16-byte load and store) and finds their rows by one division.
// Needs V * C < 2^31, C >= 4 and 16-byte aligned arrays; the last V * C % 4 floats are
// done one by one by the first lanes of the grid.
typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kCeThreads) void ce_grad_flat(const float *__restrict__ x,
                                                           const int32_t *__restrict__ y32,
                                                           const int64_t *__restrict__ y64,
                                                           const float *__restrict__ lse,
                                                           const int32_t *__restrict__ count,
                                                           const float *__restrict__ grad_loss, int V, int C,
                                                           float *__restrict__ grad)
{
    const int n = count[0];
    const float scale = (grad_loss ? grad_loss[0] : 1.f) / (float)n;
    const uint32_t total = (uint32_t)V * (uint32_t)C;
    const uint32_t quads = total / 4;
    const uint32_t t = blockIdx.x * kCeThreads + threadIdx.x;
    auto one = [&](float xv, int c, int64_t lab, float l) {
        return lab >= 0 && lab < C ? scale * (expf(xv - l) - (c == lab ? 1.f : 0.f)) : 0.f;
    };
    if (t < quads) {
        const uint32_t i = t * 4;
        const f32x4 xv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x + i));
        int row = (int)(i / (uint32_t)C);
        int c = (int)(i - (uint32_t)row * (uint32_t)C);
        // C >= 4: the four floats lie in this row and at most the next one
        const int row2 = row + 1 < V ? row + 1 : row;
        const int64_t lab_a = label_at(y32, y64, row), lab_b = label_at(y32, y64, row2);
        const float l_a = lse[row], l_b = lse[row2];
        f32x4 out;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const bool next = c + j >= C;
            out[j] = one(xv[j], next ? c + j - C : c + j, next ? lab_b : lab_a, next ? l_b : l_a);
        }
        __builtin_nontemporal_store(out, reinterpret_cast<f32x4 *>(grad + i));
    }
    if (t < total - quads * 4) {
        const uint32_t i = quads * 4 + t;
        const int row = (int)(i / (uint32_t)C), c = (int)(i - (uint32_t)row * (uint32_t)C);
        grad[i] = one(x[i], c, label_at(y32, y64, row), lse[row]);
    }
}

static int lanes_per_row(int C)
{
    int g = 8;
    while (g < kWave && 4 * g < C) g <<= 1;
    return g;
}

}  // namespace jg

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

static int ce_blocks(int64_t V) { return (int)ceil_div(V > 0 ? V : 1, ce_rows_per_block(V)); }
static size_t ce_ws(int64_t V) { return carve_bytes((size_t)ce_blocks(V), 8) + carve_bytes((size_t)ce_blocks(V), 4); }

static int32_t ce_check(const char *who, int64_t V, int32_t C)
{
    if (V < 0 || C < 0) return fail(JGAMD_ERR_SIZE, "%s: negative size (V=%lld, C=%d)", who, (long long)V, C);
    if (V > ((int64_t)1 << 40)) return fail(JGAMD_ERR_SIZE, "%s: V=%lld too large", who, (long long)V);
    return 0;
}

JG_EXPORT int32_t jgamd_cross_entropy_workspace(int64_t V, int32_t C, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "cross_entropy_workspace: bytes is NULL");
    if (int32_t rc = ce_check("cross_entropy_workspace", V, C)) return rc;
    *bytes = ce_ws(V);
    return 0;
}

JG_EXPORT int32_t jgamd_cross_entropy_fwd(const float *logits, const void *labels, int32_t labels_are_i64,
                                          int32_t log_probs, int64_t V, int32_t C, float *loss, int32_t *count,
                                          float *lse, void *ws, size_t ws_bytes, void *stream)
{
    if (int32_t rc = ce_check("cross_entropy_fwd", V, C)) return rc;
    if (!loss || !count) return fail(JGAMD_ERR_NULL, "cross_entropy_fwd: loss / count is NULL");
    // rows without classes have no logsumexp (and a [V,0] array has no address to read)
    if (V > 0 && C == 0) return fail(JGAMD_ERR_SIZE, "cross_entropy_fwd: V=%lld rows of C=0 classes", (long long)V);
    if (V > 0 && (!labels || !lse || !logits))
        return fail(JGAMD_ERR_NULL, "cross_entropy_fwd: logits / labels / lse is NULL");
    const size_t need = ce_ws(V);
    if (!ws || ws_bytes < need)
        return fail(JGAMD_ERR_WORKSPACE, "cross_entropy_fwd: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "cross_entropy_fwd: workspace not 256-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver carve(ws);
    const int nblocks = ce_blocks(V);
    const int rows = ce_rows_per_block(V);
    double *block_sum = carve.take<double>((size_t)nblocks);
    int32_t *block_cnt = carve.take<int32_t>((size_t)nblocks);
    const int32_t *y32 = labels_are_i64 ? nullptr : static_cast<const int32_t *>(labels);
    const int64_t *y64 = labels_are_i64 ? static_cast<const int64_t *>(labels) : nullptr;
    if (V > 0) {
        const int G = lanes_per_row(C);
        const bool reg = C <= 4 * G;
#define JG_CE(GG)                                                                                                    \
    if (G == GG) {                                                                                                   \
        if (reg)                                                                                                     \
            hipLaunchKernelGGL((ce_rows<GG, true>), dim3((unsigned)nblocks), dim3(kCeThreads), 0, st, logits, y32,   \
                               y64, V, C, rows, log_probs, lse, block_sum, block_cnt);                                                \
        else                                                                                                         \
            hipLaunchKernelGGL((ce_rows<GG, false>), dim3((unsigned)nblocks), dim3(kCeThreads), 0, st, logits, y32,  \
                               y64, V, C, rows, log_probs, lse, block_sum, block_cnt);                                                \
    }
        JG_CE(8) JG_CE(16) JG_CE(32) JG_CE(64)
#undef JG_CE
    }
    hipLaunchKernelGGL(ce_final, dim3(1), dim3(kCeThreads), 0, st, block_sum, block_cnt, V > 0 ? nblocks : 0, loss, count);
    return launch_status("cross_entropy_fwd");
}

JG_EXPORT int32_t jgamd_cross_entropy_bwd(const float *logits, const void *labels, int32_t labels_are_i64,
                                          const float *lse, const int32_t *count, const float *grad_loss, int64_t V,
                                          int32_t C, float *grad_logits, void *stream)
{
    if (int32_t rc = ce_check("cross_entropy_bwd", V, C)) return rc;
    if (V == 0 || C == 0) return 0;
    if (!logits || !labels || !lse || !count || !grad_logits)
        return fail(JGAMD_ERR_NULL, "cross_entropy_bwd: NULL array");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t *y32 = labels_are_i64 ? nullptr : static_cast<const int32_t *>(labels);
    const int64_t *y64 = labels_are_i64 ? static_cast<const int64_t *>(labels) : nullptr;
    if (C >= 4 && V * (int64_t)C < ((int64_t)1 << 31) && (((uintptr_t)logits | (uintptr_t)grad_logits) & 15) == 0) {
        const int64_t quads = V * (int64_t)C / 4;
        hipLaunchKernelGGL(ce_grad_flat, dim3((unsigned)ceil_div(quads > 0 ? quads : 1, kCeThreads)), dim3(kCeThreads), 0,
                           st, logits, y32, y64, lse, count, grad_loss, (int)V, C, grad_logits);
        return launch_status("cross_entropy_bwd");
    }
    const int nblocks = ce_blocks(V);
    const int G = lanes_per_row(C);
#define JG_CE(GG)                                                                                                  \
    if (G == GG)                                                                                                   \
        hipLaunchKernelGGL((ce_grad<GG>), dim3((unsigned)nblocks), dim3(kCeThreads), 0, st, logits, y32, y64, lse, \
                           count, grad_loss, V, C, ce_rows_per_block(V), grad_logits);
    JG_CE(8) JG_CE(16) JG_CE(32) JG_CE(64)
#undef JG_CE
    return launch_status("cross_entropy_bwd");
}
