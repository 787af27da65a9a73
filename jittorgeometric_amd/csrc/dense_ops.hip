// Column sums of a row-major [R,F] matrix: the bias gradient of the conv
// layers (out += bias in gcn_conv.py:100-101 of the reference; its backward
// is a sum over all nodes).  Two deterministic stages: every block sums a
// stripe of rows into partial[block][F], one more kernel adds the partials in
// block order.  Narrow odd widths (47 classes) are where a generic reduction
// falls off a cliff; here a block's threads are laid out as
// (row group, column) so that each pass reads a contiguous run of whole rows.
#include "common.h"

namespace jg {

constexpr int kColThreads = 256;
constexpr int kColStripe = 512;    // rows per block: about 2000 blocks at V = 10^6, eight per CU, to keep enough loads in flight
constexpr int kColMinStripe = 16;
constexpr int kColMaxBlocks = 2048;     // more rows per block beyond that: the second stage reads one partial row per block
constexpr int kColOneStage = 8192;      // up to this many rows the second stage's kernel sums the matrix itself: one launch

// W = floats per lane (1, or 4 when F % 4 == 0 and x is 16-byte aligned): a row is then F / W
// lanes wide and every load moves 16 bytes.
// MASK: x is an upstream gradient and y the output of a ReLU; the kernel sums and writes
// masked[r,c] = y[r,c] > 0 ? x[r,c] : 0 (the gradient in front of the ReLU) in the same pass.
template <int W, bool MASK>
__global__ __launch_bounds__(kColThreads) void column_partial_sums(const float *__restrict__ x, int64_t R, int F,
                                                                   int stripe, float *__restrict__ partial,
                                                                   const float *__restrict__ y = nullptr,
                                                                   float *__restrict__ masked = nullptr)
{
    typedef float vec __attribute__((ext_vector_type(W)));
    __shared__ float red[kColThreads][W];
    const int FW = F / W;                                   // lanes per row
    const int cols = FW < kColThreads ? FW : kColThreads;   // lanes of one row handled per slab
    const int groups = kColThreads / cols;                  // rows read together
    const int c = threadIdx.x % cols, g = threadIdx.x / cols;
    const int64_t r0 = (int64_t)blockIdx.x * stripe;
    const int64_t r1 = r0 + stripe < R ? r0 + stripe : R;
    for (int slab = 0; slab < FW; slab += cols) {
        const int col = slab + c;
        float s[W];
#pragma unroll
        for (int k = 0; k < W; k++) s[k] = 0.f;
        if (g < groups && col < FW) {
            constexpr int kB = 8;                            // loads in flight per thread
            for (int64_t rb = r0 + g; rb < r1; rb += (int64_t)kB * groups) {
                vec v[kB], yv[MASK ? kB : 1];
#pragma unroll
                for (int i = 0; i < kB; i++) {
                    const int64_t r = rb + (int64_t)i * groups;
                    v[i] = __builtin_nontemporal_load(reinterpret_cast<const vec *>(x + (r < r1 ? r : r1 - 1) * F) + col);
                    if constexpr (MASK)
                        yv[i] = __builtin_nontemporal_load(reinterpret_cast<const vec *>(y + (r < r1 ? r : r1 - 1) * F) + col);
                }
#pragma unroll
                for (int i = 0; i < kB; i++)
                    if (rb + (int64_t)i * groups < r1) {
                        if constexpr (MASK) {
                            vec m;
#pragma unroll
                            for (int k = 0; k < W; k++) m[k] = yv[i][k] > 0.f ? v[i][k] : 0.f;
                            v[i] = m;
                            *(reinterpret_cast<vec *>(masked + (rb + (int64_t)i * groups) * F) + col) = m;
                        }
#pragma unroll
                        for (int k = 0; k < W; k++) s[k] += v[i][k];
                    }
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < W; k++) red[threadIdx.x][k] = s[k];
        __syncthreads();
        if (g == 0 && col < FW) {
#pragma unroll
            for (int k = 0; k < W; k++) {
                float t = 0.f;
                for (int q = 0; q < groups; q++) t += red[q * cols + c][k];
                partial[(size_t)blockIdx.x * F + (size_t)col * W + k] = t;
            }
        }
    }
}

// Second stage: the partial rows added in block order.  A block owns COLS columns and splits the
// partial rows over 1024 / COLS groups of threads (group g takes rows g, g + groups, ...), whose
// sums are then added in group order.  COLS = 16 keeps a narrow matrix (a few dozen to a few
// hundred columns, two thousand partial rows) from being two or three blocks' serial work:
// 128 columns are 8 blocks of 64 groups instead of 2 blocks of 16 (32 -> 9 us at 1954 rows).
// MASK: the rows are an upstream gradient itself (a matrix of few rows needs no first stage),
// masked by the ReLU output y as in column_partial_sums.
template <int COLS, bool MASK = false>
__global__ __launch_bounds__(1024) void column_final_sums(const float *__restrict__ partial, int nblocks, int F,
                                                          float *__restrict__ out, const float *__restrict__ y = nullptr,
                                                          float *__restrict__ masked = nullptr)
{
    constexpr int GROUPS = 1024 / COLS;
    __shared__ float part[GROUPS][COLS];
    const int c = threadIdx.x % COLS, grp = threadIdx.x / COLS;
    const int col = blockIdx.x * COLS + c;
    float s = 0.f;
    if (col < F) {
        constexpr int kB = 8;               // rows fetched together, added in the same order as one by one
        for (int b0 = grp; b0 < nblocks; b0 += GROUPS * kB) {
            float v[kB], yv[MASK ? kB : 1];
#pragma unroll
            for (int i = 0; i < kB; i++) {
                const size_t at = (size_t)min(b0 + GROUPS * i, nblocks - 1) * F + col;
                v[i] = partial[at];
                if constexpr (MASK) yv[i] = y[at];
            }
#pragma unroll
            for (int i = 0; i < kB; i++)
                if (b0 + GROUPS * i < nblocks) {
                    if constexpr (MASK) {
                        v[i] = yv[i] > 0.f ? v[i] : 0.f;
                        masked[(size_t)(b0 + GROUPS * i) * F + col] = v[i];
                    }
                    s += v[i];
                }
        }
    }
    part[grp][c] = s;
    __syncthreads();
    if (grp == 0 && col < F) {
        float t = 0.f;
#pragma unroll 8
        for (int k = 0; k < GROUPS; k++) t += part[k][c];
        out[col] = t;
    }
}

}  // namespace jg

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

static int col_stripe(int64_t R)
{
    const int64_t s = ceil_div(R > 0 ? R : 1, kColMaxBlocks);
    if (s > kColStripe) return (int)(s < 0x7fffffff ? s : 0x7fffffff);
    // a small matrix: shorter stripes, so that a few thousand rows are still a block or two per
    // compute unit instead of half a dozen blocks in all
    int stripe = kColStripe;
    while (stripe > kColMinStripe && R / stripe < 512) stripe >>= 1;
    return stripe;
}
static int col_blocks(int64_t R) { return (int)ceil_div(R > 0 ? R : 1, col_stripe(R)); }
static size_t colsum_ws(int64_t R, int32_t F) { return carve_bytes((size_t)col_blocks(R) * F, 4); }

JG_EXPORT int32_t jgamd_column_sum_workspace(int64_t R, int32_t F, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "column_sum_workspace: bytes is NULL");
    if (R < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "column_sum: negative size");
    *bytes = F == 0 ? 0 : colsum_ws(R, F);
    return 0;
}

static int32_t column_sum(const float *x, const float *y, float *masked, float *out, int64_t R, int32_t F, void *ws,
                          size_t ws_bytes, void *stream)
{
    if (R < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "column_sum: negative size");
    if (F == 0) return 0;
    if (!out) return fail(JGAMD_ERR_NULL, "column_sum: out is NULL");
    if (R > 0 && !x) return fail(JGAMD_ERR_NULL, "column_sum: x is NULL");
    if ((y == nullptr) != (masked == nullptr) || (R > 0 && y && masked == x))
        return fail(JGAMD_ERR_NULL, "relu_backward_column_sum: y and masked go together, masked must not be g");
    const size_t need = colsum_ws(R, F);
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "column_sum: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "column_sum: workspace not 256-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (R > 0 && R <= kColOneStage && F <= 2048) {
        // a few thousand rows (a citation graph's logits): the rows are the "partial rows"
        const dim3 grid((unsigned)ceil_div(F, 16)), block(1024);
        if (y) hipLaunchKernelGGL((column_final_sums<16, true>), grid, block, 0, st, x, (int)R, F, out, y, masked);
        else hipLaunchKernelGGL((column_final_sums<16, false>), grid, block, 0, st, x, (int)R, F, out);
        return launch_status("column_sum");
    }
    float *partial = static_cast<float *>(ws);
    const int nblocks = col_blocks(R);
    const int stripe = col_stripe(R);
    if (R > 0) {
        const bool wide = F % 4 == 0 && ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)masked) & 15) == 0);
        const dim3 grid((unsigned)nblocks), block(kColThreads);
        if (y && wide)
            hipLaunchKernelGGL((column_partial_sums<4, true>), grid, block, 0, st, x, R, F, stripe, partial, y, masked);
        else if (y)
            hipLaunchKernelGGL((column_partial_sums<1, true>), grid, block, 0, st, x, R, F, stripe, partial, y, masked);
        else if (wide)
            hipLaunchKernelGGL((column_partial_sums<4, false>), grid, block, 0, st, x, R, F, stripe, partial);
        else
            hipLaunchKernelGGL((column_partial_sums<1, false>), grid, block, 0, st, x, R, F, stripe, partial);
    }
    if (F <= 2048)
        hipLaunchKernelGGL((column_final_sums<16>), dim3((unsigned)ceil_div(F, 16)), dim3(1024), 0, st, partial,
                           R > 0 ? nblocks : 0, F, out);
    else
        hipLaunchKernelGGL((column_final_sums<64>), dim3((unsigned)ceil_div(F, 64)), dim3(1024), 0, st, partial,
                           R > 0 ? nblocks : 0, F, out);
    return launch_status("column_sum");
}

JG_EXPORT int32_t jgamd_column_sum(const float *x, float *out, int64_t R, int32_t F, void *ws, size_t ws_bytes,
                                   void *stream)
{
    return column_sum(x, nullptr, nullptr, out, R, F, ws, ws_bytes, stream);
}

JG_EXPORT int32_t jgamd_relu_backward_column_sum(const float *g, const float *y, float *masked, float *out, int64_t R,
                                                 int32_t F, void *ws, size_t ws_bytes, void *stream)
{
    if (F > 0 && R > 0 && (!y || !masked)) return fail(JGAMD_ERR_NULL, "relu_backward_column_sum: y / masked is NULL");
    return column_sum(g, y, masked, out, R, F, ws, ws_bytes, stream);
}
