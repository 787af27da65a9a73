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

// W = floats per lane (1, or 4 when F % 4 == 0 and x is 16-byte aligned): a row is then F / W
// lanes wide and every load moves 16 bytes.
template <int W>
__global__ __launch_bounds__(kColThreads) void column_partial_sums(const float *__restrict__ x, int64_t R, int F,
                                                                   int stripe, float *__restrict__ partial)
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
                vec v[kB];
#pragma unroll
                for (int i = 0; i < kB; i++) {
                    const int64_t r = rb + (int64_t)i * groups;
                    v[i] = __builtin_nontemporal_load(reinterpret_cast<const vec *>(x + (r < r1 ? r : r1 - 1) * F) + col);
                }
#pragma unroll
                for (int i = 0; i < kB; i++)
                    if (rb + (int64_t)i * groups < r1) {
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

__global__ void column_final_sums(const float *__restrict__ partial, int nblocks, int F, float *__restrict__ out)
{
    __shared__ float part[16][64];
    const int col = blockIdx.x * 64 + (threadIdx.x & 63);
    const int grp = threadIdx.x >> 6;
    float s = 0.f;
    if (col < F)
        for (int b = grp; b < nblocks; b += 16) s += partial[(size_t)b * F + col];
    part[grp][threadIdx.x & 63] = s;
    __syncthreads();
    if (grp == 0 && col < F) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) t += part[k][threadIdx.x];
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

JG_EXPORT int32_t jgamd_column_sum(const float *x, float *out, int64_t R, int32_t F, void *ws, size_t ws_bytes,
                                   void *stream)
{
    if (R < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "column_sum: negative size");
    if (F == 0) return 0;
    if (!out) return fail(JGAMD_ERR_NULL, "column_sum: out is NULL");
    if (R > 0 && !x) return fail(JGAMD_ERR_NULL, "column_sum: x is NULL");
    const size_t need = colsum_ws(R, F);
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "column_sum: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "column_sum: workspace not 256-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    float *partial = static_cast<float *>(ws);
    const int nblocks = col_blocks(R);
    const int stripe = col_stripe(R);
    if (R > 0) {
        if (F % 4 == 0 && ((uintptr_t)x & 15) == 0)
            hipLaunchKernelGGL((column_partial_sums<4>), dim3((unsigned)nblocks), dim3(kColThreads), 0, st, x, R, F, stripe,
                               partial);
        else
            hipLaunchKernelGGL((column_partial_sums<1>), dim3((unsigned)nblocks), dim3(kColThreads), 0, st, x, R, F, stripe,
                               partial);
    }
    hipLaunchKernelGGL(column_final_sums, dim3((unsigned)ceil_div(F, 64)), dim3(1024), 0, st, partial, R > 0 ? nblocks : 0,
                       F, out);
    return launch_status("column_sum");
}
