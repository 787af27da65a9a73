// Error plumbing, version, and the device-wide exclusive scan used by the
// conversion kernels.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace jg {

static thread_local char g_err[512] = "";

int32_t fail(int32_t code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int32_t launch_status(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    return fail(static_cast<int32_t>(e), "%s: %s", what, hipGetErrorString(e));
}

// --------------------------------------------------------------------------
// Exclusive scan, three launches: per-tile sums, a one-block scan of the tile
// sums, then a per-tile scan seeded with its tile's prefix.  A tile is
// 512 threads x 8 consecutive ints per thread.
// --------------------------------------------------------------------------
constexpr int kScanThreads = 512;
constexpr int kScanPerThread = 8;
constexpr int kScanTile = kScanThreads * kScanPerThread;

size_t scan_ws_ints(int64_t n) { return static_cast<size_t>(ceil_div(n > 0 ? n : 1, kScanTile)) + 1; }

__device__ __forceinline__ int wave_inclusive_scan(int v)
{
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int t = __shfl_up(v, d, kWave);
        if (lane_id() >= d) v += t;
    }
    return v;
}

// Exclusive prefix of `v` over the block (thread order); total in *block_total.
__device__ __forceinline__ int block_exclusive_scan(int v, int *block_total)
{
    __shared__ int wave_sums[kScanThreads / kWave];
    __shared__ int total;
    int inc = wave_inclusive_scan(v);
    int w = threadIdx.x >> 6;
    if (lane_id() == kWave - 1) wave_sums[w] = inc;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int i = 0; i < kScanThreads / kWave; i++) {
            int t = wave_sums[i];
            wave_sums[i] = run;
            run += t;
        }
        total = run;
    }
    __syncthreads();
    int r = wave_sums[w] + inc - v;
    *block_total = total;
    __syncthreads();
    return r;
}

__device__ __forceinline__ void load_tile(const int32_t *in, int64_t n, int64_t base, int (&v)[kScanPerThread])
{
#pragma unroll
    for (int i = 0; i < kScanPerThread; i++) {
        int64_t p = base + i;
        v[i] = p < n ? in[p] : 0;
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums(const int32_t *__restrict__ in, int64_t n,
                                                               int32_t *__restrict__ sums)
{
    int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    int v[kScanPerThread];
    load_tile(in, n, base, v);
    int s = 0;
#pragma unroll
    for (int i = 0; i < kScanPerThread; i++) s += v[i];
    int total;
    block_exclusive_scan(s, &total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(kScanThreads) void scan_sums_one_block(int32_t *sums, int64_t nb)
{
    int carry = 0;
    for (int64_t base = 0; base < nb; base += kScanThreads) {
        int64_t p = base + threadIdx.x;
        int v = p < nb ? sums[p] : 0;
        int total;
        int ex = block_exclusive_scan(v, &total);
        if (p < nb) sums[p] = carry + ex;
        carry += total;
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_apply(const int32_t *in, int32_t *out, int64_t n,
                                                           const int32_t *__restrict__ sums)
{
    int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    int v[kScanPerThread];
    load_tile(in, n, base, v);
    int s = 0;
#pragma unroll
    for (int i = 0; i < kScanPerThread; i++) s += v[i];
    int total;
    int run = block_exclusive_scan(s, &total) + sums[blockIdx.x];
#pragma unroll
    for (int i = 0; i < kScanPerThread; i++) {
        int64_t p = base + i;
        if (p < n) out[p] = run;
        run += v[i];
    }
}

int32_t exclusive_scan_i32(const int32_t *in, int32_t *out, int64_t n, int32_t *sums_ws, hipStream_t s)
{
    if (n <= 0) return 0;
    int64_t nb = ceil_div(n, kScanTile);
    hipLaunchKernelGGL(scan_tile_sums, dim3((unsigned)nb), dim3(kScanThreads), 0, s, in, n, sums_ws);
    hipLaunchKernelGGL(scan_sums_one_block, dim3(1), dim3(kScanThreads), 0, s, sums_ws, nb);
    hipLaunchKernelGGL(scan_apply, dim3((unsigned)nb), dim3(kScanThreads), 0, s, in, out, n, sums_ws);
    return launch_status("exclusive_scan_i32");
}

}  // namespace jg

extern "C" __attribute__((visibility("default"))) int32_t jgamd_version(void) { return 300; }
extern "C" __attribute__((visibility("default"))) const char *jgamd_last_error(void) { return jg::g_err; }
