// Column-blocked row-gather product for matrices with long rows.
//
// out[r,:] = sum_j w[j] * x[idx[j],:] gathers rows of x at random.  When x is larger than an
// L2 (4 MB per XCD) nearly every gather is served from beyond it, and a matrix with hundreds of
// entries per row (V = 233k, 492 entries per row) then runs at the rate the fabric delivers
// 128-byte lines, whatever the row width.  Here the columns are cut into NB blocks small
// enough that a block's rows of x (one 256-byte slab of them when the rows are wider) stay in
// L2, and the entries of every row are regrouped by block, keeping their order inside a block:
// the blocked matrix has NB * R rows, row b * R + r holding the entries of row r whose column
// falls in block b.  The ordinary merge-path product over those rows, walked slab by slab,
// visits block after block, so that at any time the wavefronts on all XCDs gather from the same
// few megabytes; the NB partial rows of each output row are then added in block order.  No
// float atomics: the result does not change from run to run.
//
// The regrouping is a stable partition of each row by block: a histogram per row (one
// wavefront per row, lane b counts block b), the library's scan over the NB * R counts, and a
// scatter that ranks the entries of a 64-entry batch with ballots.  It is done once per matrix
// and kept by the caller.
#include "common.h"

namespace jg {

constexpr int kMaxBlocks = kWave;   // lane b of a wavefront owns block b
constexpr int kBlockedThreads = 256;
constexpr int kBlockedWaves = kBlockedThreads / kWave;

__device__ __forceinline__ int block_of(int col, int block_cols, int nb)
{
    const int b = (int)((unsigned)col / (unsigned)block_cols);      // a negative column lands in the last block
    return b < nb ? b : nb - 1;
}

__device__ __forceinline__ void row_range(const int32_t *__restrict__ off, int r, int64_t E, int &a, int &e)
{
    a = (int)min((int64_t)max(off[r], 0), E);
    e = (int)min((int64_t)max(off[r + 1], a), E);
}

// counts[b * R + r] = entries of row r in block b; counts[NB * R] = 0
__global__ __launch_bounds__(kBlockedThreads) void blocked_count(const int32_t *__restrict__ off,
                                                                 const int32_t *__restrict__ idx, int R, int64_t E,
                                                                 int block_cols, int nb, int32_t *__restrict__ counts)
{
    const int r = blockIdx.x * kBlockedWaves + wave_in_block();
    const int lane = lane_id();
    if (r == 0 && lane == 0) counts[(size_t)nb * R] = 0;
    if (r >= R) return;
    int a, e;
    row_range(off, uniform(r), E, a, e);
    int mine = 0;      // lane b: entries of block b so far
    for (int j0 = a; j0 < e; j0 += kWave) {
        const int j = j0 + lane;
        const int b = j < e ? block_of(idx[j], block_cols, nb) : -1;
        uint64_t todo = __ballot(b >= 0);
        while (todo) {
            const int first = __ffsll((long long)todo) - 1;
            const int bb = bcast_i(b, uniform(first));
            const uint64_t same = __ballot(b == bb);
            if (lane == bb) mine += __popcll(same);
            todo &= ~same;
        }
    }
    if (lane < nb) counts[(size_t)lane * R + r] = mine;
}

__global__ __launch_bounds__(kBlockedThreads) void blocked_scatter(const int32_t *__restrict__ off,
                                                                   const int32_t *__restrict__ idx,
                                                                   const float *__restrict__ w, int R, int64_t E,
                                                                   int block_cols, int nb,
                                                                   const int32_t *__restrict__ b_off,
                                                                   int32_t *__restrict__ b_idx, float *__restrict__ b_w)
{
    const int r = blockIdx.x * kBlockedWaves + wave_in_block();
    if (r >= R) return;
    const int lane = lane_id();
    int a, e;
    row_range(off, uniform(r), E, a, e);
    int base = lane < nb ? b_off[(size_t)lane * R + r] : 0;      // lane b: next free slot of block b
    const uint64_t below = ((uint64_t)1 << lane) - 1;
    for (int j0 = a; j0 < e; j0 += kWave) {
        const int j = j0 + lane;
        const bool ok = j < e;
        const int col = ok ? idx[j] : 0;
        const float wt = (ok && w) ? w[j] : 1.f;
        const int b = ok ? block_of(col, block_cols, nb) : -1;
        int pos = 0;
        uint64_t todo = __ballot(ok);
        while (todo) {
            const int first = __ffsll((long long)todo) - 1;
            const int bb = bcast_i(b, uniform(first));
            const uint64_t same = __ballot(b == bb);
            const int start = bcast_i(base, bb);
            if (b == bb) pos = start + __popcll(same & below);
            if (lane == bb) base += __popcll(same);
            todo &= ~same;
        }
        if (ok && pos >= 0 && pos < E) {
            b_idx[pos] = col;
            if (b_w) b_w[pos] = wt;
        }
    }
}

// out[r,f] = beta * sum_b partial[b * R + r, f] + alpha * h[r or 0, f], blocks added in order
__global__ __launch_bounds__(256) void blocked_sum(const float *__restrict__ partial, int nb, int R, int F,
                                                   float beta, float alpha, const float *__restrict__ h,
                                                   int h_stride, float *__restrict__ out)
{
    const int64_t n = (int64_t)R * F;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    int b = 0;
    for (; b + 4 <= nb; b += 4) {
        const float v0 = __builtin_nontemporal_load(partial + (size_t)b * n + i);
        const float v1 = __builtin_nontemporal_load(partial + (size_t)(b + 1) * n + i);
        const float v2 = __builtin_nontemporal_load(partial + (size_t)(b + 2) * n + i);
        const float v3 = __builtin_nontemporal_load(partial + (size_t)(b + 3) * n + i);
        s = ((s + v0) + v1) + v2 + v3;
    }
    for (; b < nb; b++) s += __builtin_nontemporal_load(partial + (size_t)b * n + i);
    if (h) s = fmaf(alpha, h[h_stride ? i : i % F], beta * s);
    else s = beta * s;
    out[i] = s;
}

// same with four floats per lane, for F % 4 == 0 and 16-byte aligned arrays
typedef float f32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void blocked_sum4(const f32x4 *__restrict__ partial, int nb, int64_t n4, int F4,
                                                    float beta, float alpha, const f32x4 *__restrict__ h,
                                                    int h_stride, f32x4 *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int b = 0; b < nb; b++) s += __builtin_nontemporal_load(partial + (size_t)b * n4 + i);
    if (h) {
        const f32x4 hv = h[h_stride ? i : i % F4];
        for (int c = 0; c < 4; c++) s[c] = fmaf(alpha, hv[c], beta * s[c]);
    } else {
        s *= beta;
    }
    out[i] = s;
}

// xp[r * fpad + f] = x[r * F + f]: rows moved apart so that each starts on a 128-byte line
__global__ __launch_bounds__(256) void blocked_pad_rows(const float *__restrict__ x, int64_t rows, int F, int fpad,
                                                        float *__restrict__ xp)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * fpad) return;
    const int64_t r = i / fpad;
    const int f = (int)(i - r * fpad);
    if (f < F) xp[i] = x[r * F + f];
}

// Row width the gathers run at.  Wide rows: a multiple of 32 floats, so that every 256-byte slab of
// a row is two whole lines (a 2408-byte row's slabs straddle three: F = 602 ran 25.4 -> 20.4 ms).
// Rows of one slab: a multiple of 16 floats, which already fixes the number of lines a row touches
// and keeps the block's footprint in L2 smaller than whole-line rows would.
// Rows of 1, 2, 4 or 8 floats stay as they are: they never straddle a line they need not, and
// the product's kernels for those widths read rows F floats apart.
static int padded_width(int F)
{
    if (F == 1 || F == 2 || F == 4 || F == 8) return F;
    return F <= kWave ? (F + 15) & ~15 : (F + 31) & ~31;
}

static int env_kb(const char *name, int dflt)
{
    const char *s = getenv(name);
    if (!s || !*s) return dflt;
    const int v = atoi(s);
    return v > 0 ? v : dflt;
}

static bool blocked_sizes_ok(int32_t R, int64_t E, int32_t nb)
{
    return nb >= 1 && nb <= kMaxBlocks && (int64_t)nb * R + E < ((int64_t)1 << 31) - 8192;
}

}  // namespace jg

using namespace jg;

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_block_plan(int32_t R, int32_t C, int64_t E,
                                                                                int32_t F, int32_t *nb,
                                                                                int32_t *block_cols)
{
    if (!nb || !block_cols) return fail(JGAMD_ERR_NULL, "spmm_block_plan: NULL result");
    if (R < 0 || C < 0 || E < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "spmm_block_plan: negative size");
    *nb = 0;
    *block_cols = 0;
    static const int off_switch = env_kb("JGAMD_SPMM_BLOCKED_OFF", 0);
    if (off_switch || R == 0 || C == 0 || F <= 8) return 0;
    // bytes of x one block may cover.  Measured on V = 233k, 492 entries per row, F = 41 .. 602:
    // 1.5 MB .. 16 MB blocks; fastest between 4.5 and 6 MB (fewer partial rows against more misses)
    static const int kb = env_kb("JGAMD_SPMM_BLOCK_KB", 4608);
    // one blocking per matrix whatever the width: a block is sized for the 256-byte slabs of wide
    // rows, and rows narrower than that just fill less of it
    const int64_t slab_bytes = (int64_t)kWave * 4;
    int64_t cols = ((int64_t)kb * 1024 / slab_bytes) & ~(int64_t)255;
    if (cols < 1024) cols = 1024;
    const int64_t blocks = ceil_div((int64_t)C, cols);
    // worth it when x does not fit anyway, the partial rows are a small share of the gathers
    // (8 entries or more per blocked row on average) and a lane per block suffices
    if (blocks < 3 || blocks > kMaxBlocks) return 0;
    if ((int64_t)C * F * 4 <= ((int64_t)8 << 20)) return 0;      // narrow rows: all of x is about an L2's worth
    if (E < 8 * blocks * (int64_t)R) return 0;
    if (!blocked_sizes_ok(R, E, (int32_t)blocks)) return 0;
    *nb = (int32_t)blocks;
    *block_cols = (int32_t)cols;
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_csx_block_columns_workspace(int32_t R, int32_t nb,
                                                                                            size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "csx_block_columns_workspace: NULL result");
    if (R < 0 || nb < 1 || nb > kMaxBlocks) return fail(JGAMD_ERR_SIZE, "csx_block_columns_workspace: R=%d nb=%d", R, nb);
    const int64_t n = (int64_t)nb * R + 1;
    *bytes = carve_bytes((size_t)n, 4) + carve_bytes(scan_ws_ints(n), 4);
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_csx_block_columns(
    const int32_t *off, const int32_t *idx, const float *w, int32_t R, int64_t E, int32_t block_cols, int32_t nb,
    int32_t *b_off, int32_t *b_idx, float *b_w, void *ws, size_t ws_bytes, void *stream)
{
    if (R < 0 || E < 0) return fail(JGAMD_ERR_SIZE, "csx_block_columns: negative size");
    if (block_cols < 1) return fail(JGAMD_ERR_SIZE, "csx_block_columns: block_cols = %d", block_cols);
    if (!blocked_sizes_ok(R, E, nb))
        return fail(JGAMD_ERR_SIZE, "csx_block_columns: nb = %d outside [1, %d] or nb * R + E above 2^31", nb, kMaxBlocks);
    if (!off || !b_off) return fail(JGAMD_ERR_NULL, "csx_block_columns: off / b_off is NULL");
    if (E > 0 && (!idx || !b_idx)) return fail(JGAMD_ERR_NULL, "csx_block_columns: idx / b_idx is NULL");
    if ((w == nullptr) != (b_w == nullptr) && E > 0)
        return fail(JGAMD_ERR_NULL, "csx_block_columns: w and b_w must both be given or both be NULL");
    size_t need = 0;
    if (int32_t rc = jgamd_csx_block_columns_workspace(R, nb, &need)) return rc;
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "csx_block_columns: workspace of %zu bytes needed", need);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t n = (int64_t)nb * R + 1;
    Carver carve(ws);
    int32_t *counts = carve.take<int32_t>((size_t)n);
    int32_t *sums = carve.take<int32_t>(scan_ws_ints(n));
    const unsigned grid = (unsigned)ceil_div(R > 0 ? R : 1, kBlockedWaves);
    hipLaunchKernelGGL(blocked_count, dim3(grid), dim3(kBlockedThreads), 0, s, off, idx, R, E, block_cols, nb, counts);
    if (int32_t rc = exclusive_scan_i32(counts, b_off, n, sums, s)) return rc;
    if (R > 0 && E > 0)
        hipLaunchKernelGGL(blocked_scatter, dim3(grid), dim3(kBlockedThreads), 0, s, off, idx, w, R, E, block_cols, nb,
                           b_off, b_idx, b_w);
    return launch_status("csx_block_columns");
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_blocked_workspace(int32_t R, int32_t C,
                                                                                           int64_t E, int32_t F,
                                                                                           int32_t nb, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "spmm_csx_blocked_workspace: NULL result");
    if (R < 0 || C < 0 || E < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "spmm_csx_blocked_workspace: negative size");
    if (!blocked_sizes_ok(R, E, nb)) return fail(JGAMD_ERR_SIZE, "spmm_csx_blocked_workspace: nb = %d, R = %d", nb, R);
    const size_t padded = padded_width(F) != F ? carve_bytes((size_t)C * (size_t)padded_width(F), 4) : 0;
    *bytes = (R == 0 || F == 0)
                 ? 0
                 : carve_bytes((size_t)nb * (size_t)R * (size_t)F, 4) + padded + spmm_ws_bytes(nb * R, E, F);
    return 0;
}

static int32_t blocked_call(const int32_t *b_off, const int32_t *b_idx, const float *b_w, const float *x, float *out,
                            float beta, float alpha, const float *h, int32_t h_rows, int32_t R, int32_t C, int64_t E,
                            int32_t F, int32_t nb, void *ws, size_t ws_bytes, void *stream, hipEvent_t k0, hipEvent_t k1)
{
    size_t need = 0;
    if (int32_t rc = jgamd_spmm_csx_blocked_workspace(R, C, E, F, nb, &need)) return rc;
    if (R == 0 || F == 0) return 0;
    if (!b_off || !out) return fail(JGAMD_ERR_NULL, "spmm_csx_blocked: b_off / out is NULL");
    if (h && h_rows != 1 && h_rows != R)
        return fail(JGAMD_ERR_SIZE, "spmm_csx_blocked: h has %d rows, expected %d or 1", h_rows, R);
    if ((((uintptr_t)x | (uintptr_t)out | (uintptr_t)h) & 3) != 0)
        return fail(JGAMD_ERR_ALIGN, "spmm_csx_blocked: x / out / h not 4-byte aligned");
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "spmm_csx_blocked: workspace of %zu bytes needed", need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "spmm_csx_blocked: workspace not 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Carver carve(ws);
    float *partial = carve.take<float>((size_t)nb * (size_t)R * (size_t)F);
    const int fpad = padded_width(F);
    const float *gathered = x;
    if (fpad != F && C > 0 && E > 0) {
        float *xp = carve.take<float>((size_t)C * (size_t)fpad);
        const int64_t n = (int64_t)C * fpad;
        hipLaunchKernelGGL(blocked_pad_rows, dim3((unsigned)ceil_div(n, (int64_t)256)), dim3(256), 0, s, x, (int64_t)C, F, fpad,
                           xp);
        gathered = xp;
    }
    void *inner = static_cast<char *>(ws) + carve.used;
    if (int32_t rc = spmm_enqueue_slabs(b_off, b_idx, b_w, gathered, partial, nb * R, C, E, F, inner,
                                        ws_bytes - carve.used, s, k0, k1, gathered == x ? 0 : fpad))
        return rc;
    const float *hh = alpha != 0.f ? h : nullptr;
    const int h_stride = h_rows == 1 ? 0 : 1;
    const int64_t n = (int64_t)R * F;
    if (F % 4 == 0 && ((((uintptr_t)out | (uintptr_t)hh) & 15) == 0)) {
        hipLaunchKernelGGL(blocked_sum4, dim3((unsigned)ceil_div(n / 4, (int64_t)256)), dim3(256), 0, s,
                           reinterpret_cast<const f32x4 *>(partial), nb, n / 4, F / 4, beta, alpha,
                           reinterpret_cast<const f32x4 *>(hh), h_stride, reinterpret_cast<f32x4 *>(out));
    } else {
        hipLaunchKernelGGL(blocked_sum, dim3((unsigned)ceil_div(n, (int64_t)256)), dim3(256), 0, s, partial, nb, R, F, beta,
                           alpha, hh, h_stride, out);
    }
    return launch_status("spmm_csx_blocked");
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_blocked(
    const int32_t *b_off, const int32_t *b_idx, const float *b_w, const float *x, float *out, float beta, float alpha,
    const float *h, int32_t h_rows, int32_t R, int32_t C, int64_t E, int32_t F, int32_t nb, void *ws, size_t ws_bytes,
    void *stream)
{
    return blocked_call(b_off, b_idx, b_w, x, out, beta, alpha, h, h_rows, R, C, E, F, nb, ws, ws_bytes, stream, nullptr,
                        nullptr);
}

// the same call `iters` times with HIP events on the launch stream: mean duration of the gather
// kernel over the regrouped rows and of the whole call (gather, fix-up, sum over the blocks)
extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_blocked_timed(
    const int32_t *b_off, const int32_t *b_idx, const float *b_w, const float *x, float *out, int32_t R, int32_t C,
    int64_t E, int32_t F, int32_t nb, void *ws, size_t ws_bytes, void *stream, int32_t iters, float *kernel_ms,
    float *call_ms)
{
    if (iters < 1 || iters > 4096) return fail(JGAMD_ERR_SIZE, "spmm_csx_blocked_timed: iters must be in [1, 4096]");
    if (!kernel_ms || !call_ms) return fail(JGAMD_ERR_NULL, "spmm_csx_blocked_timed: NULL result pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipEvent_t ev[4];
    for (auto &e : ev)
        if (hipEventCreate(&e) != hipSuccess)
            return fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx_blocked_timed: hipEventCreate failed");
    double ksum = 0, csum = 0;
    int32_t rc = 0;
    for (int i = 0; i < iters && rc == 0; i++) {
        (void)hipEventRecord(ev[0], st);
        rc = blocked_call(b_off, b_idx, b_w, x, out, 1.f, 0.f, nullptr, 1, R, C, E, F, nb, ws, ws_bytes, stream, ev[1],
                          ev[2]);
        (void)hipEventRecord(ev[3], st);
        if (hipEventSynchronize(ev[3]) != hipSuccess && rc == 0)
            rc = fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx_blocked_timed: hipEventSynchronize failed");
        float k = 0, c = 0;
        if (rc == 0 && R > 0 && F > 0) {
            (void)hipEventElapsedTime(&k, ev[1], ev[2]);
            (void)hipEventElapsedTime(&c, ev[0], ev[3]);
        }
        ksum += k;
        csum += c;
    }
    for (auto &e : ev) (void)hipEventDestroy(e);
    *kernel_ms = (float)(ksum / iters);
    *call_ms = (float)(csum / iters);
    return rc;
}
