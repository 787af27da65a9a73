// Shared host/device helpers for the gfx950 kernels (wave64 everywhere).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "../../include/jgamd.h"

namespace jg {

constexpr int kWave = 64;

// Records a message for jgamd_last_error() and returns `code`.
int32_t fail(int32_t code, const char *fmt, ...);
// Checks the launch that was just enqueued; returns 0 or the hipError_t.
int32_t launch_status(const char *what);

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Bump allocator over the caller's workspace (256-byte granules).
struct Carver {
    char *base;
    size_t used = 0;
    explicit Carver(void *p) : base(static_cast<char *>(p)) {}
    template <typename T> T *take(size_t n)
    {
        T *r = reinterpret_cast<T *>(base + used);
        used += align_up(n * sizeof(T), 256);
        return r;
    }
};
inline size_t carve_bytes(size_t n, size_t elem) { return align_up(n * elem, 256); }

// ---- device-wide exclusive scan over int32 (scan.hip) ---------------------
// out[i] = sum(in[0..i-1]); in == out allowed.  sums_ws needs
// scan_ws_ints(n) int32 of scratch.
size_t scan_ws_ints(int64_t n);
int32_t exclusive_scan_i32(const int32_t *in, int32_t *out, int64_t n, int32_t *sums_ws,
                           hipStream_t s);

// ---- per-graph partition for the merge-path and tile kernels (plan.hip) ------
constexpr int kPlanGroup = 32;             // chunks per group of pre-summed row pieces
// A row of the product that crosses at most this many group boundaries has its group sums formed
// by the wavefront that finishes the row; only longer rows use (and a plan only lists) pre-summed
// groups.  At most (kSpmmInlineGroups + 1) * kPlanGroup pieces are then added by one wavefront.
constexpr int kSpmmInlineGroups = 2;
constexpr int kTileEntriesWide = 2048;     // entries per tile at 1 or 2 floats per entry
constexpr int kTileEntriesNarrow = 1024;   // and at 4 or 8

struct ChunkPlanShape {
    int chunk, nchunks, ngroups;
    size_t header_bytes, start_bytes, fix_bytes, grp_bytes;
};
// start[k] = (row, entry) at which chunk k begins, k <= nchunks.  fix / grp: ascending lists of
// the chunks whose first row has earlier pieces / of the groups a row continues past, their
// lengths in counts[0] / counts[1]; all three NULL when only the starts were computed (every
// chunk and group is then looked at).
struct ChunkPlan {
    const int2 *start;
    const int32_t *fix, *grp, *counts;
    int chunk, nchunks;
};
struct TilePlan {
    const int32_t *tile_first, *tile_last;
};
int spmm_chunk_for(int64_t M);      // items per wavefront of the product (spmm.hip)
int gat_chunk_for(int64_t M);       // and of the fused attention kernels (gat.hip)
ChunkPlanShape chunk_plan_shape(int kind, int32_t R, int64_t E);
size_t chunk_plan_bytes(int kind, int32_t R, int64_t E);
ChunkPlan chunk_plan_view(int kind, int32_t R, int64_t E, const void *plan);
void chunk_starts_enqueue(const int32_t *off, int32_t R, int64_t E, int chunk, int nchunks, int2 *start, hipStream_t s);
size_t tile_plan_bytes(int64_t E);
TilePlan tile_plan_view(int64_t E, int T, const void *plan);
void tile_columns_enqueue(const int32_t *off, int32_t V, int64_t E, int T, int32_t *tile_first, int32_t *tile_last,
                          hipStream_t s);

// ---- row-gather SpMM for use by other kernels' host code (spmm.hip) ---------
size_t spmm_ws_bytes(int32_t R, int64_t E, int32_t F);
// tiles: the tile plan of `off` (rows of 1, 2, 4 or 8 floats take the tile kernels), or NULL
int32_t spmm_enqueue(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, int32_t R,
                     int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, hipStream_t s,
                     const void *tiles = nullptr);
// the same product walked one 64-float slab of the feature rows at a time (spmm_blocked.hip)
// k0 / k1: optional events recorded on s right before and after the gather kernel; x_stride:
// floats between the rows of x when they are padded apart (0 = F)
int32_t spmm_enqueue_slabs(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out,
                           int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, hipStream_t s,
                           hipEvent_t k0 = nullptr, hipEvent_t k1 = nullptr, int x_stride = 0);

// ---- tile-based edge softmax for 1, 2, 4 or 8 heads (entry_tiles.hip) --
// fwd: a = x, b unused; bwd: a = y, b = g.  Needs V > 0, E > 0, off[V] == E.
bool edge_softmax_flat_supported(int H);
size_t entry_tiles_ws_bytes(int64_t E);
void edge_softmax_flat_enqueue(bool fwd, const int32_t *off, const float *a, const float *b, float *out, int32_t V,
                               int64_t E, int32_t H, void *ws, hipStream_t s, const void *tiles = nullptr);

// ---- gather-sum for rows of 1, 2, 4 or 8 floats (entry_tiles.hip) ----------
// Same result as the wide-row product; shares entry_tiles_ws_bytes(E) of workspace.
bool narrow_spmm_supported(int F, const void *x);
void narrow_spmm_enqueue(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, int32_t R,
                         int32_t C, int64_t E, int32_t F, void *ws, hipStream_t s, const void *tiles = nullptr);

#ifdef __HIPCC__
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }
// Wave index inside the block as a wave-uniform (scalar) value.
__device__ __forceinline__ int wave_in_block()
{
    return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
}
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int bcast_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float bcast_f(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
#endif

}  // namespace jg
