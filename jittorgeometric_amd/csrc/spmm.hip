// Weighted row-gather SpMM  out[r,:] = sum_j w[j] * x[idx[j],:]  for gfx950.
//
// Work split (merge-path): the R row-end markers and the E entries form one
// sequence of M = R + E items (row r's entries, then its end marker).  Every
// wavefront takes `chunk` consecutive items, so a 20,000-entry hub row is cut
// into pieces and a run of empty rows costs what the same number of entries
// would.  Inside a wavefront the feature dimension lies across the 64 lanes
// (VEC floats per lane, NT tiles of 64*VEC features), the entries are walked
// in order, and (idx, w) are loaded 64 at a time, one per lane, then staged:
// through the wavefront's LDS slice (every lane reads entry i at the same
// address, a broadcast) for F >= 64, or rotated with a shuffle and handed out
// with v_readlane for narrower rows, where the two extra LDS waits per group
// show.  Either way a gathered row is (scalar base) + (32-bit byte offset),
// and the gathers of UNROLL entries are issued before the first is used.
//
// A row that ends inside a chunk is stored by that chunk's wavefront.  The
// leading piece of a row that continues into the next chunk goes to
// partial[chunk].  spmm_fixup then adds, for every row that started in an
// earlier chunk, the pieces in chunk order.  No float atomics: the result
// does not change from run to run.
#include <stdlib.h>

#include <mutex>

#include "common.h"

namespace jg {

constexpr int kSpmmThreads = 256;
// (idx, w) staging: through LDS from this width up, through registers (shuffle + readlane) below
constexpr int kLdsStageMinWidth = 64;
constexpr int kSpmmWaves = kSpmmThreads / kWave;

template <int VEC> struct Vec;
template <> struct Vec<1> { using type = float; };
template <> struct Vec<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct Vec<4> { typedef float type __attribute__((ext_vector_type(4))); };

template <int VEC> __device__ __forceinline__ void vload(float (&d)[VEC], const float *p)
{
    using V = typename Vec<VEC>::type;
    const V v = *reinterpret_cast<const V *>(p);
    const float *f = reinterpret_cast<const float *>(&v);
#pragma unroll
    for (int i = 0; i < VEC; i++) d[i] = f[i];
}
template <int VEC> __device__ __forceinline__ void vstore(float *p, const float (&s)[VEC])
{
    using V = typename Vec<VEC>::type;
    V v;
    float *f = reinterpret_cast<float *>(&v);
#pragma unroll
    for (int i = 0; i < VEC; i++) f[i] = s[i];
    *reinterpret_cast<V *>(p) = v;
}
// Streaming variants: data touched once (indices, weights, the output) is
// marked non-temporal so that it does not displace gathered x rows from L2.
template <int VEC> __device__ __forceinline__ void vstore_stream(float *p, const float (&s)[VEC])
{
    using V = typename Vec<VEC>::type;
    V v;
    float *f = reinterpret_cast<float *>(&v);
#pragma unroll
    for (int i = 0; i < VEC; i++) f[i] = s[i];
    __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
}
template <typename T> __device__ __forceinline__ T load_stream(const T *p) { return __builtin_nontemporal_load(p); }

// WIDE = false: every row of x starts less than 4 GiB from x, so a gathered
// row is addressed as (scalar base) + (32-bit byte offset): one readlane and
// one vector add per entry.  WIDE = true keeps 64-bit row arithmetic.
//
// EPI = true finishes every row as beta * sum + alpha * h[row,:] (h == nullptr
// drops the second term).  The row of h is fetched when the row begins.  A
// row that began in an earlier chunk is stored raw: spmm_fixup adds its
// pieces and applies the same finish.
struct RowFinish {
    float beta, alpha;
    const float *h;
    int h_stride;   // floats between the rows of h: F, or 0 when one row serves every output row
    int x_stride;   // floats between the rows of x when they are padded apart; 0 = F
    int relu;       // the finished row is clamped at zero (a layer's activation in the row store)
};

template <int VEC, int NT, int UNROLL, bool WIDE, bool LDS, bool EPI>
__global__ __launch_bounds__(kSpmmThreads) void spmm_merge(const int32_t *__restrict__ off,
                                                           const int32_t *__restrict__ idx,
                                                           const float *__restrict__ w,
                                                           const float *__restrict__ x, float *__restrict__ out,
                                                           float *__restrict__ partial,
                                                           const int2 *__restrict__ start, int R, int C, int E,
                                                           int F, int nchunks, RowFinish fin)
{
    static_assert(kWave % UNROLL == 0, "groups tile a 64-entry batch");
    __shared__ int2 staged_all[LDS ? kSpmmThreads : 1];
    int2 *staged = staged_all + (LDS ? (threadIdx.x & ~(kWave - 1)) : 0);   // this wavefront's 64 slots
    const int k = blockIdx.x * kSpmmWaves + wave_in_block();
    if (k >= nchunks) return;
    const int lane = lane_id();
    const int f0 = blockIdx.y * (kWave * VEC * NT) + lane * VEC;   // this lane's first feature
    bool act[NT];
    int fo[NT];           // feature offset this lane loads from in tile t (0 when the lane is past F)
    uint32_t fo_bytes[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        act[t] = f0 + t * kWave * VEC < F;
        fo[t] = act[t] ? f0 + t * kWave * VEC : 0;
        fo_bytes[t] = (uint32_t)fo[t] * 4u;
    }
    const char *xb = reinterpret_cast<const char *>(x);
    const int xs = fin.x_stride ? fin.x_stride : F;      // rows of x may be padded to whole cache lines
    const uint32_t row_bytes = (uint32_t)xs * 4u;

    // the chunk runs from (row, entry) = start[k] to start[k + 1]; both are clamped so that a
    // malformed off/E pair cannot index outside the arrays
    const int2 s0 = start[k], s1 = start[k + 1];
    const int r1 = min(max(uniform(s1.x), 0), R);
    int r = min(max(uniform(s0.x), 0), r1);
    const int j0 = min(max(uniform(s0.y), 0), E);
    const int j1 = min(uniform(s1.y), E);

    // window of 64 row ends starting at row rb: lane l holds off[rb + 1 + l].
    // row_end = entry index at which row r ends; "never" once r has reached r1
    // (the chunk's last, unfinished row), so the per-entry test is one compare.
    constexpr int kNever = 0x7fffffff;
    int rb = r;
    int ends = (rb + lane < R) ? off[rb + 1 + lane] : kNever;
    int row_end = r < r1 ? bcast_i(ends, 0) : kNever;

    float acc[NT][VEC];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;

    // EPI: h row of the current row; raw_row = the chunk's first row when it began earlier
    float hrow[EPI ? NT : 1][EPI ? VEC : 1];
    int raw_row = -1;
    auto fetch_h = [&]() {
        if constexpr (EPI) {
            if (fin.h) {
                const float *src = fin.h + (size_t)min(r, R - 1) * fin.h_stride;
#pragma unroll
                for (int t = 0; t < NT; t++) vload<VEC>(hrow[t], src + fo[t]);
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) hrow[t][v] = 0.f;
            }
        }
    };
    if constexpr (EPI) {
        if (r < r1 && uniform(off[r]) < j0) raw_row = r;
        fetch_h();
    }

    auto flush_row = [&]() {
        float *dst = out + (size_t)r * F + f0;
        if constexpr (EPI) {
            if (r != raw_row) {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) {
                        acc[t][v] = fmaf(fin.alpha, hrow[t][v], fin.beta * acc[t][v]);
                        if (fin.relu) acc[t][v] = fmaxf(acc[t][v], 0.f);
                    }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if (act[t]) vstore_stream<VEC>(dst + t * kWave * VEC, acc[t]);
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
        }
        r++;
        if constexpr (EPI) {
            // one row for every output row (a bias) was fetched before the loop; a load here would
            // make the flush wait for every gather in flight
            if (fin.h && fin.h_stride != 0) fetch_h();
        }
        if (r - rb == kWave) {
            rb = r;
            ends = (rb + lane < R) ? off[rb + 1 + lane] : kNever;
        }
        row_end = r < r1 ? bcast_i(ends, r - rb) : kNever;
    };

    // (index, weight) of the batch after the current one are fetched while the current one is
    // worked on; the index is clamped, what lies past the chunk is discarded when it is used
    const int jlast = max(j1 - 1, 0);
    int nxt_c = idx ? load_stream(idx + min(j0 + lane, jlast)) : 0;
    float nxt_w = w ? load_stream(w + min(j0 + lane, jlast)) : 1.f;
    for (int jb = j0; jb < j1; jb += kWave) {
        const int n = min(kWave, j1 - jb);
        int my_c;
        float my_w;
        {
            const bool ok = lane < n;
            const int jj = jb + lane;
            my_c = idx ? (ok ? nxt_c : 0) : jj;
            my_w = ok ? nxt_w : 0.f;
            if (idx) nxt_c = load_stream(idx + min(jj + kWave, jlast));
            if (w) nxt_w = load_stream(w + min(jj + kWave, jlast));
            if ((unsigned)my_c >= (unsigned)C) {
                my_c = 0;
                my_w = 0.f;
            }
        }
        // what each lane contributes to addressing: its row's byte offset, or its row index
        const int my_a = WIDE ? my_c : (int)((uint32_t)my_c * row_bytes);
        if (LDS) {
            // stage the batch's (address term, weight) pairs in this wavefront's LDS slice; every
            // lane then reads entry i at the same address (a broadcast read, no VALU involved)
            __builtin_amdgcn_wave_barrier();
            staged[lane] = make_int2(my_a, __float_as_int(my_w));
            __builtin_amdgcn_wave_barrier();
        }
        for (int i0 = 0; i0 < n; i0 += UNROLL) {
            // registers: rotate the group's UNROLL entries into lanes 0..UNROLL-1 so that the
            // broadcasts below take immediate lane numbers
            const int from = (lane + i0) & (kWave - 1);
            const int g_a = LDS ? 0 : __shfl(my_a, from, kWave);
            const float g_w = LDS ? 0.f : __shfl(my_w, from, kWave);
            float wl[UNROLL];
            // Issue phase: straight-line code, no branches and no lane predicates, so that the
            // UNROLL gathers leave back to back.  Slots past n re-read the row of a lane that
            // holds no entry (offset 0, weight 0, never accumulated); lanes past F read the
            // start of the row instead of being masked off.
            float xv[UNROLL][NT][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                int a;
                if (LDS) {
                    const int2 e = staged[i0 + u];
                    a = e.x;
                    wl[u] = __int_as_float(e.y);
                } else {
                    a = bcast_i(g_a, u);
                }
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    if (WIDE)
                        vload<VEC>(xv[u][t], x + (size_t)a * xs + fo[t]);
                    else
                        vload<VEC>(xv[u][t], reinterpret_cast<const float *>(
                                                 xb + (size_t)((uint32_t)a + fo_bytes[t])));
                }
            }
            // Consume phase, in entry order.  `left` = entries of this group before row r ends.
            int left = row_end - (jb + i0);
            const int m = min(UNROLL, n - i0);
            auto consume = [&](int u) {
                if (u == left) {
                    do flush_row(); while (row_end == jb + i0 + u);
                    left = row_end - (jb + i0);
                }
                const float wv = LDS ? wl[u] : bcast_f(g_w, u);
#pragma unroll
                for (int t = 0; t < NT; t++) {
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[t][v] = fmaf(wv, xv[u][t][v], acc[t][v]);
                }
            };
            if (m == UNROLL) {
#pragma unroll
                for (int u = 0; u < UNROLL; u++) consume(u);
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; u++)
                    if (u < m) consume(u);
            }
        }
    }
    while (r < r1) flush_row();   // rows whose end marker lies in this chunk after its last entry
    // the leading piece of a row that goes on in the next chunk (most chunks end where a row ends)
    if (r1 < R && j1 > uniform(off[r1])) {
        float *dst = partial + (size_t)k * F + f0;
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (act[t]) vstore<VEC>(dst + t * kWave * VEC, acc[t]);
    }
}

// Adds pieces src[first..last) (rows of F floats) to acc in order, fetching a
// few at a time so that the loads are in flight together.
template <int VEC, int NT>
__device__ __forceinline__ void add_pieces(float (&acc)[NT][VEC], const float *__restrict__ src, int first, int last,
                                           int F, int f0)
{
    constexpr int kBatch = VEC * NT >= 16 ? 2 : (VEC * NT >= 8 ? 4 : (VEC * NT >= 4 ? 8 : 16));
    for (int kb = first; kb < last; kb += kBatch) {
        // issue phase without branches: slots past `last` re-read the last piece, lanes past F
        // read offset 0; both are ignored below
        float v[kBatch][NT][VEC];
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            const float *p = src + (size_t)min(kb + b, last - 1) * F;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int f = f0 + t * kWave * VEC;
                vload<VEC>(v[b][t], p + (f < F ? f : 0));
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; b++)
            if (kb + b < last) {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    if (f0 + t * kWave * VEC < F) {
#pragma unroll
                        for (int i = 0; i < VEC; i++) acc[t][i] += v[b][t][i];
                    }
            }
    }
}

// A row cut into thousands of pieces (a hub with millions of entries) would
// make its last wavefront add them all one after the other.  Pieces are
// therefore pre-summed in groups of kGroup consecutive chunks: group g's
// wavefront adds, in order, the pieces of the row that continues past the end
// of the group (a suffix of the group's chunks) into group_sum[g].
constexpr int kGroup = kPlanGroup;

// `list` (ascending, *count entries) names the groups to look at; without one every group is.
template <int VEC, int NT>
__global__ __launch_bounds__(kSpmmThreads) void spmm_group_sums(const int32_t *__restrict__ off,
                                                                const float *__restrict__ partial,
                                                                float *__restrict__ group_sum,
                                                                const int2 *__restrict__ start,
                                                                const int32_t *__restrict__ list,
                                                                const int32_t *__restrict__ count, int R, int F,
                                                                int chunk, int nchunks)
{
    const int n = list ? uniform(count[0]) : (nchunks + kGroup - 1) / kGroup;
    const int stride = gridDim.x * kSpmmWaves;
    for (int i = blockIdx.x * kSpmmWaves + wave_in_block(); i < n; i += stride) {
        const int g = list ? uniform(list[i]) : i;
        const int kend = (g + 1) * kGroup;            // first chunk after the group
        if (kend >= nchunks) continue;                // the last group has no row continuing past it
        const int r = uniform(start[kend].x);         // row that owns the first item after the group
        if (r < 0 || r >= R) continue;
        const int s = uniform(off[r]);
        if (uniform(start[kend].y) <= s) continue;    // that chunk begins with the row: nothing continues
        const int a = max((int)(((int64_t)max(s, 0) + r) / chunk), g * kGroup);
        const int f0 = blockIdx.y * (kWave * VEC * NT) + lane_id() * VEC;
        float acc[NT][VEC];
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
        add_pieces<VEC, NT>(acc, partial, a, kend, F, f0);
        float *dst = group_sum + (size_t)g * F + f0;
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (f0 + t * kWave * VEC < F) vstore<VEC>(dst + t * kWave * VEC, acc[t]);
    }
}

// One wavefront per chunk b of `list` (or per chunk): if the first row of b started in an
// earlier chunk a and ends in b, out[row] = (pieces a .. b-1, in order) + out[row]; whole groups
// between a and b come from group_sum.
template <int VEC, int NT, bool EPI>
__global__ __launch_bounds__(kSpmmThreads) void spmm_fixup(const int32_t *__restrict__ off, float *__restrict__ out,
                                                           const float *__restrict__ partial,
                                                           const float *__restrict__ group_sum,
                                                           const int2 *__restrict__ start,
                                                           const int32_t *__restrict__ list,
                                                           const int32_t *__restrict__ count, int R, int F, int chunk,
                                                           int nchunks, RowFinish fin)
{
    const int n = list ? min(uniform(count[0]), nchunks) : nchunks;
    const int stride = gridDim.x * kSpmmWaves;
    for (int i = blockIdx.x * kSpmmWaves + wave_in_block(); i < n; i += stride) {
        const int k = list ? uniform(list[i]) : i;
        if (k < 0 || k >= nchunks) continue;
        const int r0 = uniform(start[k].x);
        const int r1 = uniform(start[k + 1].x);
        if (r0 < 0 || r0 >= R || r1 <= r0) continue;
        const int s = uniform(off[r0]);
        if (uniform(start[k].y) <= s) continue;       // the chunk begins with the row
        const int a = min((int)(((int64_t)max(s, 0) + r0) / chunk), k);
        const int lane = lane_id();
        const int f0 = blockIdx.y * (kWave * VEC * NT) + lane * VEC;
        float acc[NT][VEC], last[NT][VEC];
        float *dst = out + (size_t)r0 * F;
        // the row's last piece, as the chunk's wavefront stored it: fetched with the first pieces
        // rather than after them (one memory round trip less), added last as before
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            vload<VEC>(last[t], dst + (f < F ? f : 0));
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
        }
        const int ga = a / kGroup, gb = k / kGroup;
        if (ga == gb) {
            add_pieces<VEC, NT>(acc, partial, a, k, F, f0);
        } else if (gb - ga <= kSpmmInlineGroups) {
            // few groups: their sums are formed here, piece by piece from zero and then added in
            // order, exactly as spmm_group_sums and the branch below would
            for (int g = ga; g < gb; g++) {
                float gs[NT][VEC];
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) gs[t][v] = 0.f;
                add_pieces<VEC, NT>(gs, partial, max(a, g * kGroup), (g + 1) * kGroup, F, f0);
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[t][v] += gs[t][v];
            }
            add_pieces<VEC, NT>(acc, partial, gb * kGroup, k, F, f0);
        } else {
            // group ga's sum starts at piece a (the row continues past that group),
            // groups ga+1 .. gb-1 belong to the row entirely, the rest of gb is added piecewise
            add_pieces<VEC, NT>(acc, group_sum, ga, gb, F, f0);
            add_pieces<VEC, NT>(acc, partial, gb * kGroup, k, F, f0);
        }
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] += last[t][v];
        if constexpr (EPI) {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[t][v] *= fin.beta;
            if (fin.h) {
                float hv[NT][VEC];
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int f = f0 + t * kWave * VEC;
                    vload<VEC>(hv[t], fin.h + (size_t)r0 * fin.h_stride + (f < F ? f : 0));
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[t][v] = fmaf(fin.alpha, hv[t][v], acc[t][v]);
                }
            }
            if (fin.relu) {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[t][v] = fmaxf(acc[t][v], 0.f);
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (f0 + t * kWave * VEC < F) vstore<VEC>(dst + f0 + t * kWave * VEC, acc[t]);
    }
}

// out = beta * out + alpha * h, element-wise (the finish as a pass of its own, for the
// shapes the fused kernels do not cover).
__global__ void spmm_finish_rows(float *__restrict__ out, const float *__restrict__ h, int64_t n, int F,
                                 int h_stride, float beta, float alpha, int relu)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = fmaf(alpha, h ? h[h_stride ? i : i % F] : 0.f, beta * out[i]);
        out[i] = relu ? fmaxf(v, 0.f) : v;
    }
}

// ------------------------------------------------------------------ host ---
static int env_int(const char *name, int dflt)
{
    const char *s = getenv(name);
    if (!s || !*s) return dflt;
    int v = atoi(s);
    return v > 0 ? v : dflt;
}

// Items per wavefront: enough chunks to fill the 256 CUs many times over,
// few enough that the per-chunk partial row stays a small share of the work.
int spmm_chunk_for(int64_t M)
{
    // benchmark override, read once per process (the workspace query and the launch agree)
    static const int forced = env_int("JGAMD_SPMM_CHUNK", 0);
    if (forced) return forced < 16 ? 16 : (forced > 4096 ? 4096 : forced);
    int c = 512;
    while (c > 32 && M / c < 32768) c >>= 1;
    return c;
}

struct SpmmShape {
    int vec, nt, slabs, chunk, nchunks;
};

// narrow_slabs: one 64-float tile per wavefront and the other tiles in grid.y.  Workgroups are
// handed out with grid.x running fastest, so the whole matrix is walked for one 256-byte slab of
// the feature rows before the next slab starts: what the column-blocked product needs to keep
// the gathered block of x inside an L2.
static SpmmShape spmm_shape(int32_t R, int64_t E, int32_t F, bool aligned16, bool aligned8, bool narrow_slabs = false)
{
    SpmmShape s{};
    const int64_t M = (int64_t)R + E;
    s.chunk = spmm_chunk_for(M);
    s.nchunks = (int)ceil_div(M > 0 ? M : 1, s.chunk);
    s.vec = (F % 4 == 0 && aligned16) ? 4 : (F % 2 == 0 && aligned8) ? 2 : 1;
    if (narrow_slabs && F > kWave) {
        s.vec = 1;
        s.nt = 1;
        s.slabs = (int)ceil_div(F, kWave);
        return s;
    }
    // prefer the narrowest vector that still covers F with one tile per lane:
    // more lanes per row keeps every load instruction a full 64-lane access
    while (s.vec > 1 && F <= kWave * (s.vec / 2)) s.vec >>= 1;
    int per_tile = kWave * s.vec;
    int tiles = (int)ceil_div(F, per_tile);
    s.nt = tiles <= 8 ? tiles : 8;
    if (s.nt == 7) s.nt = 8;
    s.slabs = (int)ceil_div(F, per_tile * s.nt);
    return s;
}

static bool narrow_width(int32_t F) { return F == 1 || F == 2 || F == 4 || F == 8; }

// Row pieces and group sums; `with_starts` adds the chunk starts of a call that brings no plan.
static size_t spmm_scratch_bytes(int32_t R, int64_t E, int32_t F, bool with_starts)
{
    SpmmShape s = spmm_shape(R, E, F, true, true);
    const size_t wide = (with_starts ? carve_bytes((size_t)s.nchunks + 1, sizeof(int2)) : 0) +
                        carve_bytes((size_t)s.nchunks * (size_t)F, 4) +
                        carve_bytes((size_t)ceil_div(s.nchunks, kGroup) * (size_t)F, 4);
    const size_t narrow = narrow_width(F) ? entry_tiles_ws_bytes(E) : 0;
    return wide > narrow ? wide : narrow;
}

size_t spmm_ws_bytes(int32_t R, int64_t E, int32_t F) { return spmm_scratch_bytes(R, E, F, true); }

// What the host knows about the lists of a plan: -1 = nothing (the kernels read the lengths from
// the plan and loop over a grid of fixed size), 0 = empty (no launch), n > 0 = at most n entries.
struct PlanHints {
    int n_fix = -1, n_grp = -1;
};

static unsigned list_grid(int hint, int upper)
{
    const int64_t n = hint >= 0 ? (hint < upper ? hint : upper) : (upper < 8192 ? upper : 8192);
    return (unsigned)ceil_div(n > 0 ? n : 1, kSpmmWaves);
}

template <int VEC, int NT>
static void launch_spmm(const SpmmShape &s, const int32_t *off, const int32_t *idx, const float *w, const float *x,
                        float *out, float *partial, float *group_sum, const ChunkPlan &plan, const PlanHints &hints,
                        int R, int C, int E, int F, hipStream_t st, hipEvent_t k0 = nullptr, hipEvent_t k1 = nullptr,
                        const RowFinish *fin = nullptr, int x_stride = 0)
{
    dim3 grid((unsigned)ceil_div(s.nchunks, kSpmmWaves), (unsigned)s.slabs), block(kSpmmThreads);
    // gathers in flight per wavefront: bounded by the registers they land in
    constexpr int U = (VEC * NT >= 16) ? 4 : (VEC * NT >= 8 ? 8 : (VEC * NT >= 2 ? 16 : 32));
    if (k0) (void)hipEventRecord(k0, st);
    // 32-bit byte offsets reach every row of x when C*F*4 < 2^32.  (idx, w) staging: LDS or
    // registers (JGAMD_SPMM_STAGE=lds|reg overrides the default).
    static const int stage_env = [] {
        const char *e = getenv("JGAMD_SPMM_STAGE");
        return !e ? 0 : (e[0] == 'l' ? 1 : (e[0] == 'r' ? 2 : 0));
    }();
    const bool lds = stage_env ? stage_env == 1 : F >= kLdsStageMinWidth;
    const bool narrow = (uint64_t)C * (uint64_t)(x_stride ? x_stride : F) * 4u < ((uint64_t)1 << 32);
    // the fused row finish exists for 32-bit offsets only; wide shapes finish in a pass of their own
    const bool fused = fin && narrow;
    const RowFinish none{1.f, 0.f, nullptr, 0, 0, 0};
    RowFinish f = fused ? *fin : none;
    f.x_stride = x_stride;
#define JG_GO(W, L, P)                                                                                              \
    hipLaunchKernelGGL((spmm_merge<VEC, NT, U, W, L, P>), grid, block, 0, st, off, idx, w, x, out, partial,         \
                       plan.start, R, C, E, F, s.nchunks, f)
    if (fused && lds) JG_GO(false, true, true);
    else if (fused) JG_GO(false, false, true);
    else if (narrow && lds) JG_GO(false, true, false);
    else if (narrow) JG_GO(false, false, false);
    else if (lds) JG_GO(true, true, false);
    else JG_GO(true, false, false);
#undef JG_GO
    if (k1) (void)hipEventRecord(k1, st);
    // pieces of rows cut across chunks: only rows longer than half a chunk ever are
    const int ngroups = (int)ceil_div(s.nchunks, kGroup);
    const bool listed = plan.fix != nullptr;
    const int n_grp = listed ? hints.n_grp : -1, n_fix = listed ? hints.n_fix : -1;
    if (ngroups > 1 && n_grp != 0 && n_fix != 0)
        hipLaunchKernelGGL((spmm_group_sums<VEC, NT>),
                           dim3(listed ? list_grid(n_grp, ngroups) : (unsigned)ceil_div(ngroups, kSpmmWaves),
                                (unsigned)s.slabs),
                           block, 0, st, off, partial, group_sum, plan.start, plan.grp, plan.counts + 1, R, F, s.chunk,
                           s.nchunks);
    if (n_fix != 0) {
        const dim3 fgrid(listed ? list_grid(n_fix, s.nchunks) : grid.x, (unsigned)s.slabs);
        if (fused)
            hipLaunchKernelGGL((spmm_fixup<VEC, NT, true>), fgrid, block, 0, st, off, out, partial, group_sum,
                               plan.start, plan.fix, plan.counts, R, F, s.chunk, s.nchunks, f);
        else
            hipLaunchKernelGGL((spmm_fixup<VEC, NT, false>), fgrid, block, 0, st, off, out, partial, group_sum,
                               plan.start, plan.fix, plan.counts, R, F, s.chunk, s.nchunks, f);
    }
    if (fin && !fused) {
        const int64_t n = (int64_t)R * F;
        hipLaunchKernelGGL(spmm_finish_rows, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, out, fin->h, n, F,
                           fin->h_stride, fin->beta, fin->alpha, fin->relu);
    }
}

}  // namespace jg

using namespace jg;

static int32_t check_spmm_sizes(int32_t R, int64_t E, int32_t F)
{
    if (R < 0 || E < 0 || F < 0) return fail(JGAMD_ERR_SIZE, "spmm_csx: negative size");
    if ((int64_t)R + E >= ((int64_t)1 << 31) - 4096)
        return fail(JGAMD_ERR_SIZE, "spmm_csx: R + E = %lld does not fit int32", (long long)((int64_t)R + E));
    return 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_workspace(int32_t R, int64_t E, int32_t F, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "spmm_csx_workspace: bytes is NULL");
    if (int32_t rc = check_spmm_sizes(R, E, F)) return rc;
    *bytes = (R == 0 || F == 0) ? 0 : spmm_ws_bytes(R, E, F);
    return 0;
}

// plan == nullptr: the chunk starts are computed into the workspace first (one more launch) and
// every chunk and group is looked at by the fix-up kernels.
static int32_t spmm_call(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out,
                         int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, void *stream,
                         hipEvent_t k0, hipEvent_t k1, const RowFinish *fin = nullptr, bool narrow_slabs = false,
                         int x_stride = 0, const void *plan = nullptr, const void *tiles = nullptr,
                         PlanHints hints = PlanHints(), bool planned_call = false)
{
    if (int32_t rc = check_spmm_sizes(R, E, F)) return rc;
    if (C < 0) return fail(JGAMD_ERR_SIZE, "spmm_csx: negative C");
    if (R == 0 || F == 0) return 0;
    if (!off || !out) return fail(JGAMD_ERR_NULL, "spmm_csx: off/out is NULL");
    if (E > 0 && !x) return fail(JGAMD_ERR_NULL, "spmm_csx: x is NULL with E > 0");
    if (E > 0 && C == 0) return fail(JGAMD_ERR_SIZE, "spmm_csx: E > 0 entries but x has no rows");
    if ((((uintptr_t)x | (uintptr_t)out) & 3) != 0) return fail(JGAMD_ERR_ALIGN, "spmm_csx: x/out not 4-byte aligned");
    // Rows of 1, 2, 4 or 8 floats: a lane per entry and a segmented scan instead of a wavefront
    // per entry (JGAMD_SPMM_NARROW=merge keeps the wide-row kernels).  Entries must tile [0, E).
    static const bool narrow_off = [] {
        const char *e = getenv("JGAMD_SPMM_NARROW");
        return e && e[0] == 'm';
    }();
    const bool narrow_route = !fin && !k0 && !narrow_off && x_stride == 0 && E > 0 && narrow_width(F) &&
                              narrow_spmm_supported(F, x) && (tiles || !plan);
    // a planned call that brought the tile plan only: the tile kernels must be able to take it
    if (planned_call && !plan && !narrow_route)
        return fail(JGAMD_ERR_NULL, "spmm_csx_planned: this product (F=%d%s) takes the chunk kernels: pass the chunk plan, "
                    "not only the tile plan", F, fin ? ", with a row finish" : "");
    const size_t need = narrow_route ? entry_tiles_ws_bytes(E) : spmm_scratch_bytes(R, E, F, plan == nullptr);
    if (!ws || ws_bytes < need)
        return fail(JGAMD_ERR_WORKSPACE, "spmm_csx: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "spmm_csx: workspace not 256-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (narrow_route) {
        narrow_spmm_enqueue(off, idx, w, x, out, R, C, E, F, ws, st, tiles);
        return launch_status("spmm_csx");
    }

    // Rows of two or more whole 64-float slabs are walked slab by slab as well: an L2 then holds the
    // hot rows' 256-byte pieces of one slab instead of their whole rows, i.e. more hot rows, and the
    // (index, weight) arrays read once more per slab are small next to the gathers.  Measured on
    // V = 1M / E = 17M: F = 128 0.99 -> 0.98 ms, F = 256 2.12 -> 1.87 ms, F = 512 4.49 -> 3.64 ms;
    // V = 2.45M / E = 126M: F = 256 13.0 -> 12.3 ms.  Slabs of 128 or 256 floats gain less, and a
    // partial last slab loses (F = 100: 0.98 -> 1.34 ms), so other widths keep whole rows.
    if (F >= 2 * kWave && F % kWave == 0) narrow_slabs = true;
    // h is read with x's vector width: its alignment counts too
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)out | (uintptr_t)(fin ? fin->h : nullptr);
    const SpmmShape s = spmm_shape(R, E, F, (bits & 15) == 0, (bits & 7) == 0, narrow_slabs);
    Carver carve(ws);
    ChunkPlan pv{};
    if (plan) {
        pv = chunk_plan_view(JGAMD_PLAN_SPMM, R, E, plan);
    } else {
        int2 *start = carve.take<int2>((size_t)s.nchunks + 1);
        chunk_starts_enqueue(off, R, E, s.chunk, s.nchunks, start, st);
        pv.start = start;
        pv.chunk = s.chunk;
        pv.nchunks = s.nchunks;
    }
    float *partial = carve.take<float>((size_t)s.nchunks * (size_t)F);
    float *group_sum = carve.take<float>((size_t)ceil_div(s.nchunks, kGroup) * (size_t)F);

#define JG_CASE(V, N)                                                                                \
    if (s.vec == V && s.nt == N) {                                                                   \
        launch_spmm<V, N>(s, off, idx, w, x, out, partial, group_sum, pv, hints, R, C, (int)E, F, st, k0, k1, fin, x_stride); \
        return launch_status("spmm_csx");                                                            \
    }
#define JG_CASES(V) JG_CASE(V, 1) JG_CASE(V, 2) JG_CASE(V, 3) JG_CASE(V, 4) JG_CASE(V, 5) JG_CASE(V, 6) JG_CASE(V, 8)
    JG_CASES(1)
    JG_CASES(2)
    JG_CASES(4)
#undef JG_CASES
#undef JG_CASE
    return fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx: no kernel for F=%d (vec %d, tiles %d)", F, s.vec, s.nt);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx(const int32_t *off, const int32_t *idx,
                                                                         const float *w, const float *x, float *out,
                                                                         int32_t R, int32_t C, int64_t E, int32_t F,
                                                                         void *ws, size_t ws_bytes, void *stream)
{
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, stream, nullptr, nullptr);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_axpby(
    const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, float beta, float alpha,
    const float *h, int32_t h_rows, int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes,
    void *stream)
{
    if (h && (((uintptr_t)h & 3) != 0)) return fail(JGAMD_ERR_ALIGN, "spmm_csx_axpby: h not 4-byte aligned");
    if (h && h_rows != 1 && h_rows != R)
        return fail(JGAMD_ERR_SIZE, "spmm_csx_axpby: h has %d rows, expected %d or 1", h_rows, R);
    const RowFinish fin{beta, alpha, alpha != 0.f ? h : nullptr, h_rows == 1 ? 0 : F, 0, 0};
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, stream, nullptr, nullptr, &fin);
}

// The product with the partition of a plan (jgamd_csx_plan): no per-call search of the chunk
// starts, and the piece kernels run over the plan's lists only.
extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_planned(
    const void *plan, const void *tiles, int32_t n_fix, int32_t n_grp, const int32_t *off, const int32_t *idx,
    const float *w, const float *x, float *out, float beta, float alpha, const float *h, int32_t h_rows,
    int32_t flags, int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, void *stream)
{
    // bits 8 and up: floats between the rows of x when they are padded apart (0 = F)
    const int32_t x_stride = flags >> 8;
    flags &= 0xff;
    if (flags & ~JGAMD_ROW_RELU) return fail(JGAMD_ERR_SIZE, "spmm_csx_planned: unknown flags %d", flags);
    if (x_stride != 0 && (x_stride < F || (x_stride & 3) != 0))
        return fail(JGAMD_ERR_SIZE, "spmm_csx_planned: x row stride %d must be a multiple of 4 floats and at least F=%d",
                    x_stride, F);
    if (x_stride != 0 && !plan)
        return fail(JGAMD_ERR_NULL, "spmm_csx_planned: rows of x padded apart take the chunk kernels: pass the chunk plan");
    if (!plan && !tiles) return fail(JGAMD_ERR_NULL, "spmm_csx_planned: plan and tiles are both NULL");
    if (!plan && !narrow_width(F))
        return fail(JGAMD_ERR_NULL, "spmm_csx_planned: rows of %d floats need the chunk plan, not the tile plan", F);
    if ((((uintptr_t)plan | (uintptr_t)tiles) & 255) != 0)
        return fail(JGAMD_ERR_ALIGN, "spmm_csx_planned: plan not 256-byte aligned");
    if (h && (((uintptr_t)h & 3) != 0)) return fail(JGAMD_ERR_ALIGN, "spmm_csx_planned: h not 4-byte aligned");
    if (h && h_rows != 1 && h_rows != R)
        return fail(JGAMD_ERR_SIZE, "spmm_csx_planned: h has %d rows, expected %d or 1", h_rows, R);
    PlanHints hints;
    hints.n_fix = n_fix < 0 ? -1 : n_fix;
    hints.n_grp = n_grp < 0 ? -1 : n_grp;
    const bool plain = beta == 1.f && (alpha == 0.f || !h) && flags == 0;
    const RowFinish fin{beta, alpha, alpha != 0.f ? h : nullptr, h_rows == 1 ? 0 : F, 0, (flags & JGAMD_ROW_RELU) ? 1 : 0};
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, stream, nullptr, nullptr, plain ? nullptr : &fin,
                     false, x_stride == F ? 0 : x_stride, plan, tiles, hints, true);
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_planned_workspace(int32_t R, int64_t E,
                                                                                           int32_t F, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "spmm_csx_planned_workspace: bytes is NULL");
    if (int32_t rc = check_spmm_sizes(R, E, F)) return rc;
    *bytes = (R == 0 || F == 0) ? 0 : spmm_scratch_bytes(R, E, F, false);
    return 0;
}

namespace jg {
int32_t spmm_enqueue(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out, int32_t R,
                     int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, hipStream_t s, const void *tiles)
{
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, s, nullptr, nullptr, nullptr, false, 0, nullptr,
                     tiles);
}
int32_t spmm_enqueue_slabs(const int32_t *off, const int32_t *idx, const float *w, const float *x, float *out,
                           int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, hipStream_t s,
                           hipEvent_t k0, hipEvent_t k1, int x_stride)
{
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, s, k0, k1, nullptr, true, x_stride);
}
}  // namespace jg

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_timed(
    const void *plan, int32_t n_fix, int32_t n_grp, const int32_t *off, const int32_t *idx, const float *w,
    const float *x, float *out, int32_t R, int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes, void *stream,
    int32_t iters, float *kernel_ms, float *call_ms)
{
    if (((uintptr_t)plan & 255) != 0) return fail(JGAMD_ERR_ALIGN, "spmm_csx_timed: plan not 256-byte aligned");
    PlanHints hints;
    hints.n_fix = n_fix < 0 ? -1 : n_fix;
    hints.n_grp = n_grp < 0 ? -1 : n_grp;
    if (iters < 1 || iters > 4096) return fail(JGAMD_ERR_SIZE, "spmm_csx_timed: iters must be in [1, 4096]");
    if (!kernel_ms || !call_ms) return fail(JGAMD_ERR_NULL, "spmm_csx_timed: NULL result pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipEvent_t ev[4];
    for (auto &e : ev)
        if (hipEventCreate(&e) != hipSuccess) return fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx_timed: hipEventCreate failed");
    double ksum = 0, csum = 0;
    int32_t rc = 0;
    for (int i = 0; i < iters && rc == 0; i++) {
        (void)hipEventRecord(ev[0], st);
        rc = spmm_call(off, idx, w, x, out, R, C, E, F, ws, ws_bytes, stream, ev[1], ev[2], nullptr, false, 0, plan,
                       nullptr, hints);
        (void)hipEventRecord(ev[3], st);
        if (hipEventSynchronize(ev[3]) != hipSuccess && rc == 0)
            rc = fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx_timed: hipEventSynchronize failed");
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

// ---- the product without a workspace argument --------------------------------
// For callers that can neither allocate nor own a workspace: chunk_row, partial
// and group_sum live in a fixed device array that is part of the code object.
// Every GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends; the array's name is only a handle on the
// host, so its device address is resolved once per device and kept.
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, once known

int32_t static_scratch(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int32_t)e, "spmm_csx_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(JGAMD_ERR_UNSUPPORTED, "spmm_csx_noalloc: device %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return fail(e != hipSuccess ? (int32_t)e : JGAMD_ERR_UNSUPPORTED,
                        "spmm_csx_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int32_t jgamd_spmm_csx_noalloc(const int32_t *off, const int32_t *idx,
                                                                                 const float *w, const float *x,
                                                                                 float *out, int32_t R, int32_t C,
                                                                                 int64_t E, int32_t F, void *stream)
{
    if (int32_t rc = check_spmm_sizes(R, E, F)) return rc;
    if (R == 0 || F == 0) return 0;
    const size_t need = spmm_ws_bytes(R, E, F);
    if (need > kStaticScratchBytes)
        return fail(JGAMD_ERR_SIZE,
                    "spmm_csx_noalloc: R=%d E=%lld F=%d needs %zu bytes of scratch, the fixed array holds %zu; "
                    "use jgamd_spmm_csx with a workspace",
                    R, (long long)E, F, need, kStaticScratchBytes);
    void *ws = nullptr;
    if (int32_t rc = static_scratch(&ws)) return rc;
    // Nothing in the scratch has to start at zero: every word a kernel reads was written by an
    // earlier kernel of the same call (chunk rows; a piece is read only for chunks that stored one).
    return spmm_call(off, idx, w, x, out, R, C, E, F, ws, kStaticScratchBytes, stream, nullptr, nullptr);
}
