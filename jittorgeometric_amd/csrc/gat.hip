// Fused GAT layer core for gfx950: attention logits, edge softmax and the
// weighted aggregation in one pass over the CSC arrays; backward in one pass
// over the transposed (CSR) arrays.
//
// Reference chain being replaced (nn/conv/gat_conv.py:61-83):
//   e = [h[src] | h[dst]]  (two [E,C] copies + concat)      scattertoedge_op.cc
//   z = leaky_relu(e @ a, 0.2)                               [E,1]
//   alpha = edge softmax of z per destination                edgesoftmax_op.cc
//   out[dst] = sum alpha * h[src]                            edgetovertex_op.cc
// With a = [a_src | a_dst]:  e @ a = a_src.h[src] + a_dst.h[dst] = el[src] + er[dst],
// two per-node scalars per head, so no [E,C] tensor is ever materialised.
//
// Work split and lane layout are those of the SpMM kernel: merge-path chunks
// of (row ends + entries) per wavefront, features across lanes.  The softmax
// is carried as a running (max, sum) per lane and head, rescaling the
// accumulator when the max grows; a row cut by a chunk boundary leaves its
// unnormalised (acc, max, sum) piece in scratch and a second kernel merges
// the pieces in order.  No float atomics anywhere.
//
// Backward.  With z_e = el[src] + er[dst], alpha the softmax of lrelu(z) over a
// destination's in-edges and out[c] = sum_e alpha_e h[src_e]:
//   dz_e    = lrelu'(z_e) alpha_e (g[c].h[src_e] - g[c].out[c])
//   g_h[r]  = sum_{e out of r} alpha_e g[dst_e] + a_src g_el[r] + a_dst g_er[r]
//   g_el[r] = sum_{e out of r} dz_e          g_er[c] = sum_{e into c} dz_e
// One pass over the transposed arrays (rows = sources) gives the first two sums.
// The destination-side sum needs no pass over the edges at all: with lrelu' in
// {1, slope} and the alpha of a destination adding up to one,
//   g_er[c] = (1 - slope) (g[c].pos[c] - (g[c].out[c]) spos[c]),
//   pos[c] = sum_{e into c, z_e > 0} alpha_e h[src_e],  spos[c] = sum_{z_e > 0} alpha_e,
// two more accumulators of the forward pass, which gathers those rows anyway.
// g_er is therefore known per node before the pass over the sources starts, and
// that pass writes g_h complete; the gradients of a_src and a_dst are sums over
// the nodes of g_el[r] h[r] and g_er[r] h[r], accumulated by the same pass (the
// h row of the current source is in registers) per workgroup and added up in a
// fixed order by two small kernels.
#include <math.h>
#include <stdlib.h>

#include "common.h"

namespace jg {

constexpr int kGatThreads = 256;
constexpr int kGatWaves = kGatThreads / kWave;
// gathers in flight per wavefront, bounded by the registers they land in
constexpr int gat_unroll(int regs) { return regs >= 16 ? 2 : regs >= 8 ? 4 : 8; }

template <int VEC> struct GVec;
template <> struct GVec<1> { using type = float; };
template <> struct GVec<2> { using type = float2; };
template <> struct GVec<4> { using type = float4; };

template <int VEC> __device__ __forceinline__ void gload(float (&d)[VEC], const float *p)
{
    using V = typename GVec<VEC>::type;
    const V v = *reinterpret_cast<const V *>(p);
    const float *f = reinterpret_cast<const float *>(&v);
#pragma unroll
    for (int i = 0; i < VEC; i++) d[i] = f[i];
}
template <int VEC> __device__ __forceinline__ void gstore(float *p, const float (&s)[VEC])
{
    using V = typename GVec<VEC>::type;
    V v;
    float *f = reinterpret_cast<float *>(&v);
#pragma unroll
    for (int i = 0; i < VEC; i++) f[i] = s[i];
    *reinterpret_cast<V *>(p) = v;
}

__device__ __forceinline__ float lrelu(float z, float slope) { return z > 0.f ? z : slope * z; }

// exp for arguments <= 0 in the per-edge loops: the hardware exp2 on x*log2(e), relative error
// about |x| * 2^-23.  A term with large |x| is a correspondingly tiny share of its softmax sum
// (|x| = 16 -> 1e-7 of the largest term), so the weights stay well inside 1e-6 relative; the
// library expf costs ~20 VALU instructions per call and made these kernels VALU-bound.
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

// el[v,k] = a_src[k,:].h[v,k,:], er[v,k] = a_dst[k,:].h[v,k,:]
// Generic form: one thread per (node, head) walks the head's D values.
__global__ void gat_node_scores(const float *__restrict__ h, const float *__restrict__ a_src,
                                const float *__restrict__ a_dst, float *__restrict__ el, float *__restrict__ er,
                                int64_t VH, int H, int D)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= VH) return;
    const int k = (int)(i % H);
    const float *row = h + i * D;
    const float *as = a_src + (int64_t)k * D, *ad = a_dst + (int64_t)k * D;
    float s = 0.f, d = 0.f;
    for (int j = 0; j < D; j++) {
        const float v = row[j];
        s = fmaf(v, as[j], s);
        d = fmaf(v, ad[j], d);
    }
    el[i] = s;
    er[i] = d;
}

// Coalesced form for D = 4*lph with lph a power of two <= 64: the array is
// read as one stream of float4, lph consecutive lanes hold one (node, head)
// and fold their partial dot products with xor-shuffles.
__global__ __launch_bounds__(256) void gat_node_scores_vec(const float4 *__restrict__ h,
                                                           const float4 *__restrict__ a_src,
                                                           const float4 *__restrict__ a_dst, float *__restrict__ el,
                                                           float *__restrict__ er, int64_t n4, int H, int lph)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // float4 index into h
    float s = 0.f, d = 0.f;
    if (i < n4) {
        const float4 v = h[i];
        const int64_t vh = i / lph;                 // (node, head) pair
        const int q = (int)(vh % H) * lph + (int)(i % lph);
        const float4 as = a_src[q], ad = a_dst[q];
        s = v.x * as.x + v.y * as.y + v.z * as.z + v.w * as.w;
        d = v.x * ad.x + v.y * ad.y + v.z * ad.z + v.w * ad.w;
    }
    for (int o = 1; o < lph; o <<= 1) {
        s += __shfl_xor(s, o, kWave);
        d += __shfl_xor(d, o, kWave);
    }
    if (i < n4 && i % lph == 0) {
        el[i / lph] = s;
        er[i / lph] = d;
    }
}

// The value lane CTRL (0x00, 0x55, 0xAA, 0xFF = 0, 1, 2, 3) of every quad holds, in all four lanes.
template <int CTRL> __device__ __forceinline__ float quad_lane(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// Sum of v over aligned groups of `lanes` consecutive lanes (a power of two), left in every
// lane of the group.  Up to 16 lanes the exchanges are DPP modifiers on the adds (quad
// permutes, then the half-row and row mirrors); only 32 and 64 go through the LDS crossbar.
template <int CTRL> __device__ __forceinline__ float dpp_add(float v)
{
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(moved);
}
__device__ __forceinline__ float lane_group_sum(float v, int lanes)
{
    if (lanes >= 2) v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    if (lanes >= 4) v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    if (lanes >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
    if (lanes >= 16) v = dpp_add<0x140>(v);  // row_mirror
    if (lanes >= 32) v += __shfl_xor(v, 16, kWave);
    if (lanes >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

// ----------------------------------------------------------------- forward ---
// POS: also accumulate, per destination, the share of the softmax that lies on positive
// logits -- pos[r,:] = sum_{z_e > 0} alpha_e h[src_e], spos[r,k] = sum_{z_e > 0} alpha_e --
// which is what the backward pass needs for the destination-side logit gradient.  The two
// accumulators ride along with (acc, l): same rescaling, same pieces, same fix-up.
struct GatPieces {
    float *vec, *mx, *sum;     // [n, F], [n, H], [n, H]
    float *pvec, *psum;        // the positive-logit share, POS only
};

// SCORES (one tile per lane, lph = D / VEC lanes per head, a power of two): the caller wants no
// el / er arrays (no backward pass follows), and the two dot products are taken where the rows
// pass through registers anyway -- a_src.h[src] from every gathered row, a_dst.h[r] from the
// destination's own row, fetched one row ahead as er is otherwise -- folded over the head's
// lanes with DPP adds.  The pass over h that computes the two arrays (a sixth of the forward
// time at 169k nodes of 8 x 16 features) and one 4-byte gather per entry then fall away.
template <int VEC, int NT, bool POS, bool SCORES = false>
__global__ __launch_bounds__(kGatThreads) void gat_fwd_merge(
    const int32_t *__restrict__ off, const int32_t *__restrict__ idx, const float *__restrict__ h,
    const float *__restrict__ el, const float *__restrict__ er, float slope, float *__restrict__ out,
    float *__restrict__ smax, float *__restrict__ ssum, float *__restrict__ pos, float *__restrict__ spos,
    GatPieces piece, const int2 *__restrict__ start, int R, int E, int H, int D, int nchunks,
    const float *__restrict__ a_src = nullptr, const float *__restrict__ a_dst = nullptr, int lph = 0)
{
    static_assert(!SCORES || (NT == 1 && !POS), "scores in the kernel: one tile, inference only");
    constexpr int kGatUnroll = gat_unroll(VEC * NT * (POS ? 2 : 1));
    const int k = blockIdx.x * kGatWaves + wave_in_block();
    if (k >= nchunks) return;
    const int lane = lane_id();
    const int F = H * D;
    const int f0 = lane * VEC;
    bool act[NT], lead[NT];
    int head[NT], fo[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int f = f0 + t * kWave * VEC;
        act[t] = f < F;
        head[t] = act[t] ? f / D : 0;
        lead[t] = act[t] && (f % D == 0);
        fo[t] = act[t] ? f : 0;
    }
    // the chunk runs from (row, entry) = start[k] to start[k + 1], clamped against malformed offsets
    const int2 s0 = start[k], s1 = start[k + 1];
    const int r1 = min(max(uniform(s1.x), 0), R);
    int r = min(max(uniform(s0.x), 0), r1);
    const int j0 = min(max(uniform(s0.y), 0), E);
    const int j1 = min(uniform(s1.y), E);
    // the first row of the chunk began in an earlier chunk: its piece stays unnormalised
    bool continued = (r < R) && (uniform(off[r]) < j0);

    int rb = r;
    int ends = (rb + lane < R) ? off[rb + 1 + lane] : 0x7fffffff;
    int row_end = bcast_i(ends, 0);

    // er of the current row and, already on its way, of the next one: a row end must not
    // wait for a fresh load (rows are a handful of entries long)
    float m[NT], l[NT], acc[NT][VEC], er_r[NT], er_next[NT];
    float lp[POS ? NT : 1], pacc[POS ? NT : 1][POS ? VEC : 1];
    // SCORES: this lane's slices of a_src / a_dst, and the next destination's own slice of h
    float as_[SCORES ? NT : 1][SCORES ? VEC : 1], ad_[SCORES ? NT : 1][SCORES ? VEC : 1];
    float hr_next[SCORES ? NT : 1][SCORES ? VEC : 1];
    if constexpr (SCORES) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < VEC; v++) {
                as_[t][v] = a_src[fo[t] + v];
                ad_[t][v] = a_dst[fo[t] + v];
            }
    }
    auto fetch_row = [&](int row) {
        const size_t rn = (size_t)min(row, R - 1);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if constexpr (SCORES) gload<VEC>(hr_next[t], h + rn * F + fo[t]);
            else er_next[t] = er[rn * H + head[t]];
        }
    };
    auto fetch_next = [&]() { fetch_row(r + 1); };
    auto reset = [&]() {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            m[t] = -INFINITY;
            l[t] = 0.f;
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
            if constexpr (POS) {
                lp[t] = 0.f;
#pragma unroll
                for (int v = 0; v < VEC; v++) pacc[t][v] = 0.f;
            }
            if constexpr (SCORES) {
                float d = 0.f;
#pragma unroll
                for (int v = 0; v < VEC; v++) d = fmaf(hr_next[t][v], ad_[t][v], d);
                er_r[t] = lane_group_sum(d, lph);      // every lane runs this: row ends are wave-uniform
            } else {
                er_r[t] = er_next[t];
            }
        }
        fetch_next();
    };
    fetch_row(r);
    reset();

    auto flush_row = [&]() {
        const size_t base = (size_t)r * F + f0;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if (act[t]) {
                float o[VEC];
                const float inv = continued ? 1.f : (l[t] > 0.f ? 1.f / l[t] : 0.f);
#pragma unroll
                for (int v = 0; v < VEC; v++) o[v] = acc[t][v] * inv;
                gstore<VEC>(out + base + t * kWave * VEC, o);
                if constexpr (POS) {
#pragma unroll
                    for (int v = 0; v < VEC; v++) o[v] = pacc[t][v] * inv;
                    gstore<VEC>(pos + base + t * kWave * VEC, o);
                }
                if (lead[t]) {
                    smax[(size_t)r * H + head[t]] = m[t];
                    ssum[(size_t)r * H + head[t]] = l[t];
                    if constexpr (POS) spos[(size_t)r * H + head[t]] = lp[t] * inv;
                }
            }
        }
        continued = false;
        r++;
        if (r - rb == kWave) {
            rb = r;
            ends = (rb + lane < R) ? off[rb + 1 + lane] : 0x7fffffff;
        }
        row_end = bcast_i(ends, r - rb);
        reset();
    };

    for (int jb = j0; jb < j1; jb += kWave) {
        const int n = min(kWave, j1 - jb);
        int my_c = -1;
        if (lane < n) {
            my_c = idx[jb + lane];
            if ((unsigned)my_c >= (unsigned)R) my_c = -1;
        }
        for (int i0 = 0; i0 < n; i0 += kGatUnroll) {
            // issue phase: straight-line, no branches or lane predicates (slots past n and
            // dropped entries read row 0; lanes past F read the start of the row)
            float xv[kGatUnroll][NT][VEC], sv[kGatUnroll][NT];
#pragma unroll
            for (int u = 0; u < kGatUnroll; u++) {
                const int c = max(bcast_i(my_c, (i0 + u) & (kWave - 1)), 0);
                const float *src = h + (size_t)c * F;
                const float *sl = el + (size_t)c * H;
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    gload<VEC>(xv[u][t], src + fo[t]);
                    if constexpr (!SCORES) sv[u][t] = sl[head[t]];
                }
            }
#pragma unroll
            for (int u = 0; u < kGatUnroll; u++) {
                if (i0 + u < n) {
                    const int jj = jb + i0 + u;
                    while (jj == row_end && r < r1) flush_row();
                    const int c = bcast_i(my_c, i0 + u);
                    if (c >= 0) {
                        if constexpr (SCORES) {
                            // all lanes take part (c is wave-uniform): the adds read neighbouring lanes
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                float d = 0.f;
#pragma unroll
                                for (int v = 0; v < VEC; v++) d = fmaf(xv[u][t][v], as_[t][v], d);
                                sv[u][t] = lane_group_sum(d, lph);
                            }
                        }
#pragma unroll
                        for (int t = 0; t < NT; t++)
                            if (act[t]) {
                                // One of the two factors of the running softmax is always 1: the old sums
                                // shrink by e when the entry raises the maximum, else the entry weighs e
                                // (e = 0 on a row's first entry, m = -inf).  One exp per entry, and the
                                // accumulators are scaled in place before the entry is added, which keeps
                                // each of them in its register.
                                const float z = sv[u][t] + er_r[t];
                                const bool above = z > 0.f;
                                const float s = above ? z : slope * z;
                                const float d = s - m[t];
                                const float e = fast_exp(-fabsf(d));
                                const bool up = d > 0.f;
                                const float sc = up ? e : 1.f, p = up ? 1.f : e;
                                m[t] = up ? s : m[t];
                                l[t] = fmaf(l[t], sc, p);
#pragma unroll
                                for (int v = 0; v < VEC; v++) acc[t][v] = fmaf(p, xv[u][t][v], __fmul_rn(acc[t][v], sc));
                                if constexpr (POS) {
                                    const float pp = above ? p : 0.f;
                                    lp[t] = fmaf(lp[t], sc, pp);
#pragma unroll
                                    for (int v = 0; v < VEC; v++)
                                        pacc[t][v] = fmaf(pp, xv[u][t][v], __fmul_rn(pacc[t][v], sc));
                                }
                            }
                    }
                }
            }
        }
    }
    while (r < r1) flush_row();
    if (r1 < R && j1 > uniform(off[r1])) {     // the leading piece of a row that goes on in the next chunk
        const size_t base = (size_t)k * F + f0;
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (act[t]) {
                gstore<VEC>(piece.vec + base + t * kWave * VEC, acc[t]);
                if constexpr (POS) gstore<VEC>(piece.pvec + base + t * kWave * VEC, pacc[t]);
                if (lead[t]) {
                    piece.mx[(size_t)k * H + head[t]] = m[t];
                    piece.sum[(size_t)k * H + head[t]] = l[t];
                    if constexpr (POS) piece.psum[(size_t)k * H + head[t]] = lp[t];
                }
            }
    }
}

// Running softmax state of one row piece per lane: acc (unnormalised), max, sum, and with POS
// the positive-logit share of both.
template <int VEC, int NT, bool POS> struct SoftState {
    float M[NT], L[NT], acc[NT][VEC];
    float LP[POS ? NT : 1], pacc[POS ? NT : 1][POS ? VEC : 1];
    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            M[t] = -INFINITY;
            L[t] = 0.f;
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
            if constexpr (POS) {
                LP[t] = 0.f;
#pragma unroll
                for (int v = 0; v < VEC; v++) pacc[t][v] = 0.f;
            }
        }
    }
    // Merges pieces first..last-1 of p in order; a few pieces are fetched at a time so that
    // their loads overlap.
    __device__ __forceinline__ void merge(const GatPieces &p, int first, int last, int F, int H, int D, int f0)
    {
        // pieces in flight: a long row's merge is a chain of such batches, one memory latency each
        constexpr int kRegs = VEC * NT * (POS ? 2 : 1);
        constexpr int kBatch = kRegs >= 16 ? 2 : (kRegs >= 8 ? 4 : (kRegs >= 4 ? 8 : 16));
        for (int kb = first; kb < last; kb += kBatch) {
            float x[kBatch][NT][VEC], pm[kBatch][NT], pl[kBatch][NT];
            float px[POS ? kBatch : 1][POS ? NT : 1][POS ? VEC : 1], pp[POS ? kBatch : 1][POS ? NT : 1];
            // issue phase without branches: slots past `last` re-read the last piece and
            // lanes past F read offset 0; both are ignored below
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                const size_t pc = (size_t)min(kb + b, last - 1);
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int f = f0 + t * kWave * VEC;
                    const int fc = f < F ? f : 0;
                    gload<VEC>(x[b][t], p.vec + pc * F + fc);
                    pm[b][t] = p.mx[pc * H + fc / D];
                    pl[b][t] = p.sum[pc * H + fc / D];
                    if constexpr (POS) {
                        gload<VEC>(px[b][t], p.pvec + pc * F + fc);
                        pp[b][t] = p.psum[pc * H + fc / D];
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < kBatch; b++)
                if (kb + b < last) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        const int f = f0 + t * kWave * VEC;
                        if (f < F && pl[b][t] > 0.f) {
                            const float mn = fmaxf(M[t], pm[b][t]);
                            const float so = expf(M[t] - mn), si = expf(pm[b][t] - mn);
                            L[t] = L[t] * so + pl[b][t] * si;
#pragma unroll
                            for (int v = 0; v < VEC; v++) acc[t][v] = acc[t][v] * so + x[b][t][v] * si;
                            if constexpr (POS) {
                                LP[t] = LP[t] * so + pp[b][t] * si;
#pragma unroll
                                for (int v = 0; v < VEC; v++) pacc[t][v] = pacc[t][v] * so + px[b][t][v] * si;
                            }
                            M[t] = mn;
                        }
                    }
                }
        }
    }
};

// Pieces of a long row are pre-merged in groups of kGatGroup consecutive
// chunks (see spmm_group_sums): group g's wavefront merges the pieces of the
// row that continues past the end of the group.
constexpr int kGatGroup = kPlanGroup;

// `list` (ascending, count[0] entries) names the groups to look at; without one every group is.
template <int VEC, int NT, bool POS>
__global__ __launch_bounds__(kGatThreads) void gat_fwd_group(const int32_t *__restrict__ off, GatPieces piece,
                                                             GatPieces group, const int2 *__restrict__ start,
                                                             const int32_t *__restrict__ list,
                                                             const int32_t *__restrict__ count, int R, int H,
                                                             int D, int chunk, int nchunks)
{
    const int n = list ? uniform(count[0]) : (nchunks + kGatGroup - 1) / kGatGroup;
    const int stride = gridDim.x * kGatWaves;
    for (int i = blockIdx.x * kGatWaves + wave_in_block(); i < n; i += stride) {
        const int g = list ? uniform(list[i]) : i;
        const int kend = (g + 1) * kGatGroup;
        if (g < 0 || kend >= nchunks) continue;
        const int r = uniform(start[kend].x);
        if (r < 0 || r >= R) continue;
        const int s = uniform(off[r]);
        if (uniform(start[kend].y) <= s) continue;
        const int a = max((int)(((int64_t)max(s, 0) + r) / chunk), g * kGatGroup);
        const int F = H * D;
        const int f0 = lane_id() * VEC;
        SoftState<VEC, NT, POS> st;
        st.clear();
        st.merge(piece, a, kend, F, H, D, f0);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F) {
                gstore<VEC>(group.vec + (size_t)g * F + f, st.acc[t]);
                if constexpr (POS) gstore<VEC>(group.pvec + (size_t)g * F + f, st.pacc[t]);
                if (f % D == 0) {
                    group.mx[(size_t)g * H + f / D] = st.M[t];
                    group.sum[(size_t)g * H + f / D] = st.L[t];
                    if constexpr (POS) group.psum[(size_t)g * H + f / D] = st.LP[t];
                }
            }
        }
    }
}

// Merges, in chunk order, the pieces of a row that started in an earlier
// chunk and ends in chunk k (its last piece sits unnormalised in out/smax/ssum).
template <int VEC, int NT, bool POS>
__global__ __launch_bounds__(kGatThreads) void gat_fwd_fixup(
    const int32_t *__restrict__ off, float *__restrict__ out, float *__restrict__ smax, float *__restrict__ ssum,
    float *__restrict__ pos, float *__restrict__ spos, GatPieces piece, GatPieces group,
    const int2 *__restrict__ start, const int32_t *__restrict__ list, const int32_t *__restrict__ count, int R, int H,
    int D, int chunk, int nchunks)
{
    const int n = list ? min(uniform(count[0]), nchunks) : nchunks;
    const int stride = gridDim.x * kGatWaves;
    for (int i = blockIdx.x * kGatWaves + wave_in_block(); i < n; i += stride) {
        const int k = list ? uniform(list[i]) : i;
        if (k < 0 || k >= nchunks) continue;
        const int r0 = uniform(start[k].x);
        const int r1 = uniform(start[k + 1].x);
        if (r0 < 0 || r0 >= R || r1 <= r0) continue;
        const int s = uniform(off[r0]);
        if (uniform(start[k].y) <= s) continue;
        const int a = min((int)(((int64_t)max(s, 0) + r0) / chunk), k);
        const int F = H * D;
        const int f0 = lane_id() * VEC;
        SoftState<VEC, NT, POS> st;
        st.clear();
        const int ga = a / kGatGroup, gb = k / kGatGroup;
        if (ga == gb) {
            st.merge(piece, a, k, F, H, D, f0);
        } else {
            st.merge(group, ga, gb, F, H, D, f0);
            st.merge(piece, gb * kGatGroup, k, F, H, D, f0);
        }
        // the row's last piece, as the chunk's wavefront left it in the output arrays
        const GatPieces last{out, smax, ssum, pos, spos};
        st.merge(last, r0, r0 + 1, F, H, D, f0);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F) {
                float o[VEC];
                const float inv = st.L[t] > 0.f ? 1.f / st.L[t] : 0.f;
#pragma unroll
                for (int v = 0; v < VEC; v++) o[v] = st.acc[t][v] * inv;
                gstore<VEC>(out + (size_t)r0 * F + f, o);
                if constexpr (POS) {
#pragma unroll
                    for (int v = 0; v < VEC; v++) o[v] = st.pacc[t][v] * inv;
                    gstore<VEC>(pos + (size_t)r0 * F + f, o);
                }
            }
        }
        // every lane of a head holds the same (M, L); the head's first lane stores them.  The
        // loads of the old values above are complete before these stores issue (their
        // results feed the stored values, same wavefront).
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F && f % D == 0) {
                const float inv = st.L[t] > 0.f ? 1.f / st.L[t] : 0.f;
                smax[(size_t)r0 * H + f / D] = st.M[t];
                ssum[(size_t)r0 * H + f / D] = st.L[t];
                if constexpr (POS) spos[(size_t)r0 * H + f / D] = st.LP[t] * inv;
            }
        }
    }
}

// Column (destination) of every CSC slot by binary search; one thread per (slot, head).
__global__ void gat_alpha(const int32_t *__restrict__ off, const int32_t *__restrict__ idx,
                          const float *__restrict__ el, const float *__restrict__ er,
                          const float *__restrict__ smax, const float *__restrict__ ssum, float slope,
                          float *__restrict__ alpha, int V, int64_t E, int H)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= E * H) return;
    const int64_t j = i / H;
    const int k = (int)(i % H);
    int lo = 0, hi = V;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)off[mid] <= j) lo = mid; else hi = mid;
    }
    const int c = idx[j];
    float a = 0.f;
    if ((unsigned)c < (unsigned)V) {
        const float s = lrelu(el[(size_t)c * H + k] + er[(size_t)lo * H + k], slope);
        a = expf(s - smax[(size_t)lo * H + k]) / ssum[(size_t)lo * H + k];
    }
    alpha[i] = a;
}

// ---------------------------------------------------------------- backward ---
// Per node and head: stat[v,k] = (er, smax + log ssum, g[v,k,:].out[v,k,:], -) for the pass over
// the sources (alpha = exp(lrelu(z) - smax) / ssum = exp(lrelu(z) - (smax + log ssum)): one
// value to gather instead of two), and the destination-side logit gradient
//   g_er[v,k] = (1 - slope) (g[v,k,:].pos[v,k,:] - (g[v,k,:].out[v,k,:]) spos[v,k]).
__device__ __forceinline__ float log_denominator(float smax, float ssum)
{
    return ssum > 0.f ? smax + logf(ssum) : INFINITY;      // no in-edges: alpha = exp(-inf) = 0
}
__global__ void gat_bwd_node_stats(const float *__restrict__ er, const float *__restrict__ smax,
                                   const float *__restrict__ ssum, const float *__restrict__ spos,
                                   const float *__restrict__ g_out, const float *__restrict__ out,
                                   const float *__restrict__ pos, float slope, float4 *__restrict__ stat,
                                   float *__restrict__ g_er, int64_t VH, int D)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= VH) return;
    const float *g = g_out + i * D, *o = out + i * D, *p = pos + i * D;
    float dot = 0.f, dp = 0.f;
    for (int j = 0; j < D; j++) {
        dot = fmaf(g[j], o[j], dot);
        dp = fmaf(g[j], p[j], dp);
    }
    stat[i] = make_float4(er[i], log_denominator(smax[i], ssum[i]), dot, 0.f);
    g_er[i] = (1.f - slope) * (dp - dot * spos[i]);
}

// Coalesced form (D = 4*lph, lph a power of two <= 64), as gat_node_scores_vec.
__global__ __launch_bounds__(256) void gat_bwd_node_stats_vec(const float *__restrict__ er,
                                                              const float *__restrict__ smax,
                                                              const float *__restrict__ ssum,
                                                              const float *__restrict__ spos,
                                                              const float4 *__restrict__ g_out,
                                                              const float4 *__restrict__ out,
                                                              const float4 *__restrict__ pos, float slope,
                                                              float4 *__restrict__ stat, float *__restrict__ g_er,
                                                              int64_t n4, int lph)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float dot = 0.f, dp = 0.f;
    if (i < n4) {
        const float4 g = g_out[i], o = out[i], p = pos[i];
        dot = g.x * o.x + g.y * o.y + g.z * o.z + g.w * o.w;
        dp = g.x * p.x + g.y * p.y + g.z * p.z + g.w * p.w;
    }
    for (int o = 1; o < lph; o <<= 1) {
        dot += __shfl_xor(dot, o, kWave);
        dp += __shfl_xor(dp, o, kWave);
    }
    if (i < n4 && i % lph == 0) {
        const int64_t vh = i / lph;
        stat[vh] = make_float4(er[vh], log_denominator(smax[vh], ssum[vh]), dot, 0.f);
        g_er[vh] = (1.f - slope) * (dp - dot * spos[vh]);
    }
}

// Pass over the transposed arrays: row r = source, entries = destinations c.
//   alpha  = exp(lrelu(el[r]+er[c]) - smax[c]) / ssum[c]  (as one exp, see gat_bwd_node_stats)
//   galpha = g_out[c,k,:].h[r,k,:]                     (reduced over the head's lanes)
//   dz     = alpha (galpha - g_out[c,k,:].out[c,k,:]) * lrelu'(z)
//   acc   += alpha g_out[c,:];  g_el += dz
// and at the end of the row  g_h[r,:] = acc + g_el a_src + g_er[r] a_dst.  The row of h and the
// two scalars of the current source are in registers, so the gradients of a_src and a_dst
// (sums over the nodes of g_el[r] h[r,:] and g_er[r] h[r,:]) are accumulated on the way: every
// piece of a row adds its share of g_el, the piece that ends the row adds the g_er term, and
// the wavefront leaves one partial row of each in red[chunk][2][F].
// A row cut across chunks: the leading pieces (acc, g_el) go to `partial` / `pel`; the piece that
// ends the row is stored as it is in g_h / g_el_row, and gat_bwd_fixup adds everything up.
// lph = lanes per head (power of two) when H > 1; for H == 1 the whole
// wavefront (all tiles) reduces into the single head.
template <int VEC, int NT, bool QUADS>
__global__ __launch_bounds__(kGatThreads) void gat_bwd_merge(
    const int32_t *__restrict__ t_off, const int32_t *__restrict__ t_idx,
    const float *__restrict__ h, const float *__restrict__ el, const float4 *__restrict__ stat,
    const float *__restrict__ g_er, const float *__restrict__ g_out, const float *__restrict__ a_src,
    const float *__restrict__ a_dst, float slope, float *__restrict__ g_h, float *__restrict__ g_el_row,
    float *__restrict__ partial, float *__restrict__ pel, float *__restrict__ red,
    const int2 *__restrict__ start, int R, int E, int H, int D, int lph, int nchunks)
{
    constexpr int kGatUnroll = gat_unroll(VEC * NT);
    // a_src and a_dst wait in LDS for the row ends (a read there costs no vector-memory wait,
    // and the registers are needed for the gathers in flight)
    __shared__ float a_lds[2][NT * VEC * kWave];
    const int k = blockIdx.x * kGatWaves + wave_in_block();
    const int lane = lane_id();
    const int F = H * D;
    const int f0 = lane * VEC;
    for (int f = threadIdx.x; f < NT * VEC * kWave; f += kGatThreads) {
        a_lds[0][f] = f < F ? a_src[f] : 0.f;
        a_lds[1][f] = f < F ? a_dst[f] : 0.f;
    }
    __syncthreads();
    if (k >= nchunks) return;
    bool act[NT], lead[NT];
    int head[NT], fo[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int f = f0 + t * kWave * VEC;
        act[t] = f < F;
        head[t] = act[t] ? f / D : 0;
        lead[t] = act[t] && (f % D == 0);
        fo[t] = act[t] ? f : 0;
    }
    constexpr bool quads = QUADS;      // the lanes of a head are whole quads (D a multiple of 4 VEC)
    // this wavefront's share of the gradients of a_src and a_dst
    float pas[NT][VEC], pad[NT][VEC];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < VEC; v++) pas[t][v] = pad[t][v] = 0.f;

    {
        const int2 s0 = start[k], s1 = start[k + 1];
        const int r1 = min(max(uniform(s1.x), 0), R);
        int r = min(max(uniform(s0.x), 0), r1);
        const int j0 = min(max(uniform(s0.y), 0), E);
        const int j1 = min(uniform(s1.y), E);
        // the chunk's first row began in an earlier chunk: its sums are one piece of several
        const int raw_row = (r < r1 && uniform(t_off[r]) < j0) ? r : -1;

        int rb = r;
        int ends = (rb + lane < R) ? t_off[rb + 1 + lane] : 0x7fffffff;
        int row_end = bcast_i(ends, 0);

        // h row, el and g_er of the current source row and, already on their way, of the next one:
        // a row end must not wait for fresh loads (lanes past F read offset 0 and are ignored)
        float acc[NT][VEC], gel[NT], hr[NT][VEC], el_r[NT], ger_r[NT];
        float hr_next[NT][VEC], el_next[NT], ger_next[NT];
        auto fetch_row = [&](int row) {
            const size_t rc = (size_t)min(row, R - 1);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                gload<VEC>(hr_next[t], h + rc * F + fo[t]);
                el_next[t] = el[rc * H + head[t]];
                ger_next[t] = g_er[rc * H + head[t]];
            }
        };
        auto reset = [&]() {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                gel[t] = 0.f;
                el_r[t] = el_next[t];
                ger_r[t] = ger_next[t];
#pragma unroll
                for (int v = 0; v < VEC; v++) {
                    acc[t][v] = 0.f;
                    hr[t][v] = hr_next[t][v];
                }
            }
            fetch_row(r + 1);
        };
        fetch_row(r);
        reset();
        // this piece's share of sum_r g_el[r] h[r,:]
        auto add_el_share = [&]() {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int v = 0; v < VEC; v++) pas[t][v] = fmaf(gel[t], hr[t][v], pas[t][v]);
        };
        auto store_piece = [&](float *vec, float *elp) {
#pragma unroll
            for (int t = 0; t < NT; t++)
                if (act[t]) {
                    gstore<VEC>(vec + f0 + t * kWave * VEC, acc[t]);
                    if (lead[t]) elp[head[t]] = gel[t];
                }
        };
        auto flush_row = [&]() {
            add_el_share();
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int v = 0; v < VEC; v++) pad[t][v] = fmaf(ger_r[t], hr[t][v], pad[t][v]);
            if (r == raw_row) {
                store_piece(g_h + (size_t)r * F, g_el_row + (size_t)r * H);
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    if (act[t]) {
                        float o[VEC];
#pragma unroll
                        for (int v = 0; v < VEC; v++)
                            o[v] = acc[t][v] + gel[t] * a_lds[0][fo[t] + v] + ger_r[t] * a_lds[1][fo[t] + v];
                        gstore<VEC>(g_h + (size_t)r * F + f0 + t * kWave * VEC, o);
                    }
            }
            r++;
            if (r - rb == kWave) {
                rb = r;
                ends = (rb + lane < R) ? t_off[rb + 1 + lane] : 0x7fffffff;
            }
            row_end = bcast_i(ends, r - rb);
            reset();
        };

        for (int jb = j0; jb < j1; jb += kWave) {
            const int n = min(kWave, j1 - jb);
            int my_c = -1;
            if (lane < n) {
                my_c = t_idx[jb + lane];
                if ((unsigned)my_c >= (unsigned)R) my_c = -1;
            }
            for (int i0 = 0; i0 < n; i0 += kGatUnroll) {
                float gv[kGatUnroll][NT][VEC];
                // (er, smax + log ssum, g.out) of the destination and head: one float per lane, the
                // lane's number inside its quad choosing which (a head's lanes are whole quads when
                // quads holds; the three values are spread over the quad when they are used).  Twelve
                // bytes per lane instead cost the address unit three times as long per entry, more
                // than the 512-byte row gathered beside them.
                float sq[QUADS ? kGatUnroll : 1][QUADS ? NT : 1];
                float3 st[QUADS ? 1 : kGatUnroll][QUADS ? 1 : NT];
#pragma unroll
                for (int u = 0; u < kGatUnroll; u++) {
                    const int c = max(bcast_i(my_c, (i0 + u) & (kWave - 1)), 0);
                    const float *src = g_out + (size_t)c * F;
                    const float4 *ss = stat + (size_t)c * H;
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        gload<VEC>(gv[u][t], src + fo[t]);
                        if constexpr (quads) sq[u][t] = reinterpret_cast<const float *>(ss + head[t])[lane & 3];
                        else st[u][t] = *reinterpret_cast<const float3 *>(ss + head[t]);
                    }
                }
#pragma unroll
                for (int u = 0; u < kGatUnroll; u++) {
                    if (i0 + u < n) {
                        const int jj = jb + i0 + u;
                        while (jj == row_end && r < r1) flush_row();
                        const int c = bcast_i(my_c, i0 + u);
                        if (c >= 0) {        // a destination out of range counts for nothing on either side
                            float dot[NT];
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                dot[t] = 0.f;
                                if (act[t]) {
#pragma unroll
                                    for (int v = 0; v < VEC; v++) dot[t] = fmaf(gv[u][t][v], hr[t][v], dot[t]);
                                }
                            }
                            if (H == 1) {
                                float s = 0.f;
#pragma unroll
                                for (int t = 0; t < NT; t++) s += dot[t];
                                s = lane_group_sum(s, kWave);
#pragma unroll
                                for (int t = 0; t < NT; t++) dot[t] = s;
                            } else {
#pragma unroll
                                for (int t = 0; t < NT; t++) dot[t] = lane_group_sum(dot[t], lph);
                            }
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                float3 sv;
                                if constexpr (quads) {
                                    sv.x = quad_lane<0x00>(sq[u][t]);
                                    sv.y = quad_lane<0x55>(sq[u][t]);
                                    sv.z = quad_lane<0xAA>(sq[u][t]);
                                } else {
                                    sv = st[u][t];
                                }
                                if (act[t]) {
                                    const float z = el_r[t] + sv.x;
                                    const float alpha = fast_exp(lrelu(z, slope) - sv.y);
                                    const float gz = alpha * (dot[t] - sv.z) * (z > 0.f ? 1.f : slope);
                                    gel[t] += gz;
#pragma unroll
                                    for (int v = 0; v < VEC; v++) acc[t][v] = fmaf(alpha, gv[u][t][v], acc[t][v]);
                                }
                            }
                        }
                    }
                }
            }
        }
        while (r < r1) flush_row();
        if (r1 < R && j1 > uniform(t_off[r1])) {
            add_el_share();
            store_piece(partial + (size_t)k * F, pel + (size_t)k * H);
        }
    }

    // this chunk's partial rows of the two parameter gradients
#pragma unroll
    for (int t = 0; t < NT; t++)
        if (act[t]) {
            float *dst = red + (size_t)k * 2 * F + f0 + t * kWave * VEC;
            gstore<VEC>(dst, pas[t]);
            gstore<VEC>(dst + F, pad[t]);
        }
}

// Plain sums of backward pieces: vec [.,F] and per-head scalars elp [.,H].
template <int VEC, int NT> struct SumState {
    float acc[NT][VEC], gel[NT];
    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            gel[t] = 0.f;
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[t][v] = 0.f;
        }
    }
    __device__ __forceinline__ void add(const float *__restrict__ vec, const float *__restrict__ elp, int first,
                                        int last, int F, int H, int D, int f0)
    {
        constexpr int kBatch = VEC * NT >= 16 ? 2 : (VEC * NT >= 8 ? 4 : (VEC * NT >= 4 ? 8 : 16));
        for (int kb = first; kb < last; kb += kBatch) {
            float x[kBatch][NT][VEC], pe[kBatch][NT];
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                const size_t pc = (size_t)min(kb + b, last - 1);
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int f = f0 + t * kWave * VEC;
                    const int fc = f < F ? f : 0;
                    gload<VEC>(x[b][t], vec + pc * F + fc);
                    pe[b][t] = elp[pc * H + fc / D];
                }
            }
#pragma unroll
            for (int b = 0; b < kBatch; b++)
                if (kb + b < last) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        const int f = f0 + t * kWave * VEC;
                        if (f < F) {
#pragma unroll
                            for (int v = 0; v < VEC; v++) acc[t][v] += x[b][t][v];
                            gel[t] += pe[b][t];
                        }
                    }
                }
        }
    }
    __device__ __forceinline__ void store(float *vec, float *elp, int F, int D, int f0) const
    {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F) gstore<VEC>(vec + f, acc[t]);
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F && f % D == 0) elp[f / D] = gel[t];
        }
    }
};

template <int VEC, int NT>
__global__ __launch_bounds__(kGatThreads) void gat_bwd_group(const int32_t *__restrict__ t_off,
                                                             const float *__restrict__ partial,
                                                             const float *__restrict__ pel, float *__restrict__ gvec,
                                                             float *__restrict__ gel,
                                                             const int2 *__restrict__ start,
                                                             const int32_t *__restrict__ list,
                                                             const int32_t *__restrict__ count, int R, int H,
                                                             int D, int chunk, int nchunks)
{
    const int n = list ? uniform(count[0]) : (nchunks + kGatGroup - 1) / kGatGroup;
    const int stride = gridDim.x * kGatWaves;
    for (int i = blockIdx.x * kGatWaves + wave_in_block(); i < n; i += stride) {
        const int g = list ? uniform(list[i]) : i;
        const int kend = (g + 1) * kGatGroup;
        if (g < 0 || kend >= nchunks) continue;
        const int r = uniform(start[kend].x);
        if (r < 0 || r >= R) continue;
        const int s = uniform(t_off[r]);
        if (uniform(start[kend].y) <= s) continue;
        const int a = max((int)(((int64_t)max(s, 0) + r) / chunk), g * kGatGroup);
        const int F = H * D;
        const int f0 = lane_id() * VEC;
        SumState<VEC, NT> st;
        st.clear();
        st.add(partial, pel, a, kend, F, H, D, f0);
        st.store(gvec + (size_t)g * F, gel + (size_t)g * H, F, D, f0);
    }
}

// A row cut across chunks and ending in chunk k: adds its pieces in chunk order to the last
// piece (left in g_h / g_el_row by that chunk's wavefront) and finishes the row,
// g_h[r,:] = acc + g_el a_src + g_er[r] a_dst.
template <int VEC, int NT>
__global__ __launch_bounds__(kGatThreads) void gat_bwd_fixup(const int32_t *__restrict__ t_off,
                                                             float *__restrict__ g_h,
                                                             const float *__restrict__ g_el_row,
                                                             const float *__restrict__ g_er,
                                                             const float *__restrict__ a_src,
                                                             const float *__restrict__ a_dst,
                                                             const float *__restrict__ partial,
                                                             const float *__restrict__ pel,
                                                             const float *__restrict__ gvec,
                                                             const float *__restrict__ gel,
                                                             const int2 *__restrict__ start,
                                                             const int32_t *__restrict__ list,
                                                             const int32_t *__restrict__ count, int R, int H, int D,
                                                             int chunk, int nchunks)
{
    const int n = list ? min(uniform(count[0]), nchunks) : nchunks;
    const int stride = gridDim.x * kGatWaves;
    for (int i = blockIdx.x * kGatWaves + wave_in_block(); i < n; i += stride) {
        const int k = list ? uniform(list[i]) : i;
        if (k < 0 || k >= nchunks) continue;
        const int r0 = uniform(start[k].x);
        const int r1 = uniform(start[k + 1].x);
        if (r0 < 0 || r0 >= R || r1 <= r0) continue;
        const int s = uniform(t_off[r0]);
        if (uniform(start[k].y) <= s) continue;
        const int a = min((int)(((int64_t)max(s, 0) + r0) / chunk), k);
        const int F = H * D;
        const int f0 = lane_id() * VEC;
        SumState<VEC, NT> st;
        st.clear();
        const int ga = a / kGatGroup, gb = k / kGatGroup;
        if (ga == gb) {
            st.add(partial, pel, a, k, F, H, D, f0);
        } else {
            st.add(gvec, gel, ga, gb, F, H, D, f0);
            st.add(partial, pel, gb * kGatGroup, k, F, H, D, f0);
        }
        st.add(g_h, g_el_row, r0, r0 + 1, F, H, D, f0);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int f = f0 + t * kWave * VEC;
            if (f < F) {
                float as[VEC], ad[VEC], o[VEC];
                gload<VEC>(as, a_src + f);
                gload<VEC>(ad, a_dst + f);
                const float ger = g_er[(size_t)r0 * H + f / D];
#pragma unroll
                for (int v = 0; v < VEC; v++) o[v] = st.acc[t][v] + st.gel[t] * as[v] + ger * ad[v];
                gstore<VEC>(g_h + (size_t)r0 * F + f, o);
            }
        }
    }
}

// Sums of the per-chunk partial rows red[0..nrows)[2][F], in two fixed-order stages:
// kRedSlices slices of the rows into mid[slice][2F], then the slices.  64 columns per block,
// 16 strided groups of rows added in a fixed order, then the 16 group sums in order.
constexpr int kRedSlices = 32;
__global__ __launch_bounds__(1024) void gat_bwd_reduce(const float *__restrict__ red, int nrows, int per_slice, int W,
                                                       float *__restrict__ out_rows, float *__restrict__ g_a_src,
                                                       float *__restrict__ g_a_dst, int F)
{
    __shared__ float part[16][64];
    const int col = blockIdx.x * 64 + (threadIdx.x & 63);   // index into [2][F]
    const int grp = threadIdx.x >> 6;
    const int b_lo = blockIdx.y * per_slice, b_hi = min(nrows, b_lo + per_slice);
    float s = 0.f;
    if (col < W) {
        // eight partials fetched together, added in the same order as one by one
        constexpr int kB = 8;
        for (int b0 = b_lo + grp; b0 < b_hi; b0 += 16 * kB) {
            float v[kB];
#pragma unroll
            for (int i = 0; i < kB; i++) {
                const int b = min(b0 + 16 * i, b_hi - 1);
                v[i] = red[(size_t)b * W + col];
            }
#pragma unroll
            for (int i = 0; i < kB; i++)
                if (b0 + 16 * i < b_hi) s += v[i];
        }
    }
    part[grp][threadIdx.x & 63] = s;
    __syncthreads();
    if (grp == 0 && col < W) {
        float t = 0.f;
#pragma unroll
        for (int g = 0; g < 16; g++) t += part[g][threadIdx.x];
        if (out_rows) out_rows[(size_t)blockIdx.y * W + col] = t;
        else (col / F ? g_a_dst : g_a_src)[col % F] = t;
    }
}

// ------------------------------------------------------------------ host ---
struct GatShape {
    int vec, nt, chunk, nchunks, lph;
    bool bwd_ok;
};

// items per wavefront: the start-up chain of a chunk (row lookup, offsets, indices, first
// gathers) is a few microseconds, so chunks stay at 64 items or more
int gat_chunk_for(int64_t M)
{
    // tuning aid, read once per process
    static const int forced = [] {
        const char *e = getenv("JGAMD_GAT_CHUNK");
        const int v = e ? atoi(e) : 0;
        return v < 16 ? 0 : (v > 4096 ? 4096 : v);
    }();
    if (forced) return forced;
    int chunk = 128;
    while (chunk > 64 && M / chunk < 16384) chunk >>= 1;
    return chunk;
}

static unsigned gat_list_grid(int hint, int upper)
{
    const int64_t n = hint >= 0 ? (hint < upper ? hint : upper) : (upper < 8192 ? upper : 8192);
    return (unsigned)ceil_div(n > 0 ? n : 1, kGatWaves);
}

static GatShape gat_shape(int32_t V, int64_t E, int32_t H, int32_t D)
{
    GatShape s{};
    const int F = H * D;
    s.vec = D % 4 == 0 ? 4 : D % 2 == 0 ? 2 : 1;
    while (s.vec > 1 && F <= kWave * (s.vec / 2)) s.vec >>= 1;
    s.nt = (int)ceil_div(F, kWave * s.vec);
    const int64_t M = (int64_t)V + E;
    s.chunk = gat_chunk_for(M);
    s.nchunks = (int)ceil_div(M > 0 ? M : 1, s.chunk);
    s.lph = D / s.vec;
    s.bwd_ok = H == 1 || (s.lph >= 1 && s.lph <= kWave && (s.lph & (s.lph - 1)) == 0);
    return s;
}

// float4 streaming form of the node kernels: D = 4*lph, lph a power of two <= 64
static bool vec_nodes_ok(int D)
{
    const int lph = D / 4;
    return D % 4 == 0 && lph >= 1 && lph <= kWave && (lph & (lph - 1)) == 0;
}

static int32_t check_gat(const char *who, int32_t V, int64_t E, int32_t H, int32_t D)
{
    if (V < 0 || E < 0 || H < 1 || D < 1) return fail(JGAMD_ERR_SIZE, "%s: bad size (V=%d E=%lld H=%d D=%d)", who, V, (long long)E, H, D);
    if ((int64_t)V + E >= ((int64_t)1 << 31) - 4096) return fail(JGAMD_ERR_SIZE, "%s: V + E does not fit int32", who);
    if ((int64_t)H * D > 2048) return fail(JGAMD_ERR_UNSUPPORTED, "%s: H*D = %lld above 2048", who, (long long)H * D);
    GatShape s = gat_shape(V, E, H, D);
    if (s.nt > 8) return fail(JGAMD_ERR_UNSUPPORTED, "%s: H*D = %d needs %d feature tiles (max 8) at vector width %d", who, H * D, s.nt, s.vec);
    return 0;
}

static size_t pieces_bytes(size_t n, int H, int D)
{
    return 2 * carve_bytes(n * H * D, 4) + 3 * carve_bytes(n * H, 4);
}
static GatPieces carve_pieces(Carver &carve, size_t n, int H, int D)
{
    GatPieces p;
    p.vec = carve.take<float>(n * H * D);
    p.pvec = carve.take<float>(n * H * D);
    p.mx = carve.take<float>(n * H);
    p.sum = carve.take<float>(n * H);
    p.psum = carve.take<float>(n * H);
    return p;
}

static size_t gat_fwd_ws(int32_t V, int64_t E, int32_t H, int32_t D)
{
    GatShape s = gat_shape(V, E, H, D);
    const size_t ng = (size_t)ceil_div(s.nchunks, kGatGroup);
    // + el / er of a call that brings none and whose shape the in-kernel scores do not cover
    return carve_bytes((size_t)s.nchunks + 1, sizeof(int2)) + pieces_bytes((size_t)s.nchunks, H, D) +
           pieces_bytes(ng, H, D) + 2 * carve_bytes((size_t)V * H, 4);
}

static size_t gat_bwd_ws(int32_t V, int64_t E, int32_t H, int32_t D)
{
    GatShape s = gat_shape(V, E, H, D);
    const size_t ng = (size_t)ceil_div(s.nchunks, kGatGroup);
    const size_t F = (size_t)H * D;
    return carve_bytes(ng * F, 4) + carve_bytes(ng * H, 4) + carve_bytes((size_t)s.nchunks + 1, sizeof(int2)) +
           carve_bytes((size_t)s.nchunks * F, 4) + carve_bytes((size_t)s.nchunks * H, 4) +
           carve_bytes((size_t)V * H, 16) + 2 * carve_bytes((size_t)V * H, 4) +
           carve_bytes((size_t)s.nchunks * 2 * F, 4) + carve_bytes((size_t)kRedSlices * 2 * F, 4);
}

#define JG_GAT_DISPATCH(CALL)                         \
    switch (s.vec * 16 + s.nt) {                      \
        CALL(1, 1) CALL(1, 2) CALL(1, 3) CALL(1, 4) CALL(1, 5) CALL(1, 6) CALL(1, 7) CALL(1, 8) \
        CALL(2, 1) CALL(2, 2) CALL(2, 3) CALL(2, 4) CALL(2, 5) CALL(2, 6) CALL(2, 7) CALL(2, 8) \
        CALL(4, 1) CALL(4, 2) CALL(4, 3) CALL(4, 4) CALL(4, 5) CALL(4, 6) CALL(4, 7) CALL(4, 8) \
    default: break;                                   \
    }

}  // namespace jg

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

JG_EXPORT int32_t jgamd_gat_fwd_workspace(int32_t V, int64_t E, int32_t H, int32_t D, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "gat_fwd_workspace: bytes is NULL");
    if (int32_t rc = check_gat("gat_fwd", V, E, H, D)) return rc;
    *bytes = V == 0 ? 0 : gat_fwd_ws(V, E, H, D);
    return 0;
}

JG_EXPORT int32_t jgamd_gat_fwd(const void *plan, int32_t n_fix, int32_t n_grp, const int32_t *off,
                                const int32_t *idx, const float *h, const float *a_src, const float *a_dst,
                                float slope, float *el, float *er, float *smax, float *ssum, float *pos, float *spos,
                                float *alpha, float *out, int32_t V, int64_t E, int32_t H, int32_t D, void *ws,
                                size_t ws_bytes, void *stream)
{
    if (int32_t rc = check_gat("gat_fwd", V, E, H, D)) return rc;
    if (V == 0) return 0;
    if (!off || !h || !a_src || !a_dst || !smax || !ssum || !out)
        return fail(JGAMD_ERR_NULL, "gat_fwd: NULL array");
    if ((el == nullptr) != (er == nullptr)) return fail(JGAMD_ERR_NULL, "gat_fwd: el and er go together");
    if (!el && (pos || alpha)) return fail(JGAMD_ERR_NULL, "gat_fwd: pos / alpha need el and er");
    if ((pos == nullptr) != (spos == nullptr)) return fail(JGAMD_ERR_NULL, "gat_fwd: pos and spos go together");
    if (E > 0 && !idx) return fail(JGAMD_ERR_NULL, "gat_fwd: idx is NULL with E > 0");
    if ((((uintptr_t)h | (uintptr_t)out | (uintptr_t)pos) & 15) != 0)
        return fail(JGAMD_ERR_ALIGN, "gat_fwd: h/out/pos not 16-byte aligned");
    const size_t need = gat_fwd_ws(V, E, H, D);
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "gat_fwd: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "gat_fwd: workspace not 256-byte aligned");
    if (((uintptr_t)plan & 255) != 0) return fail(JGAMD_ERR_ALIGN, "gat_fwd: plan not 256-byte aligned");
    const GatShape s = gat_shape(V, E, H, D);
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver carve(ws);
    int2 *own_start = carve.take<int2>((size_t)s.nchunks + 1);
    ChunkPlan pv{};
    if (plan) {
        pv = chunk_plan_view(JGAMD_PLAN_GAT, V, E, plan);
    } else {
        chunk_starts_enqueue(off, V, E, s.chunk, s.nchunks, own_start, st);
        pv.start = own_start;
        n_fix = n_grp = -1;
    }
    const int ngroups = (int)ceil_div(s.nchunks, kGatGroup);
    const GatPieces piece = carve_pieces(carve, (size_t)s.nchunks, H, D);
    const GatPieces group = carve_pieces(carve, (size_t)ngroups, H, D);
    const int64_t VH = (int64_t)V * H;
    if (pos && !s.bwd_ok) return fail(JGAMD_ERR_UNSUPPORTED, "gat_fwd: pos / spos need a shape jgamd_gat_bwd takes");
    float *own_el = carve.take<float>((size_t)V * H), *own_er = carve.take<float>((size_t)V * H);
    // no el / er wanted: the scores are taken inside the merge kernel where its lane layout allows
    static const bool no_fuse = [] { const char *e = getenv("JGAMD_GAT_SCORES"); return e && e[0] == 'n'; }();
    const bool fuse = !el && !no_fuse && s.nt == 1 && D % s.vec == 0 && s.lph >= 1 && s.lph <= kWave &&
                      (s.lph & (s.lph - 1)) == 0;
    if (!el) {
        el = own_el;
        er = own_er;
    }
    if (fuse) {
    } else if (vec_nodes_ok(D) && (((uintptr_t)a_src | (uintptr_t)a_dst) & 15) == 0)
        hipLaunchKernelGGL(gat_node_scores_vec, dim3((unsigned)ceil_div(VH * (D / 4), 256)), dim3(256), 0, st,
                           reinterpret_cast<const float4 *>(h), reinterpret_cast<const float4 *>(a_src),
                           reinterpret_cast<const float4 *>(a_dst), el, er, VH * (D / 4), H, D / 4);
    else
        hipLaunchKernelGGL(gat_node_scores, dim3((unsigned)ceil_div(VH, 256)), dim3(256), 0, st, h, a_src, a_dst, el,
                           er, VH, H, D);
    dim3 grid((unsigned)ceil_div(s.nchunks, kGatWaves)), block(kGatThreads);
    // pieces of rows cut across chunks: over the plan's lists, or over every chunk and group
    const bool listed = pv.fix != nullptr;
    const dim3 ggrid(listed ? gat_list_grid(n_grp, ngroups) : (unsigned)ceil_div(ngroups, kGatWaves));
    const dim3 fgrid(listed ? gat_list_grid(n_fix, s.nchunks) : grid.x);
    const bool with_group = ngroups > 1 && n_grp != 0 && n_fix != 0;
#define JG_FWD_P(VV, NN, PP)                                                                                     \
    {                                                                                                            \
        if (!PP && fuse)                                                                                         \
            hipLaunchKernelGGL((gat_fwd_merge<VV, 1, false, true>), grid, block, 0, st, off, idx, h, el, er,     \
                               slope, out, smax, ssum, pos, spos, piece, pv.start, V, (int)E, H, D, s.nchunks,   \
                               a_src, a_dst, s.lph);                                                             \
        else                                                                                                     \
            hipLaunchKernelGGL((gat_fwd_merge<VV, NN, PP>), grid, block, 0, st, off, idx, h, el, er, slope, out, \
                               smax, ssum, pos, spos, piece, pv.start, V, (int)E, H, D, s.nchunks);              \
        if (with_group)                                                                                          \
            hipLaunchKernelGGL((gat_fwd_group<VV, NN, PP>), ggrid, block, 0, st, off, piece, group, pv.start,    \
                               pv.grp, pv.counts + 1, V, H, D, s.chunk, s.nchunks);                              \
        if (n_fix != 0)                                                                                          \
            hipLaunchKernelGGL((gat_fwd_fixup<VV, NN, PP>), fgrid, block, 0, st, off, out, smax, ssum, pos,      \
                               spos, piece, group, pv.start, pv.fix, pv.counts, V, H, D, s.chunk, s.nchunks);    \
    }
#define JG_FWD(VV, NN)                  \
    case VV * 16 + NN:                  \
        if (pos) JG_FWD_P(VV, NN, true) \
        else JG_FWD_P(VV, NN, false)    \
        break;
    JG_GAT_DISPATCH(JG_FWD)
#undef JG_FWD
#undef JG_FWD_P
    if (alpha && E > 0)
        hipLaunchKernelGGL(gat_alpha, dim3((unsigned)ceil_div(E * H, 256)), dim3(256), 0, st, off, idx, el, er, smax,
                           ssum, slope, alpha, V, E, H);
    return launch_status("gat_fwd");
}

static int32_t check_gat_bwd(int32_t V, int64_t E, int32_t H, int32_t D)
{
    if (int32_t rc = check_gat("gat_bwd", V, E, H, D)) return rc;
    if (!gat_shape(V, E, H, D).bwd_ok)
        return fail(JGAMD_ERR_UNSUPPORTED, "gat_bwd: with H > 1 the head width D=%d must give a power-of-two lane count", D);
    return 0;
}

JG_EXPORT int32_t jgamd_gat_bwd_workspace(int32_t V, int64_t E, int32_t H, int32_t D, size_t *bytes)
{
    if (!bytes) return fail(JGAMD_ERR_NULL, "gat_bwd_workspace: bytes is NULL");
    if (int32_t rc = check_gat_bwd(V, E, H, D)) return rc;
    *bytes = V == 0 ? 0 : gat_bwd_ws(V, E, H, D);
    return 0;
}

JG_EXPORT int32_t jgamd_gat_bwd(const void *t_plan, int32_t n_fix, int32_t n_grp, const int32_t *t_off,
                                const int32_t *t_idx, const float *h, const float *a_src, const float *a_dst,
                                float slope, const float *el, const float *er, const float *smax, const float *ssum,
                                const float *spos, const float *out, const float *pos, const float *g_out,
                                float *g_h, float *g_a_src, float *g_a_dst, int32_t V, int64_t E, int32_t H, int32_t D,
                                void *ws, size_t ws_bytes, void *stream)
{
    if (int32_t rc = check_gat_bwd(V, E, H, D)) return rc;
    const GatShape s = gat_shape(V, E, H, D);
    if (!g_a_src || !g_a_dst) return fail(JGAMD_ERR_NULL, "gat_bwd: NULL gradient output");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int F = H * D;
    const unsigned col_blocks = (unsigned)ceil_div(2 * F, 64);
    if (V == 0) {
        hipLaunchKernelGGL(gat_bwd_reduce, dim3(col_blocks), dim3(1024), 0, st, nullptr, 0, 1, 2 * F, nullptr, g_a_src,
                           g_a_dst, F);
        return launch_status("gat_bwd");
    }
    if (!t_off || !h || !a_src || !a_dst || !el || !er || !smax || !ssum || !spos || !out || !pos || !g_out || !g_h)
        return fail(JGAMD_ERR_NULL, "gat_bwd: NULL array");
    if (E > 0 && !t_idx) return fail(JGAMD_ERR_NULL, "gat_bwd: t_idx is NULL with E > 0");
    if ((((uintptr_t)h | (uintptr_t)g_out | (uintptr_t)g_h | (uintptr_t)out | (uintptr_t)pos) & 15) != 0)
        return fail(JGAMD_ERR_ALIGN, "gat_bwd: h/g_out/g_h/out/pos not 16-byte aligned");
    if ((((uintptr_t)a_src | (uintptr_t)a_dst) & (uintptr_t)(4 * s.vec - 1)) != 0)
        return fail(JGAMD_ERR_ALIGN, "gat_bwd: a_src/a_dst not %d-byte aligned", 4 * s.vec);
    const size_t need = gat_bwd_ws(V, E, H, D);
    if (!ws || ws_bytes < need) return fail(JGAMD_ERR_WORKSPACE, "gat_bwd: workspace %zu < %zu bytes", ws ? ws_bytes : (size_t)0, need);
    if (((uintptr_t)ws & 255) != 0) return fail(JGAMD_ERR_ALIGN, "gat_bwd: workspace not 256-byte aligned");
    if (((uintptr_t)t_plan & 255) != 0) return fail(JGAMD_ERR_ALIGN, "gat_bwd: plan not 256-byte aligned");
    Carver carve(ws);
    const int ngroups = (int)ceil_div(s.nchunks, kGatGroup);
    float *gvec = carve.take<float>((size_t)ngroups * F);
    float *ggel = carve.take<float>((size_t)ngroups * H);
    int2 *own_start = carve.take<int2>((size_t)s.nchunks + 1);
    ChunkPlan pv{};
    if (t_plan) {
        pv = chunk_plan_view(JGAMD_PLAN_GAT, V, E, t_plan);
    } else {
        chunk_starts_enqueue(t_off, V, E, s.chunk, s.nchunks, own_start, st);
        pv.start = own_start;
        n_fix = n_grp = -1;
    }
    float *partial = carve.take<float>((size_t)s.nchunks * F);
    float *pel = carve.take<float>((size_t)s.nchunks * H);
    float4 *stat = carve.take<float4>((size_t)V * H);
    float *g_er = carve.take<float>((size_t)V * H);
    float *g_el_row = carve.take<float>((size_t)V * H);
    const int nblocks = (int)ceil_div(s.nchunks, kGatWaves);
    const int nred = s.nchunks;                                     // one partial row per chunk
    float *red = carve.take<float>((size_t)nred * 2 * F);
    float *mid = carve.take<float>((size_t)kRedSlices * 2 * F);
    const int64_t VH = (int64_t)V * H;

    if (vec_nodes_ok(D))
        hipLaunchKernelGGL(gat_bwd_node_stats_vec, dim3((unsigned)ceil_div(VH * (D / 4), 256)), dim3(256), 0, st, er,
                           smax, ssum, spos, reinterpret_cast<const float4 *>(g_out),
                           reinterpret_cast<const float4 *>(out), reinterpret_cast<const float4 *>(pos), slope, stat,
                           g_er, VH * (D / 4), D / 4);
    else
        hipLaunchKernelGGL(gat_bwd_node_stats, dim3((unsigned)ceil_div(VH, 256)), dim3(256), 0, st, er, smax, ssum,
                           spos, g_out, out, pos, slope, stat, g_er, VH, D);
    dim3 grid((unsigned)nblocks), block(kGatThreads);
    const bool listed = pv.fix != nullptr;
    const dim3 ggrid(listed ? gat_list_grid(n_grp, ngroups) : (unsigned)ceil_div(ngroups, kGatWaves));
    const dim3 fgrid(listed ? gat_list_grid(n_fix, s.nchunks) : grid.x);
#define JG_BWD(VV, NN)                                                                                             \
    case VV * 16 + NN:                                                                                             \
        if (D % (4 * VV) == 0)                                                                                     \
            hipLaunchKernelGGL((gat_bwd_merge<VV, NN, true>), grid, block, 0, st, t_off, t_idx, h, el, stat, g_er, \
                               g_out, a_src, a_dst, slope, g_h, g_el_row, partial, pel, red, pv.start, V, (int)E,  \
                               H, D, s.lph, s.nchunks);                                                            \
        else                                                                                                       \
            hipLaunchKernelGGL((gat_bwd_merge<VV, NN, false>), grid, block, 0, st, t_off, t_idx, h, el, stat,      \
                               g_er, g_out, a_src, a_dst, slope, g_h, g_el_row, partial, pel, red, pv.start, V,    \
                               (int)E, H, D, s.lph, s.nchunks);                                                    \
        if (ngroups > 1 && n_grp != 0 && n_fix != 0)                                                               \
            hipLaunchKernelGGL((gat_bwd_group<VV, NN>), ggrid, block, 0, st, t_off, partial, pel, gvec, ggel,      \
                               pv.start, pv.grp, pv.counts + 1, V, H, D, s.chunk, s.nchunks);                      \
        if (n_fix != 0)                                                                                            \
            hipLaunchKernelGGL((gat_bwd_fixup<VV, NN>), fgrid, block, 0, st, t_off, g_h, g_el_row, g_er, a_src,    \
                               a_dst, partial, pel, gvec, ggel, pv.start, pv.fix, pv.counts, V, H, D, s.chunk,     \
                               s.nchunks);                                                                         \
        break;
    JG_GAT_DISPATCH(JG_BWD)
#undef JG_BWD
    // the parameter gradients: the workgroups' partial rows, summed in a fixed order
    if (nred > 4 * kRedSlices) {
        const int per_slice = (int)ceil_div(nred, kRedSlices);
        hipLaunchKernelGGL(gat_bwd_reduce, dim3(col_blocks, kRedSlices), dim3(1024), 0, st, red, nred, per_slice,
                           2 * F, mid, nullptr, nullptr, F);
        hipLaunchKernelGGL(gat_bwd_reduce, dim3(col_blocks), dim3(1024), 0, st, mid, kRedSlices, kRedSlices, 2 * F,
                           nullptr, g_a_src, g_a_dst, F);
    } else {
        hipLaunchKernelGGL(gat_bwd_reduce, dim3(col_blocks), dim3(1024), 0, st, red, nred, nred, 2 * F, nullptr,
                           g_a_src, g_a_dst, F);
    }
    return launch_status("gat_bwd");
}
