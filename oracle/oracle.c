/*
 * TEST INFRASTRUCTURE — CPU oracle for the sparse message-passing path.
 *
 * Plain-C restatement of the single-threaded CPU loops of the reference
 * (the .cc files of jittor_geometric/ops/cpp, the `JIT_cpu` bodies).  Every function
 * names the reference lines it follows.  Nothing in the shipped library
 * links, loads or calls this file: it is used by the tests, by the smoke
 * check and by the CPU-baseline leg of the benchmark only.
 *
 * Pinning of each function (what, other than this file, fixes its answer):
 *   orc_cootocsr / orc_cootocsc   stable-argsort closed form, hand-derived
 *                                 fixtures of the reference's test graphs
 *   orc_aggregate                 dense fp64 A@x, transpose identity, the
 *                                 integer-valued 10-node fixture
 *   orc_edgesoftmax               per-segment scipy softmax, fixture
 *                                 [1, 0.2689414, 0.7310586, 1]
 *   orc_edgesoftmax_backward      closed form y*(g - sum(y*g)), finite
 *                                 differences of the forward
 *   orc_scattertoedge             numpy fancy indexing
 *   orc_edgetovertex              numpy add.at
 * The SpmmCsr operator of the reference runs inside NVIDIA cuSPARSE through
 * the jittor wheel (jittor==1.3.9.14, op cusparse_spmmcsr), which is not
 * part of the reference tree: its internal summation order is "parity
 * unpinned"; its value is pinned to orc_aggregate, which the reference's
 * tests/test_mp_spmm.py:26-36 prints beside it as the same quantity.
 *
 * Build: see oracle/Makefile  (gcc -O2 -mavx -mfma, single thread).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ops/cpp/cootocsr_op.cc:24-57.  edge_index is [2,E] row-major (src row
 * first).  Outputs are zeroed here; the reference relies on its caller
 * passing zero-filled arrays (ops/cootocsr.py:30-32). */
int orc_cootocsr(const int32_t *edge_index, const float *coo_w, int64_t E,
                 int32_t v_num, int32_t *column_indices, int32_t *row_offset,
                 float *csr_w)
{
    memset(row_offset, 0, sizeof(int32_t) * ((size_t)v_num + 1));
    for (int64_t i = 0; i < E; i++)                 /* :35-37 */
        row_offset[edge_index[i] + 1] += 1;
    for (int32_t i = 0; i < v_num; i++)             /* :39-41 */
        row_offset[i + 1] += row_offset[i];
    int32_t *vertex_index = (int32_t *)calloc(v_num > 0 ? v_num : 1, sizeof(int32_t));
    if (!vertex_index) return -1;
    for (int64_t i = 0; i < E; i++) {               /* :45-53 */
        int32_t src = edge_index[i];
        int32_t dst = edge_index[i + E];
        int32_t index = vertex_index[src]++;
        index += row_offset[src];
        column_indices[index] = dst;
        csr_w[index] = coo_w[i];
    }
    free(vertex_index);
    return 0;
}

/* ops/cpp/cootocsc_op.cc:23-53: the same, keyed on the destination row of
 * edge_index; the stored index is the source. */
int orc_cootocsc(const int32_t *edge_index, const float *coo_w, int64_t E,
                 int32_t v_num, int32_t *row_indices, int32_t *column_offset,
                 float *csc_w)
{
    memset(column_offset, 0, sizeof(int32_t) * ((size_t)v_num + 1));
    for (int64_t i = 0; i < E; i++)                 /* :33-35 */
        column_offset[edge_index[i + E] + 1] += 1;
    for (int32_t i = 0; i < v_num; i++)             /* :37-39 */
        column_offset[i + 1] += column_offset[i];
    int32_t *vertex_index = (int32_t *)calloc(v_num > 0 ? v_num : 1, sizeof(int32_t));
    if (!vertex_index) return -1;
    for (int64_t i = 0; i < E; i++) {               /* :43-51 */
        int32_t src = edge_index[i];
        int32_t dst = edge_index[i + E];
        int32_t index = vertex_index[dst]++;
        index += column_offset[dst];
        row_indices[index] = src;
        csc_w[index] = coo_w[i];
    }
    free(vertex_index);
    return 0;
}

/* ops/cpp/aggregate_op.cc:26-59 (AVX branch): out is zeroed by the caller in
 * the reference (ops/aggregateWithWeight.py:28); here it is zeroed first.
 * Rows are visited in order, edges of a row in order, features 8 at a time as
 * mul-then-add on the in-memory accumulator, then a scalar tail.  Row
 * addressing is widened to 64 bits (the reference multiplies in the index
 * type, :46), which changes nothing while V*F < 2^31. */
void orc_aggregate(float *out, const float *x, const int32_t *indices,
                   const int32_t *offset, const float *weight, int32_t v_num,
                   int32_t feature_dim)
{
    const int32_t LEN = 8;
    int32_t loop = feature_dim / LEN;
    memset(out, 0, sizeof(float) * (size_t)v_num * (size_t)feature_dim);
    for (int32_t i = 0; i < v_num; i++) {
        int32_t start = offset[i], end = offset[i + 1];
        float *o = out + (size_t)i * feature_dim;
        for (int32_t j = start; j < end; j++) {
            const float *xr = x + (size_t)indices[j] * feature_dim;
            __m256 w_val = _mm256_set1_ps(weight[j]);
            for (int32_t k = 0; k < loop; k++) {
                __m256 x_val = _mm256_loadu_ps(xr + k * LEN);
                __m256 out_val = _mm256_loadu_ps(o + k * LEN);
                _mm256_storeu_ps(o + k * LEN,
                                 _mm256_add_ps(_mm256_mul_ps(x_val, w_val), out_val));
            }
            for (int32_t k = LEN * loop; k < feature_dim; k++)   /* :54-56 */
                o[k] += xr[k] * weight[j];
        }
    }
}

/* ops/cpp/aggregate_op.cc:61-69 (non-AVX branch): plain scalar loops. */
void orc_aggregate_scalar(float *out, const float *x, const int32_t *indices,
                          const int32_t *offset, const float *weight,
                          int32_t v_num, int32_t feature_dim)
{
    memset(out, 0, sizeof(float) * (size_t)v_num * (size_t)feature_dim);
    for (int32_t i = 0; i < v_num; i++)
        for (int32_t j = offset[i]; j < offset[i + 1]; j++)
            for (int32_t k = 0; k < feature_dim; k++)
                out[(size_t)i * feature_dim + k] =
                    out[(size_t)i * feature_dim + k] +
                    x[(size_t)indices[j] * feature_dim + k] * weight[j];
}

/* Not a restatement of the reference: the same row sums with double accumulators,
 * i.e. the exact value of sum_j w[j] * x[indices[j],:] up to fp64 rounding.  The
 * reference's sequential fp32 sum drifts from it by up to (deg - 1) * 2^-24 of the sum
 * of the absolute terms (0.5 % on a row of 3.8 million same-sign terms); this is the
 * arbiter the tests hold both that loop and the kernels against.  terms (optional)
 * receives the sums of the absolute terms.  Pinned by scipy's fp64 sparse product. */
void orc_aggregate_f64(double *out, double *terms, const float *x, const int32_t *indices,
                       const int32_t *offset, const float *weight, int32_t v_num,
                       int32_t feature_dim)
{
    for (int32_t i = 0; i < v_num; i++) {
        double *o = out + (size_t)i * feature_dim;
        double *t = terms ? terms + (size_t)i * feature_dim : NULL;
        for (int32_t k = 0; k < feature_dim; k++) o[k] = 0.0;
        if (t) for (int32_t k = 0; k < feature_dim; k++) t[k] = 0.0;
        for (int32_t j = offset[i]; j < offset[i + 1]; j++) {
            const float *xr = x + (size_t)indices[j] * feature_dim;
            const double w = (double)weight[j];
            for (int32_t k = 0; k < feature_dim; k++) o[k] += w * (double)xr[k];
            if (t) for (int32_t k = 0; k < feature_dim; k++) t[k] += fabs(w) * fabs((double)xr[k]);
        }
    }
}

/* ops/cpp/edgesoftmax_op.cc:36-66.  One scalar per edge (x is [E] or [E,1]).
 * `exp` on a float argument resolves to the float overload in the
 * reference's C++ translation unit, hence expf here.  The reference reads
 * x[start] even for an empty column (:52); that read has no effect and is
 * skipped so that a trailing empty column cannot read past the array. */
void orc_edgesoftmax(float *out, const float *x, const int32_t *offset,
                     int32_t v_num)
{
    for (int32_t vtx = 0; vtx < v_num; vtx++) {
        int32_t start = offset[vtx], end = offset[vtx + 1];
        if (start >= end) continue;
        float total = 0;
        float max_weight = x[start];
        for (int32_t i = start; i < end; i++)
            if (max_weight < x[i]) max_weight = x[i];
        for (int32_t i = start; i < end; i++) {
            out[i] = x[i] - max_weight;
            total += expf(out[i]);
        }
        for (int32_t i = start; i < end; i++)
            out[i] = expf(out[i]) / total;
    }
}

/* Multi-head generalisation used by the 8-head GAT configuration: x is
 * [E,H] row-major and every head is an independent instance of
 * orc_edgesoftmax over the same columns.  H == 1 is the function above. */
void orc_edgesoftmax_heads(float *out, const float *x, const int32_t *offset,
                           int32_t v_num, int32_t H)
{
    for (int32_t vtx = 0; vtx < v_num; vtx++) {
        int32_t start = offset[vtx], end = offset[vtx + 1];
        if (start >= end) continue;
        for (int32_t h = 0; h < H; h++) {
            float total = 0;
            float max_weight = x[(size_t)start * H + h];
            for (int32_t i = start; i < end; i++)
                if (max_weight < x[(size_t)i * H + h]) max_weight = x[(size_t)i * H + h];
            for (int32_t i = start; i < end; i++) {
                out[(size_t)i * H + h] = x[(size_t)i * H + h] - max_weight;
                total += expf(out[(size_t)i * H + h]);
            }
            for (int32_t i = start; i < end; i++)
                out[(size_t)i * H + h] = expf(out[(size_t)i * H + h]) / total;
        }
    }
}

/* ops/cpp/edgesoftmaxbackward_op.cc:27-54.  x is the upstream gradient, y the
 * saved forward output.  The reference wraps the body in one more loop over
 * the column's edges (:44) that recomputes the same values deg times; one
 * iteration gives the identical result and is what is kept here. */
void orc_edgesoftmax_backward(float *out, const float *x, const float *y,
                              const int32_t *offset, int32_t v_num, int32_t H)
{
    for (int32_t vtx = 0; vtx < v_num; vtx++) {
        int32_t start = offset[vtx], end = offset[vtx + 1];
        for (int32_t h = 0; h < H; h++) {
            float dot = 0.0f;
            for (int32_t i = start; i < end; ++i)
                dot += y[(size_t)i * H + h] * x[(size_t)i * H + h];
            for (int32_t i = start; i < end; ++i)
                out[(size_t)i * H + h] =
                    (y[(size_t)i * H + h] * x[(size_t)i * H + h]) - y[(size_t)i * H + h] * dot;
        }
    }
}

/* ops/cpp/scattertoedge_op.cc:67-88 (edge_weight == nullptr branch, the only
 * one the Python wrapper reaches: ops/scatterToEdge.py:38 passes False).
 * flag 0: out[e,:] = x[indices[e],:]; flag 1: out[e,:] = x[vtx,:] for e in
 * the column of vtx.  The reference accumulates into zero-filled output. */
void orc_scattertoedge(float *out, const float *x, const int32_t *indices,
                       const int32_t *offset, int32_t v_num, int64_t e_num,
                       int32_t feature_dim, int32_t flag)
{
    memset(out, 0, sizeof(float) * (size_t)e_num * (size_t)feature_dim);
    for (int32_t vtx = 0; vtx < v_num; vtx++)
        for (int32_t i = offset[vtx]; i < offset[vtx + 1]; i++) {
            int32_t node = flag == 0 ? indices[i] : vtx;
            for (int32_t j = 0; j < feature_dim; j++)
                out[(size_t)i * feature_dim + j] =
                    out[(size_t)i * feature_dim + j] + x[(size_t)node * feature_dim + j];
        }
}

/* ops/cpp/edgetovertex_op.cc:36-55.  flag 0: out[indices[e],:] += x[e,:];
 * flag 1: out[vtx,:] += x[e,:] for e in the column of vtx; both in edge
 * order.  out has out_rows rows and is zeroed first. */
void orc_edgetovertex(float *out, const float *x, const int32_t *indices,
                      const int32_t *offset, int32_t v_num, int32_t out_rows,
                      int32_t feature_dim, int32_t flag)
{
    memset(out, 0, sizeof(float) * (size_t)out_rows * (size_t)feature_dim);
    for (int32_t vtx = 0; vtx < v_num; vtx++)
        for (int32_t i = offset[vtx]; i < offset[vtx + 1]; i++) {
            int32_t node = flag == 0 ? indices[i] : vtx;
            for (int32_t j = 0; j < feature_dim; j++)
                out[(size_t)node * feature_dim + j] =
                    out[(size_t)node * feature_dim + j] + x[(size_t)i * feature_dim + j];
        }
}

/* Seeded restatement of ops/cpp/sampleprocessing_op.cc:47-84: all neighbours
 * of dst[i] when it has at most `fanout` (or fanout < 0), else `fanout`
 * distinct ones.  The reference draws them with rand() (:66-69), which fixes
 * no answer; the draw here is Floyd's subset algorithm on a 64-bit mix of
 * (seed, destination, step), and the picks keep their order in g_idx. */
static uint32_t orc_sample_mix(uint64_t seed, uint32_t node, uint32_t step)
{
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (((uint64_t)node << 32) | step);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint32_t)(z >> 32);
}

int orc_sample_neighbors(const int32_t *dst, const int32_t *layer_off, const int32_t *g_off,
                         const int32_t *g_idx, int32_t n_dst, int32_t fanout, uint64_t seed,
                         int32_t *out)
{
    for (int32_t i = 0; i < n_dst; i++) {
        int32_t pos = layer_off[i];
        int32_t cap = layer_off[i + 1] - pos;
        int32_t node = dst[i];
        int32_t start = g_off[node];
        int32_t deg = g_off[node + 1] - start;
        if (cap <= 0 || deg <= 0) continue;
        if (fanout < 0 || deg <= fanout) {
            for (int32_t j = 0; j < deg && j < cap; j++) out[pos + j] = g_idx[start + j];
            continue;
        }
        int32_t k = fanout < cap ? fanout : cap;
        int32_t *mine = out + pos;
        int32_t have = 0;
        for (int32_t j = deg - k; j < deg; j++) {
            uint32_t r = orc_sample_mix(seed, (uint32_t)node, (uint32_t)(j - (deg - k)));
            int32_t t = (int32_t)(((uint64_t)r * (uint64_t)(j + 1)) >> 32);
            int taken = 0;
            for (int32_t q = 0; q < have; q++) taken |= mine[q] == t;
            if (taken) t = j;
            int32_t q = have;
            while (q > 0 && mine[q - 1] > t) {
                mine[q] = mine[q - 1];
                q--;
            }
            mine[q] = t;
            have++;
        }
        for (int32_t q = 0; q < k; q++) mine[q] = g_idx[start + mine[q]];
    }
    return 0;
}
