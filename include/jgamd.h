/*
 * jgamd — C ABI of the MI355X (gfx950) sparse message-passing kernels.
 *
 * Drop-in boundary for the native half of jittor_geometric.ops: every entry
 * point replaces one Jittor custom Op (or one jittor-wheel cuSPARSE op) of the
 * reference; the citation above each declaration names it.
 *
 * Conventions (all entry points):
 *   - extern "C", plain pointers and sizes; no C++ or torch types.
 *   - All data pointers are DEVICE pointers to contiguous arrays; indices are
 *     int32, values fp32 (the only combination the reference's hot path uses:
 *     data/data.py:103-106 casts edge_index to int32).
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream).  Nothing synchronises the device; nothing allocates or
 *     frees device memory: scratch comes in through `ws` / `ws_bytes`, sized by
 *     the matching *_workspace() query (host-only arithmetic, needs no GPU).
 *   - Return value: 0 = enqueued; negative = argument error found on the host
 *     (nothing was enqueued); positive = a hipError_t from a launch.
 *     jgamd_last_error() returns a thread-local description of the last
 *     non-zero status.
 *   - Outputs are overwritten (beta = 0); they need not be zeroed by the
 *     caller, unlike the reference ops which accumulate into zero-filled Vars.
 *   - Calls are re-entrant; two calls may overlap on one GPU when they use
 *     different workspaces and outputs.
 */
#ifndef JGAMD_H
#define JGAMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JGAMD_OK 0
#define JGAMD_ERR_NULL (-1)        /* a required pointer is NULL              */
#define JGAMD_ERR_SIZE (-2)        /* negative / overflowing / inconsistent size */
#define JGAMD_ERR_WORKSPACE (-3)   /* ws is NULL or smaller than the query says */
#define JGAMD_ERR_UNSUPPORTED (-4) /* shape outside what the kernels handle   */
#define JGAMD_ERR_ALIGN (-5)       /* pointer not 4-byte aligned              */

/* flag of the entry points that finish output rows: clamp the row at zero (ReLU) */
#define JGAMD_ROW_RELU 1
/* jgamd_spmm_csx_planned, or-ed into `flags`: the rows of x lie n floats apart (n >= F, a
 * multiple of 4; a producer that pads its rows to whole 128-byte lines, e.g. a BLAS product
 * written with that leading dimension, spares the gathers the lines an odd width straddles) */
#define JGAMD_ROW_X_STRIDE(n) ((int32_t)(n) << 8)

/* Library version, major*10000 + minor*100 + patch. */
int32_t jgamd_version(void);
/* Thread-local text of the last error returned on this thread ("" if none). */
const char *jgamd_last_error(void);

/* ------------------------------------------------------------------------
 * COO -> CSR / CSC.
 * Replaces CootocsrOp::jit_run (ops/cpp/cootocsr_op.cc:24-57, Python wrapper
 * ops/cootocsr.py:28-35) with key_row = 0 and CootocscOp::jit_run
 * (ops/cpp/cootocsc_op.cc:23-53, ops/cootocsc.py:29-36) with key_row = 1.
 *
 *   edge_index [2,E] row-major: row 0 = source, row 1 = destination
 *   key_row    0: group by source (CSR; out_idx = destinations)
 *              1: group by destination (CSC; out_idx = sources)
 *   out_off    [V+1]  out_idx [E]  out_w [E]
 *   out_perm   optional [E]: original edge id stored at each output slot
 *              (NULL to skip).  Not produced by the reference; used to move
 *              per-edge tensors between the CSR and CSC orders.
 *
 * Result is bit-identical to the reference: a stable counting sort, i.e.
 * inside a row the edges keep their input order; weights are copied.
 * Edges whose key is outside [0,V) are dropped (the reference would write out
 * of bounds); out_off[V] is then below E and the slots of out_idx / out_w /
 * out_perm from out_off[V] on are set to zero.
 * Limits: 0 <= E < 2^31 - 2^20, 0 <= V < 2^31 - 1 (V <= 2^22 takes the
 * two-level path, larger V plain radix passes over the same records).
 */
int32_t jgamd_coo_to_csx_workspace(int64_t E, int32_t V, int32_t with_perm, size_t *bytes);
int32_t jgamd_coo_to_csx(const int32_t *edge_index, const float *edge_weight, int64_t E,
                         int32_t V, int32_t key_row, int32_t *out_idx, int32_t *out_off,
                         float *out_w, int32_t *out_perm, void *ws, size_t ws_bytes,
                         void *stream);

/* Transpose of a compressed structure (CSR of an R x C matrix -> CSC arrays of
 * the same matrix, or the reverse): expands the row ids and runs the stable
 * conversion keyed on idx.  No single reference op; it is what
 * SpmmCsr(trans_A=True) (ops/spmmcsr.py:31, cuSPARSE op(A)=T inside the
 * jittor wheel) and the flag-0 edgetovertex backward
 * (ops/cpp/edgetovertex_op.cc:36-45) need to run as gathers instead of
 * scatters.  out_off has C+1 entries.  out_w / out_perm / w may be NULL.
 */
int32_t jgamd_csx_transpose_workspace(int64_t E, int32_t R, int32_t C, size_t *bytes);
int32_t jgamd_csx_transpose(const int32_t *off, const int32_t *idx, const float *w, int32_t R,
                            int32_t C, int64_t E, int32_t *out_off, int32_t *out_idx,
                            float *out_w, int32_t *out_perm, void *ws, size_t ws_bytes,
                            void *stream);

/* inv[perm[i]] = i for a permutation of [0,n) (entries outside the range are
 * skipped).  No reference counterpart: it turns the out_perm of
 * jgamd_csx_transpose (transposed slot -> original slot) into the map
 * original slot -> transposed slot that jgamd_gat_bwd gathers through.
 */
int32_t jgamd_invert_permutation(const int32_t *perm, int64_t n, int32_t *inv, void *stream);

/* ------------------------------------------------------------------------
 * Weighted row-gather SpMM:  out[r,:] = sum_{j in [off[r],off[r+1])} w[j] * x[idx[j],:]
 * Replaces AggregateOp::jit_run (ops/cpp/aggregate_op.cc:26-71 CPU,
 * :74-106 CUDA; wrapper ops/aggregateWithWeight.py:20-41: forward passes the
 * CSC arrays, backward the CSR arrays) and cusparse_ops.cusparse_spmmcsr as
 * called by ops/spmmcsr.py:31,37.
 *
 *   off [R+1], idx [E], w [E], x [C,F] (leading dimension F), out [R,F]
 *   idx == NULL means idx[j] = j (x is then per-edge, [E,F]); w == NULL means 1.
 *   With those two the same entry point is EdgetovertexOp::jit_run
 *   (ops/cpp/edgetovertex_op.cc:36-55): flag 1 = (idx NULL, w NULL) over the
 *   CSC offsets; flag 0 = (idx = perm, w NULL) over the transposed offsets.
 *
 * Rows are summed in edge order inside one wavefront's share of the edges and
 * pieces of a row that span several wavefronts are added in edge order by a
 * second kernel: results are run-to-run reproducible (no float atomics) and
 * agree with the sequential reference sum to fp32 rounding.
 * Entries with idx outside [0,C) contribute nothing.
 * Limits: E + R < 2^31, 1 <= F <= 65535*2048.
 * Environment: JGAMD_SPMM_CHUNK=<16..4096> overrides the number of merged items
 * per wavefront; JGAMD_SPMM_STAGE=lds|reg forces how (idx, w) are staged
 * (tuning aids; read once per process).
 */
int32_t jgamd_spmm_csx_workspace(int32_t R, int64_t E, int32_t F, size_t *bytes);
int32_t jgamd_spmm_csx(const int32_t *off, const int32_t *idx, const float *w, const float *x,
                       float *out, int32_t R, int32_t C, int64_t E, int32_t F, void *ws,
                       size_t ws_bytes, void *stream);

/* jgamd_spmm_csx with a row finish:
 *   out[r,:] = beta * sum_j w[j] * x[idx[j],:] + alpha * h[r,:]
 * h is [h_rows,F] with h_rows = R, or 1 for one row added to every output row
 * (a layer's bias: nn/conv/gcn_conv.py:109-110 adds it after the product);
 * NULL or alpha == 0 drops the term.  h may be x itself; out must not overlap
 * x or h.  One call is one hop of the reference's polynomial
 * propagation layers, whose Python loop runs the product and then two
 * element-wise passes (nn/conv/appnp_conv.py:42-51: x = propagate(x);
 * x = x * (1 - alpha); x = x + alpha * h).  Same workspace as jgamd_spmm_csx.
 */
int32_t jgamd_spmm_csx_axpby(const int32_t *off, const int32_t *idx, const float *w,
                             const float *x, float *out, float beta, float alpha,
                             const float *h, int32_t h_rows, int32_t R, int32_t C, int64_t E,
                             int32_t F, void *ws, size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Per-graph plans.  The reference's aggregate is one launch per call
 * (ops/cpp/aggregate_op.cc:93-106); how the merge-path kernels here cut a
 * matrix into chunks, and which chunks hold pieces of a cut row, depends on the
 * offsets alone, so it can be computed once per graph, kept by the caller (like
 * the CSR / CSC objects themselves, data/data.py:42-52) and handed to the
 * *_planned entry points, which then skip the per-call search and launch the
 * piece kernels over the listed chunks only.  A plan is an opaque block of
 * device memory owned by the caller, 256-byte aligned, valid for the offsets
 * array (contents, R, E) it was built from; results with and without a plan are
 * bit-identical.
 *
 *   kind  JGAMD_PLAN_SPMM   chunks for jgamd_spmm_csx_planned
 *         JGAMD_PLAN_GAT    chunks for jgamd_gat_fwd / jgamd_gat_bwd (of the
 *                           CSC offsets / of the transposed offsets)
 *         JGAMD_PLAN_TILES  tile -> column map for jgamd_edge_softmax_*_planned
 *                           and for products with rows of 1, 2, 4 or 8 floats
 *
 * jgamd_csx_plan_counts copies the lengths of the two chunk lists of a SPMM /
 * GAT plan to the host (it waits for `stream`: the one synchronising call of
 * this library besides the *_timed ones).  Passing them as n_fix / n_grp lets a
 * planned call size or skip its piece kernels: 0 = the list is empty, nothing
 * is launched for it (a graph without rows longer than half a chunk is then
 * one launch per product); -1 = unknown, the kernels read the lengths from the
 * plan.
 */
#define JGAMD_PLAN_SPMM 0
#define JGAMD_PLAN_GAT 1
#define JGAMD_PLAN_TILES 2
int32_t jgamd_csx_plan_bytes(int32_t R, int64_t E, int32_t kind, size_t *bytes);
int32_t jgamd_csx_plan(const int32_t *off, int32_t R, int64_t E, int32_t kind, void *plan,
                       size_t plan_bytes, void *stream);
int32_t jgamd_csx_plan_counts(const void *plan, int32_t *n_fix, int32_t *n_grp, void *stream);

/* jgamd_spmm_csx_axpby with the partition taken from a plan of `off`:
 * plan = a JGAMD_PLAN_SPMM plan, tiles = a JGAMD_PLAN_TILES plan (either may be
 * NULL, not both).  The plain product (beta = 1, alpha = 0 or h = NULL, no
 * flags: AggregateOp::jit_run, ops/cpp/aggregate_op.cc:26-71) at rows of 1, 2,
 * 4 or 8 floats, x aligned to min(16, 4 F) bytes, uses `tiles` when it is
 * given; every other width, and any product with a row finish, needs `plan`
 * and is refused with JGAMD_ERR_NULL when only `tiles` came.
 * flags: JGAMD_ROW_RELU clamps every finished row at zero in the row store,
 * out = max(0, beta * A x + alpha * h): the activation the reference's models
 * apply in a pass of their own after the layer (examples/gcn_example.py:84-90).
 * The workspace holds row pieces only (jgamd_spmm_csx_planned_workspace).
 */
int32_t jgamd_spmm_csx_planned_workspace(int32_t R, int64_t E, int32_t F, size_t *bytes);
int32_t jgamd_spmm_csx_planned(const void *plan, const void *tiles, int32_t n_fix, int32_t n_grp,
                               const int32_t *off, const int32_t *idx, const float *w,
                               const float *x, float *out, float beta, float alpha,
                               const float *h, int32_t h_rows, int32_t flags, int32_t R,
                               int32_t C, int64_t E, int32_t F, void *ws, size_t ws_bytes,
                               void *stream);

/* jgamd_spmm_csx without a workspace argument.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory or own a
 * workspace (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  Same kernels, same result bit for bit; the scratch
 * (chunk rows, row pieces, group sums) is a fixed 64 MiB device array inside
 * the library, one copy per GPU, held until the process ends.
 *   - Shapes whose jgamd_spmm_csx_workspace() exceeds 64 MiB are rejected with
 *     JGAMD_ERR_SIZE and nothing is enqueued (the 1M-node / 17M-entry graph at
 *     F = 128 needs 36 MiB).
 *   - Calls no hipMalloc / hipFree or allocating routine.  The first call on
 *     a device looks up the array's address (hipGetSymbolAddress) with that
 *     device current and keeps it; make that call outside a stream capture.
 *   - All calls on one GPU share the array: two calls that overlap in time on
 *     one GPU (different streams) race.  Calls on one stream are ordered.
 */
int32_t jgamd_spmm_csx_noalloc(const int32_t *off, const int32_t *idx, const float *w,
                               const float *x, float *out, int32_t R, int32_t C, int64_t E,
                               int32_t F, void *stream);

/* Benchmark support; no counterpart in the reference.  Runs the product
 * `iters` times on `stream` (jgamd_spmm_csx_planned with `plan`, n_fix, n_grp,
 * or jgamd_spmm_csx when plan is NULL), with one hipEvent pair around each
 * launch of the gather kernel (spmm_merge) and one around each whole call,
 * WAITS for the stream after every call, and returns the two mean durations
 * in milliseconds.  Unlike every other entry point it synchronises and
 * creates/destroys events. */
int32_t jgamd_spmm_csx_timed(const void *plan, int32_t n_fix, int32_t n_grp, const int32_t *off,
                             const int32_t *idx, const float *w, const float *x, float *out,
                             int32_t R, int32_t C, int64_t E, int32_t F, void *ws,
                             size_t ws_bytes, void *stream, int32_t iters, float *kernel_ms,
                             float *call_ms);

/* ------------------------------------------------------------------------
 * Edge softmax over the in-edges of every destination (CSC column).
 * Replaces EdgesoftmaxOp::jit_run (ops/cpp/edgesoftmax_op.cc:36-66, the
 * max-subtracted CPU form; wrapper ops/edgesoftmax.py:62-69) and
 * EdgesoftmaxbackwardOp::jit_run (ops/cpp/edgesoftmaxbackward_op.cc:27-54,
 * wrapper ops/edgesoftmax.py:71-74).
 *   x, y, g, dx are [E,H] row-major; H = 1 is the reference's shape ([E] or
 *   [E,1]); H > 1 treats every head as an independent softmax.
 *   fwd:  y = exp(x - max_col) / sum_col exp(x - max_col)
 *   bwd:  dx = y*g - y*sum_col(y*g)
 * The workspace holds the list of hub columns (more than 512 entries), which
 * get a whole thread block each.
 */
int32_t jgamd_edge_softmax_workspace(int32_t V, int64_t E, size_t *bytes);
int32_t jgamd_edge_softmax_fwd(const int32_t *off, const float *x, float *y, int32_t V,
                               int64_t E, int32_t H, void *ws, size_t ws_bytes, void *stream);
int32_t jgamd_edge_softmax_bwd(const int32_t *off, const float *y, const float *g, float *dx,
                               int32_t V, int64_t E, int32_t H, void *ws, size_t ws_bytes,
                               void *stream);
/* The same two with the tile -> column map taken from a JGAMD_PLAN_TILES plan
 * of `off` instead of being computed by a launch of its own per call (1, 2, 4
 * and 8 heads use it; other head counts ignore it). */
int32_t jgamd_edge_softmax_fwd_planned(const void *tiles, const int32_t *off, const float *x,
                                       float *y, int32_t V, int64_t E, int32_t H, void *ws,
                                       size_t ws_bytes, void *stream);
int32_t jgamd_edge_softmax_bwd_planned(const void *tiles, const int32_t *off, const float *y,
                                       const float *g, float *dx, int32_t V, int64_t E,
                                       int32_t H, void *ws, size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Vertex -> edge copy.  Replaces ScattertoedgeOp::jit_run
 * (ops/cpp/scattertoedge_op.cc:67-88 CPU, :91-137 CUDA; wrapper
 * ops/scatterToEdge.py:22-40).  flag 0: out[e,:] = x[idx[e],:] ("src");
 * flag 1: out[e,:] = x[v,:] for every e in column v ("dst").
 *   off [V+1], idx [E], x [V,F], out [E,F].
 */
int32_t jgamd_scatter_to_edge(const int32_t *off, const int32_t *idx, const float *x,
                              float *out, int32_t V, int64_t E, int32_t F, int32_t flag,
                              void *stream);

/* ------------------------------------------------------------------------
 * Fused GAT layer core (attention logits + edge softmax + weighted
 * aggregation) over the CSC arrays.  Replaces the op chain of
 * GATConv.propagate (nn/conv/gat_conv.py:61-83): ScatterToEdge x2, concat,
 * [E,2C]x[2C,1] product, leaky_relu, EdgeSoftmax, multiply, ScatterToVertex.
 *   h      [V,H,D]   node features after vertex_forward
 *   a_src  [H,D], a_dst [H,D]  the two halves of GATConv.edge_weight
 *   el,er  [V,H]  outputs: a_src.h and a_dst.h per node and head; both NULL
 *          when no backward pass follows (pos, spos and alpha then NULL as
 *          well): the scores are then taken inside the aggregation kernel and
 *          the pass over h that computes the two arrays is not run
 *   smax, ssum [V,H] outputs: per destination and head, the max logit and
 *          the sum of exp(logit - max) (what backward needs to rebuild alpha)
 *   pos [V,H,D], spos [V,H]  optional outputs (both or neither): the share of
 *          out / of the attention that lies on edges with a positive logit,
 *          pos[v,k,:] = sum_{e: z_e > 0} alpha[e,k] h[idx[e],k,:],
 *          spos[v,k] = sum_{e: z_e > 0} alpha[e,k].  jgamd_gat_bwd takes them:
 *          with LeakyReLU' in {1, slope} they give the gradient with respect
 *          to er per node, without a second pass over the edges.
 *   alpha  optional [E,H] output (NULL to skip): attention per CSC slot
 *   out    [V,H,D]:  out[v,k,:] = sum_e alpha[e,k] * h[idx[e],k,:]
 *   plan   a JGAMD_PLAN_GAT plan of `off` with its list lengths n_fix / n_grp
 *          (see jgamd_csx_plan), or NULL (n_fix, n_grp ignored)
 * H = 1, D = C reproduces the reference's single head.
 */
int32_t jgamd_gat_fwd_workspace(int32_t V, int64_t E, int32_t H, int32_t D, size_t *bytes);
int32_t jgamd_gat_fwd(const void *plan, int32_t n_fix, int32_t n_grp, const int32_t *off,
                      const int32_t *idx, const float *h, const float *a_src,
                      const float *a_dst, float slope, float *el, float *er, float *smax,
                      float *ssum, float *pos, float *spos, float *alpha, float *out, int32_t V,
                      int64_t E, int32_t H, int32_t D, void *ws, size_t ws_bytes, void *stream);

/* Backward of jgamd_gat_fwd, one pass over the transposed arrays (t_off, t_idx)
 * of the graph as produced by jgamd_csx_transpose (rows = sources); t_plan is a
 * JGAMD_PLAN_GAT plan of t_off, or NULL.
 * With H > 1 the head width D must span a power-of-two number of lanes
 * (D in {1,2,4,...,256}); other shapes return JGAMD_ERR_UNSUPPORTED and are
 * served by the unfused operator chain.
 *   el, er, smax, ssum, spos, out, pos: what jgamd_gat_fwd wrote
 *   g_out [V,H,D] upstream gradient
 *   g_h   [V,H,D], g_a_src [H,D], g_a_dst [H,D] outputs
 * Replaces the grad chain edgetovertex <-> scattertoedge <->
 * edgesoftmaxbackward that Jittor autograd builds for gat_conv.py:61-83.
 */
int32_t jgamd_gat_bwd_workspace(int32_t V, int64_t E, int32_t H, int32_t D, size_t *bytes);
int32_t jgamd_gat_bwd(const void *t_plan, int32_t n_fix, int32_t n_grp, const int32_t *t_off,
                      const int32_t *t_idx, const float *h, const float *a_src,
                      const float *a_dst, float slope, const float *el, const float *er,
                      const float *smax, const float *ssum, const float *spos, const float *out,
                      const float *pos, const float *g_out, float *g_h, float *g_a_src,
                      float *g_a_dst, int32_t V, int64_t E, int32_t H, int32_t D, void *ws,
                      size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Column-blocked product for matrices with long rows (hundreds of entries
 * per row, x larger than an L2): the same result as jgamd_spmm_csx_axpby,
 * out = beta * (A x) + alpha * h, with the gathers of x confined to one block
 * of columns at a time.  Follows the same reference loops as jgamd_spmm_csx
 * (aggregate_op.cc:107-114, spmmcsr_op.cc:81-127); the reference has no
 * blocked layout.  Sums differ from the unblocked kernels' in rounding only
 * (per-block partial sums added in block order; no atomics, run-to-run
 * identical).
 *
 * jgamd_spmm_block_plan: *nb = number of column blocks and *block_cols =
 * columns per block that pay for this shape, or *nb = 0 when the unblocked
 * product is the better one (short rows, x that fits, too many blocks).
 *
 * jgamd_csx_block_columns: regroups the entries of every row by column block,
 * keeping their order inside a block: b_off [nb*R+1], b_idx [E], b_w [E]
 * (w and b_w may both be NULL); row b*R + r of the result holds the entries
 * of row r whose column lies in [b*block_cols, (b+1)*block_cols), the last
 * block taking what lies beyond.  Entries from off[R] on are not part of it.
 * Done once per matrix; nb <= 64.
 *
 * jgamd_spmm_csx_blocked: the product over arrays made by that call.  When F
 * is not a multiple of 32 the rows of x are first copied 128-byte aligned into
 * the workspace (one pass over x), so that the gathered pieces are whole lines.
 */
int32_t jgamd_spmm_block_plan(int32_t R, int32_t C, int64_t E, int32_t F, int32_t *nb,
                              int32_t *block_cols);
int32_t jgamd_csx_block_columns_workspace(int32_t R, int32_t nb, size_t *bytes);
int32_t jgamd_csx_block_columns(const int32_t *off, const int32_t *idx, const float *w, int32_t R,
                                int64_t E, int32_t block_cols, int32_t nb, int32_t *b_off,
                                int32_t *b_idx, float *b_w, void *ws, size_t ws_bytes,
                                void *stream);
int32_t jgamd_spmm_csx_blocked_workspace(int32_t R, int32_t C, int64_t E, int32_t F, int32_t nb,
                                         size_t *bytes);
int32_t jgamd_spmm_csx_blocked(const int32_t *b_off, const int32_t *b_idx, const float *b_w,
                               const float *x, float *out, float beta, float alpha,
                               const float *h, int32_t h_rows, int32_t R, int32_t C, int64_t E,
                               int32_t F, int32_t nb, void *ws, size_t ws_bytes, void *stream);
/* measurement aid, as jgamd_spmm_csx_timed: the plain product (beta 1, alpha 0) `iters` times,
 * mean milliseconds of the gather kernel and of the whole call from HIP events on `stream` */
int32_t jgamd_spmm_csx_blocked_timed(const int32_t *b_off, const int32_t *b_idx, const float *b_w,
                                     const float *x, float *out, int32_t R, int32_t C, int64_t E,
                                     int32_t F, int32_t nb, void *ws, size_t ws_bytes, void *stream,
                                     int32_t iters, float *kernel_ms, float *call_ms);

/* ------------------------------------------------------------------------
 * Dense feature transform of the conv layers on the matrix cores (fp32 in,
 * fp32 accumulate): out[V,N] = x1[V,K1] @ w1[K1,N] (+ x2[V,K2] @ w2[K2,N])
 * (+ bias[N]).  Replaces `x @ self.weight` (nn/conv/gcn_conv.py:95) and
 * `out @ weight1 + x @ root_weight + bias` (nn/conv/sage_conv.py:186-190),
 * which Jittor runs as cuBLAS products and element-wise additions.  K1, K2
 * and N must be multiples of 4 with K1 + K2 <= 256 (jgamd_dense_rows_supported
 * returns 1 for such a shape, else 0; other shapes stay with the BLAS
 * library); x1, x2, out and bias 16-byte aligned.  K2 = 0 leaves out the
 * second product, bias = NULL the added row.  flags: JGAMD_ROW_RELU clamps
 * the result at zero in the store (see jgamd_spmm_csx_planned).  Needs no
 * workspace.
 */
int32_t jgamd_dense_rows_supported(int32_t K1, int32_t K2, int32_t N);
int32_t jgamd_dense_rows(const float *x1, const float *w1, int32_t K1, const float *x2,
                         const float *w2, int32_t K2, const float *bias, float *out, int32_t V,
                         int32_t N, int32_t flags, void *stream);

/* ------------------------------------------------------------------------
 * Column sums of a row-major [R,F] matrix: out[f] = sum_r x[r,f].  The bias
 * gradient of the conv layers (`out += self.bias`, nn/conv/gcn_conv.py:100-101,
 * nn/conv/sage_conv.py:189-190; Jittor derives the reduction).  Two stages,
 * fixed order, no atomics.
 */
int32_t jgamd_column_sum_workspace(int64_t R, int32_t F, size_t *bytes);
int32_t jgamd_column_sum(const float *x, float *out, int64_t R, int32_t F, void *ws,
                         size_t ws_bytes, void *stream);

/* The gradient in front of a ReLU and its column sums in one pass:
 *   masked[r,c] = y[r,c] > 0 ? g[r,c] : 0,   out[c] = sum_r masked[r,c]
 * for the upstream gradient g and the ReLU's output y, both [R,F]; masked must
 * not be g.  Together with JGAMD_ROW_RELU this is the backward of a layer whose
 * activation was applied in the product's row store: the bias gradient reads
 * the upstream gradient anyway (nn/conv/gcn_conv.py:109-110 adds the bias,
 * examples/gcn_example.py:84-90 applies relu after the layer).  Same workspace
 * as jgamd_column_sum.
 */
int32_t jgamd_relu_backward_column_sum(const float *g, const float *y, float *masked, float *out,
                                       int64_t R, int32_t F, void *ws, size_t ws_bytes,
                                       void *stream);

/* ------------------------------------------------------------------------
 * Mean cross-entropy of row-major logits [V,C] against integer labels, the
 * loss of the full-graph training step (nn.cross_entropy_loss(pred, label),
 * examples/gcn_example.py:113; nn.log_softmax + nn.nll_loss,
 * examples/sage_example.py:69,83 — both live in the jittor package):
 *   lse[i] = log sum_c exp(logits[i,c])           (max-subtracted)
 *   loss   = mean over rows with 0 <= label < C of (lse[i] - logits[i,label[i]])
 * Rows whose label lies outside [0,C) are left out of the mean and get a zero
 * gradient.  labels: int32, or int64 when labels_are_i64 != 0.  loss[1],
 * count[1] (rows counted) and lse[V] are written by fwd and read by bwd:
 *   grad_logits[i,c] = grad_loss[0] / count * (exp(logits[i,c] - lse[i]) - [c == label[i]])
 * (grad_loss NULL = 1).  log_probs != 0: the rows already are log-probabilities
 * (nn.nll_loss): loss = mean of -logits[i,label[i]], lse is written as +inf
 * and bwd then yields -[c == label[i]] * grad_loss[0] / count.  Two
 * fixed-order reduction stages, no atomics.
 */
int32_t jgamd_cross_entropy_workspace(int64_t V, int32_t C, size_t *bytes);
int32_t jgamd_cross_entropy_fwd(const float *logits, const void *labels, int32_t labels_are_i64,
                                int32_t log_probs, int64_t V, int32_t C, float *loss,
                                int32_t *count, float *lse, void *ws, size_t ws_bytes,
                                void *stream);
int32_t jgamd_cross_entropy_bwd(const float *logits, const void *labels, int32_t labels_are_i64,
                                const float *lse, const int32_t *count, const float *grad_loss,
                                int64_t V, int32_t C, float *grad_logits, void *stream);

/* ------------------------------------------------------------------------
 * Neighbour sampling for one layer of a sampled subgraph: for destination
 * dst[i] (a column of the global CSC arrays g_off / g_idx with g_nodes
 * columns) write its neighbours to out[layer_off[i] .. layer_off[i+1]): all of
 * them, in order, when it has at most `fanout` (or fanout < 0), else `fanout`
 * distinct ones, in the order they have in g_idx.  Replaces
 * sampleprocessing_op.sampleprocessing(fanout, dst, column_offset,
 * row_indices, global_column_offset, global_row_indices)
 * (ops/sampleprocessing.py:34, ops/cpp/sampleprocessing_op.cc:47-84,88-160).
 * The reference draws from rand() / a clock-seeded curand state; here the
 * draw is a pure function of (seed, destination id).  fanout <= 1024.
 */
int32_t jgamd_sample_neighbors(const int32_t *dst, const int32_t *layer_off, const int32_t *g_off,
                               const int32_t *g_idx, int32_t n_dst, int32_t g_nodes,
                               int32_t fanout, int64_t out_len, uint64_t seed, int32_t *out,
                               void *stream);

/* ------------------------------------------------------------------------
 * List lengths and offsets of a layer's destinations.
 *
 * jgamd_layer_column_counts: counts[0] = 0, counts[i+1] = min(size of column
 * dst[i] of the global CSC offsets g_off, cap) for i < n_dst; counts holds
 * n_dst + 1 int32.  Replaces gpuinitco_op.gpuinitco(dst_size, fanout, dst,
 * column_offset, global_column_offset) (ops/gpuinitco.py:30-36; the kernel
 * of ops/cpp/gpuinitco_op.cc:38-52, whose caller turns the counts into
 * offsets afterwards).  A destination outside [0, g_nodes) counts 0.
 *
 * jgamd_layer_column_offsets: offsets[i] = sum of those lengths over the
 * destinations before i, offsets[n_dst] = their total (n_dst + 1 int32):
 * the slicing loops of ops/saparse_ops.py:9-71 (from_nodes / to_nodes) size
 * their result this way, one node at a time.
 */
int32_t jgamd_layer_column_counts(const int32_t *dst, const int32_t *g_off, int32_t n_dst,
                                  int32_t g_nodes, int32_t cap, int32_t *counts, void *stream);
int32_t jgamd_layer_column_offsets_workspace(int32_t n_dst, size_t *bytes);
int32_t jgamd_layer_column_offsets(const int32_t *dst, const int32_t *g_off, int32_t n_dst,
                                   int32_t g_nodes, int32_t cap, int32_t *offsets, void *ws,
                                   size_t ws_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Symmetric-normalisation weights of a layer's CSC arrays: with
 * ins[dst[i]] += size of column i and outs[row[j]] += 1 over the entries
 * below off[n_dst], w[j] = 1 / (sqrtf(outs[row[j]]) * sqrtf(ins[dst[i]]))
 * for entry j of column i.  Replaces getweight_op.getweight(vtx_size, dst,
 * src, column_offset, row_indices, edge_weight) (ops/getweight.py:29-37,
 * ops/cpp/getweight_op.cc:49-81, same float operations in the same order).
 * The degrees are integer counts, so their order of accumulation does not
 * matter.  Entries from off[n_dst] to E get weight 0.  An id outside
 * [0, vtx_size), which the reference would use as an index out of bounds,
 * is skipped wherever it would be one: its entries get weight 0 and it adds
 * to no degree.
 */
int32_t jgamd_getweight_workspace(int32_t vtx_size, size_t *bytes);
int32_t jgamd_getweight(const int32_t *dst, const int32_t *off, const int32_t *row, int32_t n_dst,
                        int32_t vtx_size, int64_t E, float *w, void *ws, size_t ws_bytes,
                        void *stream);

/* ------------------------------------------------------------------------
 * Graph preprocessing in front of the conversion.
 *
 * jgamd_add_remaining_self_loops: utils/loop.py:98-136 — the input's
 * self-loops are dropped, the other edges keep their order, one loop per
 * node is appended; a node's loop takes the weight of its last dropped loop,
 * else `fill`.  out_index must hold 2*(E+N) int32, out_weight E+N floats;
 * *out_kept (device) receives the number of kept edges K, and the result is
 * out_index[0..K+N) (rows) followed directly by out_index[K+N..2(K+N)) (cols),
 * out_weight[0..K+N).  edge_weight may be NULL (weights of one).
 *
 * jgamd_degree_power: out[v] = deg[v]^power with inf -> 0
 * (nn/conv/gcn_conv.py:35-36).  jgamd_scale_edge_weights:
 * out[e] = by_row[row[e]] * w[e] * by_col[col[e]] (either factor array may be
 * NULL) — gcn_conv.py:37, sage_conv.py:40.
 *
 * jgamd_scale_csx_weights: the same product for weights already in compressed
 * order, out[j] = by_idx[idx[j]] * w[j] * by_seg[c] for every slot j of segment
 * c of (off, idx) — term for term what jgamd_scale_edge_weights gives for the
 * edge in that slot, so a caller that has sorted an edge list once (to sum the
 * degrees) gets the normalised weights of the compressed arrays without
 * converting the edge list again (examples/gcn_example.py:48-59 calls gcn_norm,
 * then cootocsc on its result).  N bounds the factor arrays; slots past off[V]
 * are set to zero.
 */
int32_t jgamd_add_remaining_self_loops_workspace(int64_t E, int32_t N, size_t *bytes);
int32_t jgamd_add_remaining_self_loops(const int32_t *edge_index, const float *edge_weight,
                                       int64_t E, int32_t N, float fill, int32_t *out_index,
                                       float *out_weight, int32_t *out_kept, void *ws,
                                       size_t ws_bytes, void *stream);
int32_t jgamd_degree_power(const float *deg, int32_t N, float power, float *out, void *stream);
int32_t jgamd_scale_csx_weights_workspace(int64_t E, size_t *bytes);
int32_t jgamd_scale_csx_weights(const int32_t *off, const int32_t *idx, const float *w,
                                const float *by_idx, const float *by_seg, int32_t V, int64_t E,
                                int32_t N, float *out, void *ws, size_t ws_bytes, void *stream);
int32_t jgamd_scale_edge_weights(const int32_t *edge_index, const float *edge_weight,
                                 const float *by_row, const float *by_col, int64_t E, int32_t N,
                                 float *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* JGAMD_H */
