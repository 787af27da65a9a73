"""TEST INFRASTRUCTURE — CPU oracle of the sparse message-passing path.

`oracle.c` restates the reference's single-threaded CPU loops in plain C;
this module loads it with ctypes and adds numpy restatements of the Python
code either side of those loops (graph normalisation, the GAT composition,
the layer wrappers).  Only tests, the smoke check and the CPU-baseline leg of
the benchmark import this package; the shipped library never does.

Functions with no independent pin (see oracle.c header for the pins of the
rest): none of the arithmetic.  The cuSPARSE-internal summation order behind
the reference's SpmmCsr and SpmmCoo is "parity unpinned" (third-party,
jittor==1.3.9.14).  Pins of the numpy restatements at the end of this file:
  gat_backward  float64 autograd of the same layer on a small graph, a directional
                finite difference of gat_forward
  spmmcoo       hand-derived fixture of tests/test_spmmcoo.py, dense fp64 product
  toundirected  hand-derived fixture of tests/test_undirected.py, brute force over
                Python sets; which of several equal (row, col) pairs survives is
                "parity unpinned" (the reference's std::sort leaves it open)
  appnp         K = 1 closed form, fp64 power iteration, the personalised
                PageRank limit alpha * (I - (1 - alpha) A)^-1 h on a small graph
  sgconv        dense fp64 A^K x W
  gprgnn        dense fp64 sum_k temp[k] A^k x
  clustergcn_norm  integer degrees: 1 / deg[row] exactly; on a symmetric graph every row's
                outgoing weights sum to 1 (mass is kept: sum_v (A x)[v] = sum_v x[v]), which
                scaling by the other endpoint's degree does not give; the trace grows by
                diag_lambda * sum 1 / deg
  clustergcn_conv  dense fp64 (A x) W_out + x W_root + b
  get_laplacian scipy.sparse.csgraph.laplacian on a symmetric weighted graph (all three
                normalisations; 'rw' against I - D^-1 A); rows of D - A sum to zero
  cheb_norm / cheb_conv  dense fp64: L^ = 2 L / lambda - I and T_k(L^) from the eigenvalues
                of the symmetric L^ (cos(k arccos .) inside [-1, 1], cosh outside)
  lightgcn      dense fp64 A x
  gcn2conv      dense fp64 A ((1-b)(1-a) x + b x W1) + (1-b) a x0 + b x0 W2
  evennet       dense fp64 t0 x + t3 A^3 x + t4 A^4 x (the hops the loop adds as written)
  chebnet2      T_i(A) from the eigenvalues of a symmetric A (cos(i arccos lambda)); a
                polynomial sampled at the Chebyshev nodes comes back as that polynomial of A
  bernnet       dense fp64 sum_i C(K,i)/2^K t_i A1^i A2^(K-i) x; the binomial theorem
                (A1 = L, A2 = 2I - L, t = 1 gives x back)
  gpuinitco / getweight / csctocsr  brute-force Python loops on small graphs,
                the README's CSC -> CSR known answer, the inputs of the reference's
                test_getweight.py with the expected list that test carries, those of
                test_gpuinitco.py / test_fromtonodes.py / test_edgetovertex.py /
                test_scatter_to_edge.py with hand-derived answers
  sampleprocessing  "parity unpinned": the reference draws with rand() /
                clock-seeded curand, so no output of it can be reproduced.  Pinned
                here: the copy branch exactly, and for the sampled branch the
                invariants (distinct, subset, count, order) and uniformity
  cross_entropy_loss  jittor.nn.cross_entropy_loss / log_softmax + nll_loss live in the
                jittor package (jittor==1.3.9.14, absent here); the textbook formula,
                pinned by scipy's logsumexp, log(C) on equal logits, shift invariance,
                rows of the gradient summing to zero, finite differences
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile oracle.c (gcc, single thread, AVX+FMA) into liboracle.so."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------- C loops ---

def cootocsr(edge_index, edge_weight, v_num):
    """ops/cootocsr.py:28-35 -> ops/cpp/cootocsr_op.cc:24-57.
    Returns (column_indices, row_offset, csr_edge_weight)."""
    ei = _i32(edge_index)
    w = _f32(edge_weight)
    E = ei.shape[1]
    col = np.zeros(E, np.int32)
    off = np.zeros(v_num + 1, np.int32)
    wo = np.zeros(E, np.float32)
    rc = lib().orc_cootocsr(_p(ei), _p(w), ctypes.c_int64(E), ctypes.c_int32(v_num),
                            _p(col), _p(off), _p(wo))
    assert rc == 0
    return col, off, wo


def cootocsc(edge_index, edge_weight, v_num):
    """ops/cootocsc.py:29-36 -> ops/cpp/cootocsc_op.cc:23-53.
    Returns (row_indices, column_offset, csc_edge_weight)."""
    ei = _i32(edge_index)
    w = _f32(edge_weight)
    E = ei.shape[1]
    row = np.zeros(E, np.int32)
    off = np.zeros(v_num + 1, np.int32)
    wo = np.zeros(E, np.float32)
    rc = lib().orc_cootocsc(_p(ei), _p(w), ctypes.c_int64(E), ctypes.c_int32(v_num),
                            _p(row), _p(off), _p(wo))
    assert rc == 0
    return row, off, wo


def aggregate(x, indices, offset, weight, scalar=False):
    """ops/cpp/aggregate_op.cc:26-71: out[i,:] = sum_j w[j] * x[indices[j],:]
    over j in [offset[i], offset[i+1]).  The number of output rows is x's
    (aggregate_op.cc:33), as in the reference."""
    x = _f32(x)
    indices, offset, weight = _i32(indices), _i32(offset), _f32(weight)
    v_num, F = x.shape
    assert offset.shape[0] == v_num + 1
    out = np.empty_like(x)
    fn = lib().orc_aggregate_scalar if scalar else lib().orc_aggregate
    fn(_p(out), _p(x), _p(indices), _p(offset), _p(weight), ctypes.c_int32(v_num),
       ctypes.c_int32(F))
    return out


def _sub_rows(indices, offset, weight, rows):
    """Compressed arrays of the chosen rows only, each row's entries in their order."""
    rows = np.asarray(rows, dtype=np.int64)
    lens = (offset[rows + 1] - offset[rows]).astype(np.int64)
    sub_off = np.zeros(rows.shape[0] + 1, np.int64)
    np.cumsum(lens, out=sub_off[1:])
    assert sub_off[-1] < 2 ** 31
    take = np.repeat(offset[rows].astype(np.int64) - sub_off[:-1], lens) + np.arange(sub_off[-1], dtype=np.int64)
    return _i32(indices[take]), _i32(sub_off), _f32(weight[take])


def aggregate_rows_f64(x, indices, offset, weight, rows):
    """(exact, terms) for the chosen rows: sum_j w[j] * x[indices[j],:] accumulated in
    float64 and the sum of the absolute terms.  Not the reference's arithmetic: the
    value its sequential fp32 loop approximates, used to arbitrate on rows so long
    that the loop itself has drifted."""
    x = _f32(x)
    indices, offset, weight = _i32(indices), _i32(offset), _f32(weight)
    sub_idx, sub_off, sub_w = _sub_rows(indices, offset, weight, rows)
    n = sub_off.shape[0] - 1
    out = np.empty((n, x.shape[1]), np.float64)
    terms = np.empty((n, x.shape[1]), np.float64)
    lib().orc_aggregate_f64(_p(out), _p(terms), _p(x), _p(sub_idx), _p(sub_off), _p(sub_w), ctypes.c_int32(n),
                            ctypes.c_int32(x.shape[1]))
    return out, terms


def aggregate_f64(x, indices, offset, weight):
    """aggregate_rows_f64 for every row (no copy of the compressed arrays)."""
    x = _f32(x)
    indices, offset, weight = _i32(indices), _i32(offset), _f32(weight)
    n = offset.shape[0] - 1
    out = np.empty((n, x.shape[1]), np.float64)
    terms = np.empty((n, x.shape[1]), np.float64)
    lib().orc_aggregate_f64(_p(out), _p(terms), _p(x), _p(indices), _p(offset), _p(weight), ctypes.c_int32(n),
                            ctypes.c_int32(x.shape[1]))
    return out, terms


def aggregate_rows(x, indices, offset, weight, rows):
    """Rows `rows` of aggregate(x, indices, offset, weight), by the same C loop run on the
    compressed arrays of those rows only (each chosen row keeps its entries in their order),
    so that a sample of rows of a graph with 10^8 entries costs seconds.  The loop takes
    its row count from the offsets it is given and never looks at how many rows x has."""
    x = _f32(x)
    indices, offset, weight = _i32(indices), _i32(offset), _f32(weight)
    sub_idx, sub_off, sub_w = _sub_rows(indices, offset, weight, rows)
    n = sub_off.shape[0] - 1
    out = np.empty((n, x.shape[1]), np.float32)
    lib().orc_aggregate(_p(out), _p(x), _p(sub_idx), _p(sub_off), _p(sub_w), ctypes.c_int32(n),
                        ctypes.c_int32(x.shape[1]))
    return out


def edgesoftmax(x, offset):
    """ops/cpp/edgesoftmax_op.cc:36-66.  x is [E], [E,1] (reference shapes) or
    [E,H] (independent heads)."""
    x = _f32(x)
    offset = _i32(offset)
    H = 1 if x.ndim == 1 else x.shape[1]
    out = np.zeros_like(x)
    if H == 1:
        lib().orc_edgesoftmax(_p(out), _p(x), _p(offset), ctypes.c_int32(offset.shape[0] - 1))
    else:
        lib().orc_edgesoftmax_heads(_p(out), _p(x), _p(offset),
                                    ctypes.c_int32(offset.shape[0] - 1), ctypes.c_int32(H))
    return out


def edgesoftmax_backward(grad, y, offset):
    """ops/cpp/edgesoftmaxbackward_op.cc:27-54."""
    grad, y = _f32(grad), _f32(y)
    offset = _i32(offset)
    H = 1 if y.ndim == 1 else y.shape[1]
    out = np.zeros_like(y)
    lib().orc_edgesoftmax_backward(_p(out), _p(grad), _p(y), _p(offset),
                                   ctypes.c_int32(offset.shape[0] - 1), ctypes.c_int32(H))
    return out


def scattertoedge(x, indices, offset, flag):
    """ops/cpp/scattertoedge_op.cc:67-88; flag 0 = by source (row_indices),
    flag 1 = by destination (the column the edge sits in)."""
    x = _f32(x)
    indices, offset = _i32(indices), _i32(offset)
    E, F = indices.shape[0], x.shape[1]
    out = np.empty((E, F), np.float32)
    lib().orc_scattertoedge(_p(out), _p(x), _p(indices), _p(offset),
                            ctypes.c_int32(offset.shape[0] - 1), ctypes.c_int64(E),
                            ctypes.c_int32(F), ctypes.c_int32(flag))
    return out


def edgetovertex(x, indices, offset, flag, out_rows=None):
    """ops/cpp/edgetovertex_op.cc:36-55."""
    x = _f32(x)
    indices, offset = _i32(indices), _i32(offset)
    v_num = offset.shape[0] - 1
    out_rows = v_num if out_rows is None else out_rows
    F = x.shape[1]
    out = np.empty((out_rows, F), np.float32)
    lib().orc_edgetovertex(_p(out), _p(x), _p(indices), _p(offset), ctypes.c_int32(v_num),
                           ctypes.c_int32(out_rows), ctypes.c_int32(F), ctypes.c_int32(flag))
    return out


# ------------------------------------------------- numpy: graph preprocessing

def add_remaining_self_loops(edge_index, edge_weight=None, fill_value=1.0, num_nodes=None):
    """utils/loop.py:98-136: drop existing self-loops, append (i,i) for every
    node at the END; a dropped loop's weight becomes that node's loop weight
    (the last one wins when a node had several)."""
    edge_index = np.asarray(edge_index)
    N = int(edge_index.max()) + 1 if num_nodes is None else int(num_nodes)
    row, col = edge_index[0], edge_index[1]
    mask = row != col
    loop_index = np.arange(N, dtype=edge_index.dtype)
    out_index = np.concatenate([edge_index[:, mask], np.stack([loop_index, loop_index])], axis=1)
    out_w = None
    if edge_weight is not None:
        edge_weight = np.asarray(edge_weight, dtype=np.float32)
        loop_w = np.full(N, fill_value, np.float32)
        inv = ~mask
        if inv.any():
            loop_w[row[inv]] = edge_weight[inv]
        out_w = np.concatenate([edge_weight[mask], loop_w])
    return out_index, out_w


def _degree_by_col(col, w, N):
    deg = np.zeros(N, np.float32)
    np.add.at(deg, col, w)            # jt.scatter(..., reduce='add')
    return deg


def gcn_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True):
    """nn/conv/gcn_conv.py:18-37: w = d^-1/2[row] * w * d^-1/2[col] with the
    degree summed by column, inf -> 0."""
    edge_index = np.asarray(edge_index)
    N = int(edge_index.max()) + 1 if num_nodes is None else int(num_nodes)
    fill = 2.0 if improved else 1.0
    if edge_weight is None:
        edge_weight = np.ones(edge_index.shape[1], np.float32)
    if add_self_loops:
        edge_index, edge_weight = add_remaining_self_loops(edge_index, edge_weight, fill, N)
    row, col = edge_index[0], edge_index[1]
    deg = _degree_by_col(col, edge_weight, N)
    with np.errstate(divide="ignore"):
        dis = np.power(deg, np.float32(-0.5)).astype(np.float32)
    dis[np.isinf(dis)] = 0
    return edge_index, (dis[row] * edge_weight * dis[col]).astype(np.float32)


def sage_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True):
    """nn/conv/sage_conv.py:16-40: w = w * d^-1[col]."""
    edge_index = np.asarray(edge_index)
    N = int(edge_index.max()) + 1 if num_nodes is None else int(num_nodes)
    fill = 2.0 if improved else 1.0
    if edge_weight is None:
        edge_weight = np.ones(edge_index.shape[1], np.float32)
    if add_self_loops:
        edge_index, edge_weight = add_remaining_self_loops(edge_index, edge_weight, fill, N)
    col = edge_index[1]
    deg = _degree_by_col(col, edge_weight, N)
    with np.errstate(divide="ignore"):
        di = np.power(deg, np.float32(-1.0)).astype(np.float32)
    di[np.isinf(di)] = 0
    return edge_index, (edge_weight * di[col]).astype(np.float32)


def clustergcn_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True,
                    diag_lambda=0.0):
    """nn/conv/clustergcn_conv.py:14-39: deg summed by col, w = w * deg^-1[row], and every
    self-loop gets diag_lambda * deg^-1[row] on top."""
    edge_index = np.asarray(edge_index)
    N = int(edge_index.max()) + 1 if num_nodes is None else int(num_nodes)
    fill = 2.0 if improved else 1.0
    if edge_weight is None:
        edge_weight = np.ones(edge_index.shape[1], np.float32)
    if add_self_loops:
        edge_index, edge_weight = add_remaining_self_loops(edge_index, edge_weight, fill, N)
    row, col = edge_index[0], edge_index[1]
    deg = _degree_by_col(col, edge_weight, N)
    with np.errstate(divide="ignore"):
        di = np.power(deg, np.float32(-1.0)).astype(np.float32)
    di[np.isinf(di)] = 0
    w = (edge_weight * di[row]).astype(np.float32)
    loop = row == col
    w[loop] = (w[loop] + np.float32(diag_lambda) * di[row[loop]]).astype(np.float32)
    return edge_index, w


def get_laplacian(edge_index, edge_weight=None, normalization=None, num_nodes=None):
    """utils/get_laplacian.py:9-81: self-loops removed, degree summed by row (the source),
    None: L = D - A; 'sym': I - D^-1/2 A D^-1/2; 'rw': I - D^-1 A; the N diagonal entries are
    appended after the other edges."""
    ei = np.asarray(edge_index)
    keep = ei[0] != ei[1]
    w = np.ones(ei.shape[1], np.float32) if edge_weight is None else _f32(edge_weight)
    ei, w = ei[:, keep], w[keep]
    N = int(ei.max()) + 1 if num_nodes is None else int(num_nodes)
    row, col = ei[0], ei[1]
    deg = np.zeros(N, np.float32)
    np.add.at(deg, row, w)
    loops = np.stack([np.arange(N)] * 2).astype(ei.dtype)
    if normalization is None:
        return np.concatenate([ei, loops], axis=1), np.concatenate([-w, deg]).astype(np.float32)
    with np.errstate(divide="ignore"):
        if normalization == "sym":
            d = np.power(deg, np.float32(-0.5)).astype(np.float32)
            d[np.isinf(d)] = 0
            a = (d[row] * w * d[col]).astype(np.float32)
        else:
            d = (np.float32(1.0) / deg).astype(np.float32)
            d[np.isinf(d)] = 0
            a = (d[row] * w).astype(np.float32)
    return np.concatenate([ei, loops], axis=1), np.concatenate([-a, np.ones(N, np.float32)]).astype(np.float32)


def cheb_norm(edge_index, num_nodes, edge_weight=None, normalization="sym", lambda_max=None, batch=None):
    """nn/conv/cheb_conv.py:97-122: the Laplacian scaled to 2 L / lambda_max - I (lambda_max
    defaults to twice the largest entry; infinite weights become 0; 1 is taken off the loops)."""
    ei, w = get_laplacian(edge_index, edge_weight, normalization, num_nodes)
    lam = np.float32(2.0) * w.max() if lambda_max is None else np.asarray(lambda_max, np.float32).reshape(-1)
    if batch is not None and np.size(lam) > 1:
        lam = lam[np.asarray(batch)[ei[0]]]
    with np.errstate(divide="ignore", invalid="ignore"):
        w = ((np.float32(2.0) * w) / lam).astype(np.float32)
    w[np.isinf(w)] = 0
    loop = ei[0] == ei[1]
    w[loop] = w[loop] - np.float32(1)
    return ei, w


def cheb_conv(x, edge_index, weights, bias=None, edge_weight=None, normalization="sym", lambda_max=None, batch=None):
    """nn/conv/cheb_conv.py:124-155: out = Tx_0 W_0 + Tx_1 W_1 + ..., Tx_1 = L^ x,
    Tx_k = 2 L^ Tx_{k-1} - Tx_{k-2}, messages norm_e * x[src] summed at dst; weights[k] is [in, out]."""
    x = _f32(x)
    V = x.shape[0]
    ei, norm = cheb_norm(edge_index, V, edge_weight, normalization, lambda_max, batch)
    csc = cootocsc(ei.astype(np.int32), norm, V)
    mm = lambda a, w: (a.astype(np.float64) @ np.asarray(w, np.float64)).astype(np.float32)
    t0 = t1 = x
    out = mm(t0, weights[0])
    if len(weights) > 1:
        t1 = aggregate_with_weight(x, csc)
        out = (out + mm(t1, weights[1])).astype(np.float32)
    for wk in weights[2:]:
        t2 = (np.float32(2) * aggregate_with_weight(t1, csc) - t0).astype(np.float32)
        out = (out + mm(t2, wk)).astype(np.float32)
        t0, t1 = t1, t2
    return out if bias is None else (out + _f32(bias)).astype(np.float32)


# ------------------------------------------------------ numpy: op wrappers ---

def aggregate_with_weight(x, csc, csr=None):
    """ops/aggregateWithWeight.py:20-30: forward feeds the CSC arrays.
    csc = (row_indices, column_offset, edge_weight)."""
    return aggregate(x, csc[0], csc[1], csc[2])


def aggregate_with_weight_grad(grad_out, csr):
    """ops/aggregateWithWeight.py:32-41: backward feeds the CSR arrays.
    csr = (column_indices, row_offset, edge_weight)."""
    return aggregate(grad_out, csr[0], csr[1], csr[2])


def gat_forward(h, csc, a, slope=0.2):
    """nn/conv/gat_conv.py:61-83 after vertex_forward: h is [V,C] (already
    relu(x@W)), a is the [2C,1] attention vector.  Returns (out, alpha, m).
    Single head, float32 throughout like the reference."""
    row, off = _i32(csc[0]), _i32(csc[1])
    h = _f32(h)
    C = h.shape[1]
    e_src = scattertoedge(h, row, off, 0)
    e_dst = scattertoedge(h, row, off, 1)
    e = np.concatenate([e_src, e_dst], axis=1)
    out = (e @ _f32(a).reshape(2 * C, 1)).astype(np.float32)
    m = np.where(out > 0, out, np.float32(slope) * out).astype(np.float32)
    alpha = edgesoftmax(m, off)
    msg = e[:, :C] * alpha
    res = edgetovertex(msg, row, off, 1)
    return res, alpha, m


def gat_forward_heads(h, csc, a_src, a_dst, slope=0.2):
    """Multi-head generalisation: h [V,H,D], a_src/a_dst [H,D]; head k is
    gat_forward on h[:,k,:] with a = concat(a_src[k], a_dst[k]).
    Returns (out [V,H,D], alpha [E,H])."""
    V, H, D = h.shape
    outs, alphas = [], []
    for k in range(H):
        a = np.concatenate([a_src[k], a_dst[k]]).astype(np.float32)
        o, al, _ = gat_forward(np.ascontiguousarray(h[:, k, :]), csc, a, slope)
        outs.append(o)
        alphas.append(al[:, 0])
    return np.stack(outs, axis=1), np.stack(alphas, axis=1)


def gat_backward(h, csc, a, g_out, slope=0.2):
    """Gradients of gat_forward with respect to h and a for the upstream gradient g_out [V,C]:
    the chain Jittor's autograd runs through the reference operators' own grad functions
    (nn/conv/gat_conv.py:61-83 backwards): ScatterToVertex.grad = scattertoedge with flag 1
    (ops/scatterToVertex.py:43-47), the product with alpha, EdgeSoftmax.grad
    (ops/edgesoftmax.py:71-74 -> edgesoftmaxbackward_op.cc:27-54), leaky_relu', the [E,2C]x[2C,1]
    product, ScatterToEdge.grad = edgetovertex with the flag of the forward call
    (ops/scatterToEdge.py:42-46).  Returns (g_h [V,C], g_a [2C])."""
    row, off = _i32(csc[0]), _i32(csc[1])
    h, g_out = _f32(h), _f32(g_out)
    V, C = h.shape
    slope = np.float32(slope)
    a = _f32(a).reshape(2 * C, 1)
    e_src = scattertoedge(h, row, off, 0)
    e_dst = scattertoedge(h, row, off, 1)
    e = np.concatenate([e_src, e_dst], axis=1)
    z = (e @ a).astype(np.float32)
    m = np.where(z > 0, z, slope * z).astype(np.float32)
    alpha = edgesoftmax(m, off)
    g_msg = scattertoedge(g_out, row, off, 1)                       # grad of ScatterToVertex
    g_alpha = (g_msg * e_src).sum(axis=1, keepdims=True).astype(np.float32)
    g_m = edgesoftmax_backward(g_alpha, alpha, off)
    g_z = (g_m * np.where(z > 0, np.float32(1), slope)).astype(np.float32)
    g_a = (e.T @ g_z).astype(np.float32)[:, 0]
    g_e = (g_z @ a.T).astype(np.float32)
    g_e_src = (g_msg * alpha + g_e[:, :C]).astype(np.float32)
    g_h = edgetovertex(g_e_src, row, off, 0, out_rows=V) + edgetovertex(np.ascontiguousarray(g_e[:, C:]), row, off, 1)
    return g_h.astype(np.float32), g_a


def gat_backward_heads(h, csc, a_src, a_dst, g_out, slope=0.2):
    """Head k is gat_backward on h[:,k,:]; returns (g_h [V,H,D], g_a_src [H,D], g_a_dst [H,D])."""
    V, H, D = h.shape
    gh, gs, gd = [], [], []
    for k in range(H):
        a = np.concatenate([a_src[k], a_dst[k]]).astype(np.float32)
        g, ga = gat_backward(np.ascontiguousarray(h[:, k, :]), csc, a, np.ascontiguousarray(g_out[:, k, :]), slope)
        gh.append(g)
        gs.append(ga[:D])
        gd.append(ga[D:])
    return np.stack(gh, axis=1), np.stack(gs), np.stack(gd)


def spmmcoo(x, edge_index, edge_weight, trans_A=True):
    """ops/spmmcoo.py:21-33: cuSPARSE COO product op(A) x with A = (row, col, w);
    trans_A=True -> out[col] += w * x[row].  The library's summation order is not
    specified; this restatement adds in edge order, in fp32."""
    x = _f32(x)
    row, col = np.asarray(edge_index[0]), np.asarray(edge_index[1])
    w = _f32(edge_weight)
    out = np.zeros_like(x)
    dst, src = (col, row) if trans_A else (row, col)
    for e in range(row.shape[0]):
        out[dst[e]] = (out[dst[e]] + w[e] * x[src[e]]).astype(np.float32)
    return out


def toundirected(edge_index, edge_attr):
    """ops/cpp/toundirected_op.cc:35-60: append (r, c, a) and (c, r, a) per edge, sort by
    (row, col), keep the first of each run of equal pairs.  The sort here is stable."""
    ei = np.asarray(edge_index)
    attr = np.asarray(edge_attr).reshape(-1)
    E = ei.shape[1]
    rows = np.stack([ei[0], ei[1]], axis=1).reshape(-1)
    cols = np.stack([ei[1], ei[0]], axis=1).reshape(-1)
    data = np.repeat(attr, 2)
    order = np.lexsort((cols, rows))            # stable; last key is the primary one
    rows, cols, data = rows[order], cols[order], data[order]
    keep = np.ones(2 * E, bool)
    keep[1:] = (rows[1:] != rows[:-1]) | (cols[1:] != cols[:-1])
    return np.stack([rows[keep], cols[keep]]).astype(np.int32), data[keep].reshape(1, -1)


def appnp(x, csc, K, alpha):
    """nn/conv/appnp_conv.py:42-51: K times x = propagate(x); x = x * (1 - alpha);
    x = x + alpha * h, all in fp32."""
    h = _f32(x)
    x = h
    for _ in range(K):
        x = aggregate_with_weight(x, csc)
        x = (x * np.float32(1 - alpha)).astype(np.float32)
        x = (x + np.float32(alpha) * h).astype(np.float32)
    return x


def sgconv(x, csc, K, weight, bias=None):
    """nn/conv/sg_conv.py:62-69: K products, then the linear layer (weight is [in, out])."""
    x = _f32(x)
    for _ in range(K):
        x = aggregate_with_weight(x, csc)
    out = (x.astype(np.float64) @ np.asarray(weight, np.float64)).astype(np.float32)
    return out if bias is None else (out + _f32(bias)).astype(np.float32)


def gprgnn(x, csc, temp):
    """nn/conv/gpr_conv.py:80-88: out = x * temp[0]; K times x = propagate(x); out = out + temp[k+1] * x."""
    x = _f32(x)
    temp = _f32(temp)
    out = (x * temp[0]).astype(np.float32)
    for k in range(temp.shape[0] - 1):
        x = aggregate_with_weight(x, csc)
        out = (out + temp[k + 1] * x).astype(np.float32)
    return out


def lightgcn(x, csc):
    """nn/conv/lightgcn_conv.py:28-44: one product, no weights."""
    return aggregate_with_weight(_f32(x), csc)


def gcn2conv(x, x_0, csc, weight1, weight2, alpha, beta):
    """nn/conv/gcn2_conv.py:66-73: support = (1-beta)(1-alpha) x + beta x W1,
    initial = (1-beta) alpha x_0 + beta x_0 W2, out = propagate(support) + initial."""
    x, x_0 = _f32(x), _f32(x_0)
    mm = lambda a, w: (a.astype(np.float64) @ np.asarray(w, np.float64)).astype(np.float32)
    support = (np.float32((1 - beta) * (1 - alpha)) * x + np.float32(beta) * mm(x, weight1)).astype(np.float32)
    initial = (np.float32((1 - beta) * alpha) * x_0 + np.float32(beta) * mm(x_0, weight2)).astype(np.float32)
    return (aggregate_with_weight(support, csc) + initial).astype(np.float32)


def evennet_temp(K, alpha):
    """nn/conv/even_conv.py:48-50: alpha (1-alpha)^k, the last one (1-alpha)^K."""
    t = alpha * (1 - alpha) ** np.arange(K + 1)
    t[-1] = (1 - alpha) ** K
    return t


def evennet(x, csc, K, alpha):
    """nn/conv/even_conv.py:53-61: out = x * temp[0]; K hops; hop k (from 0) is added with
    temp[k+1] when k // 2 == 1, i.e. the third and the fourth hop, as the loop is written."""
    temp = evennet_temp(K, alpha)
    x = _f32(x)
    out = (x * np.float32(temp[0])).astype(np.float32)
    for k in range(K):
        x = aggregate_with_weight(x, csc)
        if k // 2 == 1:
            out = (out + np.float32(temp[k + 1]) * x).astype(np.float32)
    return out


def chebnet2_coefficients(temp):
    """nn/conv/chebnet2_conv.py:22-33,68-75: coe[i] = 2/(K+1) sum_j relu(temp)[j] T_i(x_j) with
    x_j = cos((K - j + 0.5) pi / (K + 1)), T_i by the three-term recurrence."""
    t = np.maximum(np.asarray(temp, np.float64), 0.0)
    K = t.shape[0] - 1

    def cheb(i, v):
        if i == 0:
            return 1.0
        t0, t1 = 1.0, v
        for _ in range(2, i + 1):
            t0, t1 = t1, 2 * v * t1 - t0
        return t1
    coe = np.zeros(K + 1)
    for i in range(K + 1):
        acc = 0.0
        for j in range(K + 1):
            acc += t[j] * cheb(i, np.cos((K - j + 0.5) * np.pi / (K + 1)))
        coe[i] = 2 * acc / (K + 1)
    return coe


def chebnet2(x, csc, temp):
    """nn/conv/chebnet2_conv.py:77-93: out = coe[0]/2 Tx_0 + coe[1] Tx_1, then
    Tx_2 = 2 propagate(Tx_1) - Tx_0 and out += coe[i] Tx_2 for i = 2..K."""
    coe = chebnet2_coefficients(temp).astype(np.float32)
    K = coe.shape[0] - 1
    t0 = _f32(x)
    t1 = aggregate_with_weight(t0, csc)
    out = (coe[0] / np.float32(2) * t0 + coe[1] * t1).astype(np.float32)
    for i in range(2, K + 1):
        t2 = (np.float32(2) * aggregate_with_weight(t1, csc) - t0).astype(np.float32)
        out = (out + coe[i] * t2).astype(np.float32)
        t0, t1 = t1, t2
    return out


def bernnet(x, csc1, csc2, temp):
    """nn/conv/bernnet_conv.py:56-80: tmp[k] = A2^k x; out = C(K,0)/2^K t[0] tmp[K], then for
    i = 0..K-1: out += C(K,i+1)/2^K t[i+1] A1^(i+1) tmp[K-i-1], with t = relu(temp)."""
    from math import comb
    t = np.maximum(_f32(temp), 0)
    K = t.shape[0] - 1
    tmp = [_f32(x)]
    for _ in range(K):
        tmp.append(aggregate_with_weight(tmp[-1], csc2))
    out = (np.float32(comb(K, 0) / 2 ** K) * t[0] * tmp[K]).astype(np.float32)
    for i in range(K):
        v = tmp[K - i - 1]
        for _ in range(i + 1):
            v = aggregate_with_weight(v, csc1)
        out = (out + np.float32(comb(K, i + 1) / 2 ** K) * t[i + 1] * v).astype(np.float32)
    return out


def clustergcn_conv(x, csc, weight_out, weight_root, bias=None):
    """nn/conv/clustergcn_conv.py:136-143: propagate(x) @ weight_out + x @ weight_root (+ bias)."""
    x = _f32(x)
    mm = lambda a, w: (a.astype(np.float64) @ np.asarray(w, np.float64)).astype(np.float32)
    out = (mm(aggregate_with_weight(x, csc), weight_out) + mm(x, weight_root)).astype(np.float32)
    return out if bias is None else (out + _f32(bias)).astype(np.float32)


def gpuinitco(dst_size, fanout_i, csc_layer_dst, csc_global_column_offset):
    """ops/cpp/gpuinitco_op.cc:37-50 (the GPU branch; the CPU branch :27-32 leaves zeros):
    out[i+1] = min(degree of dst[i], fanout); not a running sum."""
    dst = np.asarray(csc_layer_dst)
    g = np.asarray(csc_global_column_offset)
    out = np.zeros(dst_size + 1, np.int32)
    out[1:] = np.minimum(g[dst + 1] - g[dst], fanout_i)
    return out


def getweight(vtx_size, csc_layer_dst, csc_layer_src, csc_layer_column_offset, csc_layer_row_indices):
    """ops/cpp/getweight_op.cc:36-82: in-degree of dst[i] += size of column i, out-degree
    of every row index += 1, weight = 1 / (sqrtf(out[src]) * sqrtf(in[dst]))."""
    dst = np.asarray(csc_layer_dst)
    off = np.asarray(csc_layer_column_offset)
    row = np.asarray(csc_layer_row_indices)
    ins = np.zeros(vtx_size, np.int32)
    outs = np.zeros(vtx_size, np.int32)
    w = np.zeros(off[-1], np.float32)
    for i in range(dst.shape[0]):
        ins[dst[i]] += off[i + 1] - off[i]
        for j in range(off[i], off[i + 1]):
            outs[row[j]] += 1
    for i in range(dst.shape[0]):
        for j in range(off[i], off[i + 1]):
            w[j] = np.float32(1) / (np.sqrt(np.float32(outs[row[j]])) * np.sqrt(np.float32(ins[dst[i]])))
    return w


def csctocsr(column_offset, row_indices, dst, src):
    """ops/cpp/csctocsr_op.cc:36-78: rows are the positions of `src`; an entry whose row
    index is not in `src` is dropped; column indices hold dst ids; stable in column order."""
    off, row = np.asarray(column_offset), np.asarray(row_indices)
    dst, src = np.asarray(dst), np.asarray(src)
    where = {int(s): i for i, s in enumerate(src)}
    r_o = np.zeros(src.shape[0] + 1, np.int32)
    for j in range(off[-1]):
        if int(row[j]) in where:
            r_o[where[int(row[j])] + 1] += 1
    r_o = np.cumsum(r_o).astype(np.int32)
    c_i = np.zeros(off[-1], np.int32)
    ptr = r_o[:-1].copy()
    for i in range(dst.shape[0]):
        for j in range(off[i], off[i + 1]):
            k = where.get(int(row[j]))
            if k is not None:
                c_i[ptr[k]] = dst[i]
                ptr[k] += 1
    return r_o, c_i


def sampleprocessing(fanout_i, csc_layer_dst, csc_layer_column_offset, csc_global_column_offset,
                     csc_global_row_indices, seed=0):
    """ops/cpp/sampleprocessing_op.cc:47-84 with a seeded draw (see oracle.c)."""
    dst = _i32(csc_layer_dst)
    loff = _i32(csc_layer_column_offset)
    goff = _i32(csc_global_column_offset)
    gidx = _i32(csc_global_row_indices)
    out = np.zeros(int(loff[-1]), np.int32)
    lib().orc_sample_neighbors(_p(dst), _p(loff), _p(goff), _p(gidx), ctypes.c_int32(dst.shape[0]),
                               ctypes.c_int32(int(fanout_i)), ctypes.c_uint64(int(seed) & (2**64 - 1)), _p(out))
    return out


def from_nodes(offset, indices, nodes):
    """ops/saparse_ops.py:9-39 (and :42-71 with the CSR arrays): the neighbour lists of `nodes`,
    concatenated in the order given."""
    off, idx = np.asarray(offset), np.asarray(indices)
    parts = [idx[off[n]:off[n + 1]] for n in np.asarray(nodes).reshape(-1)]
    return np.concatenate(parts).astype(np.int32) if parts else np.zeros(0, np.int32)


def cross_entropy_loss(output, target):
    """nn.cross_entropy_loss(pred, label) as examples/gcn_example.py:113 calls it (and
    nn.nll_loss(nn.log_softmax(x, dim=1), label), examples/sage_example.py:69,83): the mean over
    rows of logsumexp(row) - row[label], in float64.  Rows whose label lies outside
    [0, classes) are left out.  Returns (loss, d loss / d output)."""
    x = np.asarray(output, dtype=np.float64)
    y = np.asarray(target).astype(np.int64).reshape(-1)
    V, C = x.shape
    m = x.max(axis=1, keepdims=True) if C else np.zeros((V, 1))
    e = np.exp(x - m)
    lse = m[:, 0] + np.log(e.sum(axis=1))
    ok = (y >= 0) & (y < C)
    n = int(ok.sum())
    rows = np.nonzero(ok)[0]
    loss = (lse[rows] - x[rows, y[rows]]).sum() / n if n else float("nan")
    grad = np.zeros_like(x)
    if n:
        p = e[rows] / e[rows].sum(axis=1, keepdims=True)
        p[np.arange(rows.size), y[rows]] -= 1.0
        grad[rows] = p / n
    return loss, grad
