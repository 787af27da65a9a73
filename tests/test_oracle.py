"""Pins the CPU oracle: reference fixtures, closed forms, library routines,
invariants.  A mistake in oracle.c (dropped term, wrong index, transposed
operand) must fail at least one of these.  No GPU needed."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp
from scipy.special import softmax as sp_softmax

import oracle

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def closed_form_csx(edge_index, w, V, key_row):
    """Stable counting sort written with library calls only."""
    key = edge_index[key_row]
    other = edge_index[1 - key_row]
    perm = np.argsort(key, kind="stable")
    off = np.concatenate([[0], np.cumsum(np.bincount(key, minlength=V))]).astype(np.int32)
    return other[perm].astype(np.int32), off, w[perm].astype(np.float32), perm


def rand_graph(rng, V, E, loops=True):
    ei = rng.integers(0, V, size=(2, E)).astype(np.int32)
    if not loops:
        ei = ei[:, ei[0] != ei[1]]
    w = rng.standard_normal(ei.shape[1]).astype(np.float32)
    return ei, w


# ------------------------------------------------------------- conversion ---

@pytest.mark.parametrize("name", ["csr_v4", "mp_spmm_v10"])
def test_conversion_reference_fixtures(name):
    g = GOLD[name]
    ei = np.array(g["edge_index"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    col, off, wo = oracle.cootocsr(ei, w, g["v_num"])
    assert col.tolist() == g["csr"]["column_indices"]
    assert off.tolist() == g["csr"]["row_offset"]
    assert wo.tolist() == g["csr"]["edge_weight"]
    row, coff, cw = oracle.cootocsc(ei, w, g["v_num"])
    assert row.tolist() == g["csc"]["row_indices"]
    assert coff.tolist() == g["csc"]["column_offset"]
    assert cw.tolist() == g["csc"]["edge_weight"]


def test_conversion_readme_csc_to_csr_known_answer():
    g = GOLD["csctocsr_readme_v4"]
    off = np.array(g["column_offset"])
    dst = np.repeat(np.arange(len(off) - 1), np.diff(off)).astype(np.int32)
    ei = np.stack([np.array(g["row_indices"], np.int32), dst])
    col, roff, _ = oracle.cootocsr(ei, np.ones(ei.shape[1], np.float32), 4)
    assert roff.tolist() == g["row_offset"]
    assert col.tolist() == g["column_indices"]


@pytest.mark.parametrize("V,E,seed", [(1, 0, 0), (1, 5, 1), (7, 0, 2), (50, 400, 3), (1000, 30000, 4),
                                      (5000, 5000, 5)])
def test_conversion_closed_form_and_invariants(V, E, seed):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E)
    for key_row, fn in ((0, oracle.cootocsr), (1, oracle.cootocsc)):
        idx, off, wo = fn(ei, w, V)
        cidx, coff, cw, perm = closed_form_csx(ei, w, V, key_row)
        assert np.array_equal(idx, cidx) and np.array_equal(off, coff)
        assert np.array_equal(wo.view(np.int32), cw.view(np.int32))
        assert off[0] == 0 and off[-1] == ei.shape[1] and np.all(np.diff(off) >= 0)
        # within a row the original edge ids increase strictly (stability)
        keys_sorted = ei[key_row][perm]
        same = keys_sorted[1:] == keys_sorted[:-1]
        assert np.all(perm[1:][same] > perm[:-1][same])


def test_conversion_bruteforce_tiny():
    rng = np.random.default_rng(11)
    for _ in range(20):
        V = int(rng.integers(1, 6))
        E = int(rng.integers(0, 12))
        ei, w = rand_graph(rng, V, E)
        col, off, wo = oracle.cootocsr(ei, w, V)
        slots = []
        for r in range(V):
            for e in range(E):
                if ei[0, e] == r:
                    slots.append(e)
        assert col.tolist() == [int(ei[1, e]) for e in slots]
        assert wo.tolist() == [float(w[e]) for e in slots]


# ------------------------------------------------------------------- SpMM ---

def test_aggregate_reference_fixture_integer_exact():
    g = GOLD["mp_spmm_v10"]
    x = np.array(g["x"], np.float32)
    ei = np.array(g["edge_index"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    csc = oracle.cootocsc(ei, w, 10)
    out = oracle.aggregate_with_weight(x, csc)
    for r, vals in g["aggregate_rows"].items():
        assert out[int(r)].tolist() == [float(v) for v in vals]
    dense = np.zeros((10, 10))
    dense[ei[1], ei[0]] += w                      # out[dst] += w * x[src]
    assert np.array_equal(out, (dense @ x.astype(np.float64)).astype(np.float32))


def test_aggregate_spmmcsr_fixture():
    g = GOLD["spmmcsr_v3"]
    x = np.array(g["x"], np.float32)
    col = np.array(g["column_indices"], np.int32)
    off = np.array(g["row_offset"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    assert oracle.aggregate(x, col, off, w).tolist() == g["out_no_trans"]
    src = np.repeat(np.arange(3), np.diff(off)).astype(np.int32)
    csc = oracle.cootocsc(np.stack([src, col]), w, 3)
    assert oracle.aggregate(x, *csc).tolist() == g["out_trans_A"]


@pytest.mark.parametrize("V,E,F,seed", [(64, 600, 7, 0), (64, 600, 8, 1), (300, 5000, 33, 2),
                                        (200, 3000, 128, 3), (50, 0, 16, 4)])
def test_aggregate_vs_scipy_fp64_and_transpose_identity(V, E, F, seed):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    csc = oracle.cootocsc(ei, w, V)
    csr = oracle.cootocsr(ei, w, V)
    A = sp.coo_matrix((w.astype(np.float64), (ei[1], ei[0])), shape=(V, V)).tocsr()
    fwd = oracle.aggregate_with_weight(x, csc)
    bwd = oracle.aggregate_with_weight_grad(g, csr)
    np.testing.assert_allclose(fwd, A @ x.astype(np.float64), rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(bwd, A.T @ g.astype(np.float64), rtol=1e-5, atol=2e-5)
    # <A x, g> == <x, A^T g>
    lhs = np.sum(fwd.astype(np.float64) * g)
    rhs = np.sum(x.astype(np.float64) * bwd)
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))
    # AVX branch and scalar branch sum in the same order per feature
    sc = oracle.aggregate(x, *csc, scalar=True)
    np.testing.assert_allclose(fwd, sc, rtol=1e-6, atol=1e-6)


# ----------------------------------------------------------- edge softmax ---

def test_aggregate_rows_equals_the_full_loop_on_those_rows():
    """aggregate_rows is the same C loop on a sub-structure: bit-identical to the
    rows of the full result (empty rows, a hub and repeated rows included)."""
    rng = np.random.default_rng(77)
    V, E, F = 300, 5000, 13
    ei = np.stack([rng.integers(0, V, E), rng.integers(0, V, E)]).astype(np.int32)
    ei[1, :900] = 5
    w = rng.standard_normal(E).astype(np.float32)
    x = rng.standard_normal((V, F)).astype(np.float32)
    row, off, cw = oracle.cootocsc(ei, w, V)
    full = oracle.aggregate(x, row, off, cw)
    rows = np.array([5, 0, 299, 17, 17, 123] + list(np.flatnonzero(np.diff(off) == 0)[:3]))
    assert np.array_equal(oracle.aggregate_rows(x, row, off, cw, rows), full[rows])
    # the float64 arbiter against scipy's sparse product in float64, and its bound on the fp32 loop
    import scipy.sparse as sp
    A = sp.csr_matrix((cw.astype(np.float64), row, off), shape=(V, V))
    exact, terms = oracle.aggregate_rows_f64(x, row, off, cw, rows)
    np.testing.assert_allclose(exact, (A @ x.astype(np.float64))[rows], rtol=1e-12, atol=1e-13)
    A_abs = sp.csr_matrix((np.abs(cw).astype(np.float64), row, off), shape=(V, V))      # duplicates add as |w|
    np.testing.assert_allclose(terms, (A_abs @ np.abs(x).astype(np.float64))[rows], rtol=1e-12)
    deg = np.diff(off)[rows][:, None]
    assert np.all(np.abs(full[rows] - exact) <= (deg + 1) * 2.0 ** -24 * terms + 1e-30)


def test_edgesoftmax_reference_fixture():
    g = GOLD["edgesoftmax_v3"]
    y = oracle.edgesoftmax(np.array(g["x"], np.float32), np.array(g["column_offset"], np.int32))
    np.testing.assert_allclose(y, np.array(g["y"]), rtol=1e-6, atol=0)


@pytest.mark.parametrize("H", [1, 2, 8])
def test_edgesoftmax_vs_scipy_and_invariants(H):
    rng = np.random.default_rng(5 + H)
    V, E = 200, 3000
    ei, w = rand_graph(rng, V, E)
    _, off, _ = oracle.cootocsc(ei, w, V)
    x = (3 * rng.standard_normal((E, H))).astype(np.float32)
    y = oracle.edgesoftmax(x if H > 1 else x[:, 0], off)
    y = y.reshape(E, H)
    for v in range(V):
        s, e = off[v], off[v + 1]
        if e > s:
            np.testing.assert_allclose(y[s:e], sp_softmax(x[s:e].astype(np.float64), axis=0),
                                       rtol=2e-6, atol=1e-7)
            np.testing.assert_allclose(y[s:e].sum(0), 1.0, rtol=1e-5)
    y2 = oracle.edgesoftmax((x + np.float32(2.0)) if H > 1 else (x + np.float32(2.0))[:, 0], off)
    np.testing.assert_allclose(y2.reshape(E, H), y, rtol=1e-5, atol=1e-7)   # shift invariance
    # [E,1] input is the reference's GAT shape and equals the [E] answer
    if H == 1:
        assert np.array_equal(oracle.edgesoftmax(x, off)[:, 0], y[:, 0])


@pytest.mark.parametrize("H", [1, 4])
def test_edgesoftmax_backward_closed_form_and_finite_difference(H):
    rng = np.random.default_rng(21 + H)
    V, E = 40, 300
    ei, w = rand_graph(rng, V, E)
    _, off, _ = oracle.cootocsc(ei, w, V)
    x = rng.standard_normal((E, H)).astype(np.float32)
    g = rng.standard_normal((E, H)).astype(np.float32)
    y = oracle.edgesoftmax(x, off).reshape(E, H)
    dx = oracle.edgesoftmax_backward(g, y, off).reshape(E, H)
    seg = np.repeat(np.arange(V), np.diff(off))
    dot = np.zeros((V, H))
    np.add.at(dot, seg, y.astype(np.float64) * g)
    np.testing.assert_allclose(dx, y * (g - dot[seg]), rtol=1e-5, atol=1e-6)
    segsum = np.zeros((V, H))
    np.add.at(segsum, seg, dx)
    np.testing.assert_allclose(segsum, 0, atol=1e-5)
    # finite differences of the fp64 closed-form forward along a random direction
    def f64(xx):
        out = np.zeros_like(xx)
        for v in range(V):
            s, e = off[v], off[v + 1]
            if e > s:
                out[s:e] = sp_softmax(xx[s:e], axis=0)
        return out
    d = rng.standard_normal((E, H))
    eps = 1e-6
    fd = (np.sum(f64(x + eps * d) * g) - np.sum(f64(x - eps * d) * g)) / (2 * eps)
    assert abs(fd - np.sum(dx * d)) < 1e-4 * max(1.0, abs(fd))


# ------------------------------------------------------------ scatter ops ---

def test_scatter_ops_vs_numpy():
    rng = np.random.default_rng(3)
    V, E, F = 60, 500, 5
    ei, w = rand_graph(rng, V, E)
    row, off, _ = oracle.cootocsc(ei, w, V)
    dst = np.repeat(np.arange(V), np.diff(off))
    x = rng.standard_normal((V, F)).astype(np.float32)
    xe = rng.standard_normal((E, F)).astype(np.float32)
    assert np.array_equal(oracle.scattertoedge(x, row, off, 0), x[row])
    assert np.array_equal(oracle.scattertoedge(x, row, off, 1), x[dst])
    for flag, tgt in ((0, row), (1, dst)):
        ref = np.zeros((V, F))
        np.add.at(ref, tgt, xe.astype(np.float64))
        np.testing.assert_allclose(oracle.edgetovertex(xe, row, off, flag), ref, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------- normalisation ---

def test_add_remaining_self_loops_order_and_weights():
    ei = np.array([[0, 1, 1, 2, 2], [1, 1, 2, 2, 0]], np.int32)
    w = np.array([1, 7, 2, 9, 3], np.float32)
    oi, ow = oracle.add_remaining_self_loops(ei, w, 1.0, 4)
    assert oi.tolist() == [[0, 1, 2, 0, 1, 2, 3], [1, 2, 0, 0, 1, 2, 3]]
    assert ow.tolist() == [1, 2, 3, 1, 7, 9, 1]


def test_gcn_and_sage_norm_closed_forms():
    rng = np.random.default_rng(8)
    V = 30
    ei, _ = rand_graph(rng, V, 200, loops=False)
    oi, ow = oracle.gcn_norm(ei, None, V)
    assert oi.shape[1] == ei.shape[1] + V and np.array_equal(oi[:, -V:], np.stack([np.arange(V)] * 2))
    deg = np.bincount(oi[1], minlength=V).astype(np.float64)       # integer degrees, exact
    np.testing.assert_allclose(ow, 1 / np.sqrt(deg[oi[0]] * deg[oi[1]]), rtol=1e-6)
    si, sw = oracle.sage_norm(ei, None, V)
    np.testing.assert_allclose(sw, 1 / deg[si[1]], rtol=1e-6)
    # mean aggregation: every column of the normalised adjacency sums to 1
    colsum = np.zeros(V)
    np.add.at(colsum, si[1], sw)
    np.testing.assert_allclose(colsum, 1, rtol=1e-5)


def test_clustergcn_norm_and_conv_closed_forms():
    rng = np.random.default_rng(81)
    V = 40
    ei, _ = rand_graph(rng, V, 260, loops=False)
    ei = np.unique(np.concatenate([ei, ei[::-1]], axis=1), axis=1).astype(np.int32)      # symmetric, no repeats
    oi, ow = oracle.clustergcn_norm(ei, None, V)
    assert oi.shape[1] == ei.shape[1] + V
    deg = np.bincount(oi[1], minlength=V).astype(np.float64)
    assert deg.min() >= 1 and len(set(deg.tolist())) > 3                                  # irregular
    np.testing.assert_allclose(ow, 1 / deg[oi[0]], rtol=1e-6)
    A = sp.coo_matrix((ow.astype(np.float64), (oi[1], oi[0])), shape=(V, V)).toarray()   # A[dst, src]
    np.testing.assert_allclose(A.sum(0), 1, rtol=1e-5)             # what leaves a node sums to 1 ...
    assert np.abs(A.sum(1) - 1).max() > 0.05                       # ... what arrives does not
    x = rng.standard_normal((V, 5)).astype(np.float32)
    csc = oracle.cootocsc(oi, ow, V)
    np.testing.assert_allclose(oracle.aggregate_with_weight(x, csc).astype(np.float64).sum(0), x.astype(np.float64).sum(0),
                               rtol=1e-4, atol=1e-4)
    # diagonal enhancement: only the self-loops change, by lambda / deg
    li, lw = oracle.clustergcn_norm(ei, None, V, diag_lambda=0.7)
    assert np.array_equal(li, oi)
    loop = li[0] == li[1]
    np.testing.assert_allclose(lw[~loop], ow[~loop], rtol=0)
    np.testing.assert_allclose(lw[loop], (1 + 0.7) / deg[li[0][loop]], rtol=1e-6)
    # weighted, improved self-loops
    w = (rng.random(ei.shape[1]) + 0.5).astype(np.float32)
    wi, ww = oracle.clustergcn_norm(ei, w, V, improved=True, diag_lambda=0.25)
    full_w = np.concatenate([w, np.full(V, 2.0, np.float32)]).astype(np.float64)
    degw = np.zeros(V)
    np.add.at(degw, wi[1], full_w)
    want = full_w / degw[wi[0]] + 0.25 * (wi[0] == wi[1]) / degw[wi[0]]
    np.testing.assert_allclose(ww, want, rtol=1e-5)
    # the layer
    Wo, Wr, b = rng.standard_normal((5, 3)), rng.standard_normal((5, 3)), rng.standard_normal(3)
    want = A @ x.astype(np.float64) @ Wo + x.astype(np.float64) @ Wr + b
    np.testing.assert_allclose(oracle.clustergcn_conv(x, csc, Wo, Wr, b), want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.clustergcn_conv(x, csc, Wo, Wr), want - b, rtol=1e-5, atol=1e-5)


def test_get_laplacian_against_scipy_and_cheb_conv_dense():
    from scipy.sparse.csgraph import laplacian
    rng = np.random.default_rng(83)
    V = 35
    ei, _ = rand_graph(rng, V, 220, loops=True)                      # some self-loops: they must be dropped
    und = np.unique(np.sort(ei[:, ei[0] != ei[1]], axis=0), axis=1)
    wu = (rng.random(und.shape[1]) + 0.5).astype(np.float32)
    loops = np.stack([np.arange(0, V, 5)] * 2)
    ei = np.concatenate([und, und[::-1], loops], axis=1).astype(np.int32)
    w = np.concatenate([wu, wu, np.full(loops.shape[1], 9.0, np.float32)])
    A = sp.coo_matrix((np.concatenate([wu, wu]).astype(np.float64), (np.concatenate([und[0], und[1]]), np.concatenate([und[1], und[0]]))),
                      shape=(V, V)).toarray()
    dense = lambda e, v: sp.coo_matrix((v.astype(np.float64), (e[1], e[0])), shape=(V, V)).toarray()   # [dst, src]
    li, lw = oracle.get_laplacian(ei, w, None, V)
    assert li.shape[1] == 2 * und.shape[1] + V and np.array_equal(li[:, -V:], np.stack([np.arange(V)] * 2))
    np.testing.assert_allclose(dense(li, lw), laplacian(A), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dense(li, lw).sum(1), 0, atol=1e-4)
    si, sw = oracle.get_laplacian(ei, w, "sym", V)
    np.testing.assert_allclose(dense(si, sw), laplacian(A, normed=True), rtol=1e-5, atol=1e-6)
    ri, rw = oracle.get_laplacian(ei, w, "rw", V)
    deg = A.sum(1)
    # entry (src -> dst) carries -w / deg[src]: as a [dst, src] matrix that is I - A D^-1
    np.testing.assert_allclose(dense(ri, rw), np.eye(V) - A / deg[None, :], rtol=1e-5, atol=1e-6)
    # unweighted
    ui, uw = oracle.get_laplacian(ei, None, None, V)
    np.testing.assert_allclose(dense(ui, uw), laplacian((A > 0).astype(np.float64)), atol=1e-6)

    # scaled Laplacian and the layer, symmetric case: T_k from the eigenvalues
    for lam in (None, 2.0, 3.5):
        ni, nw = oracle.cheb_norm(ei, V, w, "sym", lam)
        L = laplacian(A, normed=True)
        lam_used = 2.0 * max(1.0, np.abs(L).max()) if lam is None else lam      # largest entry of L is its unit diagonal
        Lh = 2.0 * L / lam_used - np.eye(V)
        np.testing.assert_allclose(dense(ni, nw), Lh, rtol=1e-5, atol=1e-6)
        x = rng.standard_normal((V, 4)).astype(np.float32)
        Ws = [rng.standard_normal((4, 3)).astype(np.float32) for _ in range(4)]
        b = rng.standard_normal(3).astype(np.float32)
        ev, Q = np.linalg.eigh(Lh)

        def T(k):
            inside = np.abs(ev) <= 1
            t = np.where(inside, np.cos(k * np.arccos(np.clip(ev, -1, 1))),
                         np.sign(ev) ** k * np.cosh(k * np.arccosh(np.maximum(np.abs(ev), 1))))
            return (Q * t) @ Q.T
        for K in (1, 2, 4):
            want = sum(T(k) @ x.astype(np.float64) @ Ws[k].astype(np.float64) for k in range(K)) + b
            np.testing.assert_allclose(oracle.cheb_conv(x, ei, Ws[:K], b, w, "sym", lam), want, rtol=1e-4, atol=1e-4)
    # per-graph lambda_max through the batch vector: two halves scaled apart
    batch = (np.arange(V) >= V // 2).astype(np.int64)
    lam2 = np.array([2.0, 4.0], np.float32)
    bi, bw = oracle.cheb_norm(ei, V, w, "sym", lam2, batch)
    si, sw = oracle.get_laplacian(ei, w, "sym", V)
    want = 2 * sw / lam2[batch[si[0]]] - (si[0] == si[1])
    np.testing.assert_allclose(bw, want, rtol=1e-6)


# ------------------------------------------------------------ GAT pieces ----

def test_gat_forward_matches_dense_fp64():
    rng = np.random.default_rng(13)
    V, E, C = 50, 400, 6
    ei, w = rand_graph(rng, V, E)
    csc = oracle.cootocsc(ei, w, V)
    h = np.maximum(rng.standard_normal((V, C)), 0).astype(np.float32)
    a = rng.standard_normal(2 * C).astype(np.float32)
    out, alpha, _ = oracle.gat_forward(h, csc, a)
    ref = np.zeros((V, C))
    for v in range(V):
        srcs = ei[0][ei[1] == v]
        if len(srcs) == 0:
            continue
        z = h[srcs].astype(np.float64) @ a[:C] + h[v].astype(np.float64) @ a[C:]
        z = np.where(z > 0, z, 0.2 * z)
        al = sp_softmax(z)
        ref[v] = al @ h[srcs]
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5)
    o8, a8 = oracle.gat_forward_heads(np.stack([h, 2 * h], 1), csc, np.stack([a[:C], a[:C]]),
                                      np.stack([a[C:], a[C:]]))
    np.testing.assert_allclose(o8[:, 0], out, rtol=1e-6, atol=1e-7)
    assert a8.shape == (E, 2)


def test_gat_backward_matches_float64_autograd_and_finite_differences():
    """The chain of the reference operators' grad functions against autograd on a float64
    model of the same layer (per-destination softmax written out with index_add), and one
    directional finite difference of the oracle's own forward."""
    import torch
    rng = np.random.default_rng(17)
    V, E, C = 60, 500, 5
    ei, w = rand_graph(rng, V, E)
    csc = oracle.cootocsc(ei, w, V)
    row, off = csc[0], csc[1]
    dst = np.repeat(np.arange(V), np.diff(off))
    h = rng.standard_normal((V, C)).astype(np.float32)
    a = (rng.standard_normal(2 * C) / 2).astype(np.float32)
    g = rng.standard_normal((V, C)).astype(np.float32)
    g_h, g_a = oracle.gat_backward(h, csc, a, g)

    h64 = torch.from_numpy(h.astype(np.float64)).requires_grad_(True)
    a64 = torch.from_numpy(a.astype(np.float64)).requires_grad_(True)
    r, d = torch.from_numpy(row.astype(np.int64)), torch.from_numpy(dst.astype(np.int64))
    z = torch.nn.functional.leaky_relu(h64[r] @ a64[:C] + h64[d] @ a64[C:], 0.2)
    p = torch.exp(z - z.max())
    den = torch.zeros(V, dtype=torch.float64).index_add(0, d, p)
    out = torch.zeros(V, C, dtype=torch.float64).index_add(0, d, (p / den[d]).unsqueeze(1) * h64[r])
    out.backward(torch.from_numpy(g.astype(np.float64)))
    np.testing.assert_allclose(g_h, h64.grad.numpy(), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(g_a, a64.grad.numpy(), rtol=2e-4, atol=2e-5)

    # directional derivative of sum(g * forward) along a random direction of (h, a)
    dh = rng.standard_normal((V, C)).astype(np.float32)
    da = rng.standard_normal(2 * C).astype(np.float32)
    # (a coarse check: the forward runs in float32 and leaky_relu has a kink at every logit's zero)
    eps = 1e-3
    f = lambda t: float((g.astype(np.float64) * oracle.gat_forward(h + t * dh, csc, a + t * da)[0]).sum())
    fd = (f(eps) - f(-eps)) / (2 * eps)
    an = float((g_h.astype(np.float64) * dh).sum() + (g_a.astype(np.float64) * da).sum())
    assert abs(fd - an) <= 3e-2 * (abs(an) + 1)

    # heads are independent problems
    h2 = np.stack([h, -h], 1)
    gh2, gs2, gd2 = oracle.gat_backward_heads(h2, csc, np.stack([a[:C], a[:C]]), np.stack([a[C:], a[C:]]),
                                              np.stack([g, g], 1))
    np.testing.assert_array_equal(gh2[:, 0], g_h)
    np.testing.assert_array_equal(np.concatenate([gs2[0], gd2[0]]), g_a)


# ------------------------------------------------------ committed vectors ---

def test_oracle_reproduces_committed_vectors():
    """tests/golden/oracle_vectors_v64.npz was written by make_oracle_vectors.py;
    a change in oracle.c that alters any output shows up here."""
    import importlib.util
    here = os.path.join(os.path.dirname(__file__), "golden")
    spec = importlib.util.spec_from_file_location("make_oracle_vectors", os.path.join(here, "make_oracle_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    gold = np.load(os.path.join(here, "oracle_vectors_v64.npz"))
    assert set(gold.files) == set(fresh)
    for k in gold.files:
        a, b = gold[k], np.asarray(fresh[k])
        if a.dtype.kind in "iu":
            assert np.array_equal(a, b), k
        else:
            np.testing.assert_allclose(b, a, rtol=1e-6, atol=1e-7, err_msg=k)


# ------------------------------------------- callers either side of the path ---

def test_spmmcoo_reference_fixture_and_dense_product():
    g = GOLD["spmmcoo_v3"]
    x = np.array(g["x"], np.float32)
    ei = np.array(g["edge_index"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    assert oracle.spmmcoo(x, ei, w).tolist() == g["out"]
    assert oracle.spmmcoo(x, ei, w, trans_A=False).tolist() == g["out_no_trans"]
    rng = np.random.default_rng(70)
    ei, w = rand_graph(rng, 60, 700)
    x = rng.standard_normal((60, 9)).astype(np.float32)
    A = sp.coo_matrix((w.astype(np.float64), (ei[0], ei[1])), shape=(60, 60)).tocsr()
    np.testing.assert_allclose(oracle.spmmcoo(x, ei, w), A.T @ x.astype(np.float64), rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(oracle.spmmcoo(x, ei, w, trans_A=False), A @ x.astype(np.float64), rtol=1e-5, atol=2e-5)
    # same quantity as the CSC aggregation (tests/test_mp_spmm.py:28-36 prints them side by side)
    np.testing.assert_allclose(oracle.spmmcoo(x, ei, w), oracle.aggregate_with_weight(x, oracle.cootocsc(ei, w, 60)),
                               rtol=1e-5, atol=2e-5)


def test_toundirected_reference_fixture_and_bruteforce():
    g = GOLD["toundirected_v3"]
    ni, na = oracle.toundirected(np.array(g["edge_index"], np.int32), np.array(g["edge_attr"], np.float32))
    assert ni.tolist() == g["new_edge_index"] and na.tolist() == g["new_edge_attr"]
    rng = np.random.default_rng(71)
    for _ in range(10):
        V, E = int(rng.integers(1, 8)), int(rng.integers(0, 25))
        ei = rng.integers(0, V, (2, E)).astype(np.int32)
        attr = rng.integers(0, 100, E).astype(np.float32)
        ni, na = oracle.toundirected(ei, attr)
        first = {}
        for e in range(E):                      # append order: forward, then reversed
            for pair in ((int(ei[0, e]), int(ei[1, e])), (int(ei[1, e]), int(ei[0, e]))):
                first.setdefault(pair, float(attr[e]))
        want = sorted(first)
        assert [tuple(p) for p in ni.T.tolist()] == want
        assert na.reshape(-1).tolist() == [first[p] for p in want]
        assert na.shape == (1, len(want))


def test_appnp_closed_forms():
    rng = np.random.default_rng(72)
    V = 40
    ei, _ = rand_graph(rng, V, 300, loops=False)
    ei, w = oracle.gcn_norm(ei, None, V)
    csc = oracle.cootocsc(ei, w, V)
    A = sp.coo_matrix((w.astype(np.float64), (ei[1], ei[0])), shape=(V, V)).toarray()
    h = rng.standard_normal((V, 5)).astype(np.float32)
    alpha = 0.1
    np.testing.assert_allclose(oracle.appnp(h, csc, 1, alpha), (1 - alpha) * (A @ h) + alpha * h, rtol=1e-5, atol=1e-6)
    x = h.astype(np.float64)
    for _ in range(7):
        x = (1 - alpha) * (A @ x) + alpha * h
    np.testing.assert_allclose(oracle.appnp(h, csc, 7, alpha), x, rtol=1e-5, atol=1e-5)
    limit = alpha * np.linalg.solve(np.eye(V) - (1 - alpha) * A, h.astype(np.float64))
    np.testing.assert_allclose(oracle.appnp(h, csc, 300, alpha), limit, rtol=1e-4, atol=1e-5)
    assert np.array_equal(oracle.appnp(h, csc, 0, alpha), h)


def test_sgconv_dense_closed_form():
    rng = np.random.default_rng(73)
    V = 30
    ei, _ = rand_graph(rng, V, 200, loops=False)
    ei, w = oracle.gcn_norm(ei, None, V)
    csc = oracle.cootocsc(ei, w, V)
    A = sp.coo_matrix((w.astype(np.float64), (ei[1], ei[0])), shape=(V, V)).toarray()
    x = rng.standard_normal((V, 6)).astype(np.float32)
    W = rng.standard_normal((6, 4)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    want = np.linalg.matrix_power(A, 3) @ x.astype(np.float64) @ W.astype(np.float64) + b
    np.testing.assert_allclose(oracle.sgconv(x, csc, 3, W, b), want, rtol=1e-5, atol=1e-5)


def test_gprgnn_dense_closed_form():
    rng = np.random.default_rng(74)
    V = 30
    ei, _ = rand_graph(rng, V, 200, loops=False)
    ei, w = oracle.gcn_norm(ei, None, V)
    csc = oracle.cootocsc(ei, w, V)
    A = sp.coo_matrix((w.astype(np.float64), (ei[1], ei[0])), shape=(V, V)).toarray()
    x = rng.standard_normal((V, 6)).astype(np.float32)
    temp = rng.standard_normal(5).astype(np.float32)
    want = sum(float(temp[k]) * np.linalg.matrix_power(A, k) @ x.astype(np.float64) for k in range(5))
    np.testing.assert_allclose(oracle.gprgnn(x, csc, temp), want, rtol=1e-5, atol=1e-5)


def _small_symmetric(seed, V=30, E=200):
    """A gcn-normalised undirected graph (symmetric, eigenvalues in [-1, 1]), its CSC and dense form."""
    rng = np.random.default_rng(seed)
    ei, _ = rand_graph(rng, V, E, loops=False)
    ei = np.concatenate([ei, ei[::-1]], axis=1)
    ei = np.unique(ei, axis=1).astype(np.int32)
    ei, w = oracle.gcn_norm(ei, None, V)
    A = sp.coo_matrix((w.astype(np.float64), (ei[1], ei[0])), shape=(V, V)).toarray()
    assert np.allclose(A, A.T)
    return rng, ei, w, oracle.cootocsc(ei, w, V), A


def test_lightgcn_and_gcn2conv_dense_closed_forms():
    rng, ei, w, csc, A = _small_symmetric(75)
    V = A.shape[0]
    x, x0 = rng.standard_normal((V, 6)).astype(np.float32), rng.standard_normal((V, 6)).astype(np.float32)
    np.testing.assert_allclose(oracle.lightgcn(x, csc), A @ x.astype(np.float64), rtol=1e-5, atol=1e-6)
    W1, W2 = rng.standard_normal((6, 6)).astype(np.float32), rng.standard_normal((6, 6)).astype(np.float32)
    a, b = 0.1, 0.4
    x64, x064 = x.astype(np.float64), x0.astype(np.float64)
    want = A @ ((1 - b) * (1 - a) * x64 + b * x64 @ W1) + (1 - b) * a * x064 + b * x064 @ W2
    np.testing.assert_allclose(oracle.gcn2conv(x, x0, csc, W1, W2, a, b), want, rtol=1e-5, atol=1e-5)
    # beta = 0, alpha = 0: the plain product; alpha = 1: the input of the first layer comes back
    np.testing.assert_allclose(oracle.gcn2conv(x, x0, csc, W1, W2, 0.0, 0.0), A @ x64, rtol=1e-5, atol=1e-6)
    assert np.array_equal(oracle.gcn2conv(x, x0, csc, W1, W2, 1.0, 0.0), x0)


def test_evennet_adds_the_hops_the_loop_names():
    rng, ei, w, csc, A = _small_symmetric(76)
    V = A.shape[0]
    x = rng.standard_normal((V, 5)).astype(np.float32)
    x64 = x.astype(np.float64)
    alpha = 0.2
    for K in (1, 2, 3, 4, 6):
        t = alpha * (1 - alpha) ** np.arange(K + 1)
        t[-1] = (1 - alpha) ** K
        assert np.allclose(oracle.evennet_temp(K, alpha), t)
        want = t[0] * x64
        if K >= 3:
            want = want + t[3] * np.linalg.matrix_power(A, 3) @ x64
        if K >= 4:
            want = want + t[4] * np.linalg.matrix_power(A, 4) @ x64
        np.testing.assert_allclose(oracle.evennet(x, csc, K, alpha), want, rtol=1e-5, atol=1e-6)


def test_chebnet2_is_the_interpolating_polynomial_of_the_node_values():
    rng, ei, w, csc, A = _small_symmetric(77)
    V = A.shape[0]
    x = rng.standard_normal((V, 4)).astype(np.float32)
    x64 = x.astype(np.float64)
    lam, Q = np.linalg.eigh(A)
    assert lam.min() > -1 - 1e-9 and lam.max() < 1 + 1e-9
    K = 5
    nodes = np.cos((K - np.arange(K + 1) + 0.5) * np.pi / (K + 1))
    # a polynomial of degree <= K, positive at the nodes, sampled there: the filter is that polynomial of A
    f = lambda v: 0.7 + 0.3 * v - 0.5 * v ** 2 + 0.2 * v ** 3 + v ** 4
    assert (f(nodes) > 0).all()
    want = (Q * f(lam)) @ Q.T @ x64
    np.testing.assert_allclose(oracle.chebnet2(x, csc, f(nodes)), want, rtol=1e-5, atol=1e-5)
    # any non-negative values: sum' coe_i T_i(A) with T_i(A) = Q cos(i arccos lambda) Q^T
    temp = rng.random(K + 1) + 0.1
    coe = oracle.chebnet2_coefficients(temp)
    ref = np.polynomial.chebyshev.chebinterpolate(lambda v: np.interp(v, nodes, temp), K)   # same nodes, library routine
    assert np.allclose(coe[0] / 2, ref[0]) and np.allclose(coe[1:], ref[1:])
    Ti = lambda i: (Q * np.cos(i * np.arccos(np.clip(lam, -1, 1)))) @ Q.T
    want = (coe[0] / 2 * Ti(0) + sum(coe[i] * Ti(i) for i in range(1, K + 1))) @ x64
    np.testing.assert_allclose(oracle.chebnet2(x, csc, temp), want, rtol=1e-5, atol=1e-5)
    # negative parameters are clamped at zero first
    assert np.array_equal(oracle.chebnet2(x, csc, [-1.0, 2.0, -3.0]), oracle.chebnet2(x, csc, [0.0, 2.0, 0.0]))


def test_bernnet_dense_closed_form_and_binomial_theorem():
    from math import comb
    rng, ei, w, csc, A = _small_symmetric(78)
    V = A.shape[0]
    x = rng.standard_normal((V, 4)).astype(np.float32)
    x64 = x.astype(np.float64)
    # L = I - A and 2I - L = I + A as weighted graphs of their own
    def as_csc(M):
        r, c = np.nonzero(M)
        e = np.stack([c, r]).astype(np.int32)             # edge j -> i carries M[i, j]
        return oracle.cootocsc(e, M[r, c].astype(np.float32), V)
    L, L2 = np.eye(V) - A, np.eye(V) + A
    csc1, csc2 = as_csc(L), as_csc(L2)
    K = 4
    temp = rng.random(K + 1).astype(np.float32)
    want = sum(comb(K, i) / 2 ** K * float(temp[i]) * np.linalg.matrix_power(L, i) @ np.linalg.matrix_power(L2, K - i) @ x64
               for i in range(K + 1))
    np.testing.assert_allclose(oracle.bernnet(x, csc1, csc2, temp), want, rtol=1e-5, atol=1e-5)
    # all weights one: ((L + (2I - L)) / 2)^K = I
    np.testing.assert_allclose(oracle.bernnet(x, csc1, csc2, np.ones(K + 1)), x64, rtol=1e-5, atol=1e-5)
    # two unrelated matrices (they do not commute): the order A1^i A2^(K-i) matters
    B = rng.standard_normal((V, V)) * (rng.random((V, V)) < 0.2)
    want = sum(comb(3, i) / 8 * np.linalg.matrix_power(L, i) @ np.linalg.matrix_power(B, 3 - i) @ x64 for i in range(4))
    np.testing.assert_allclose(oracle.bernnet(x, csc1, as_csc(B), np.ones(4)), want, rtol=1e-4, atol=1e-4)
    assert np.array_equal(oracle.bernnet(x, csc1, csc2, [-1.0, 1.0, -2.0]), oracle.bernnet(x, csc1, csc2, [0.0, 1.0, 0.0]))


# -------------------------------------------------- sampled-subgraph operators ---

def _global_csc(rng, V, E):
    ei, w = rand_graph(rng, V, E)
    row, off, _ = oracle.cootocsc(ei, w, V)
    return off, row


def test_gpuinitco_and_getweight_small_cases():
    rng = np.random.default_rng(80)
    goff, grow = _global_csc(rng, 30, 200)
    dst = rng.permutation(30)[:12].astype(np.int32)
    out = oracle.gpuinitco(12, 5, dst, goff)
    assert out[0] == 0 and out[1:].tolist() == [min(int(goff[d + 1] - goff[d]), 5) for d in dst]
    # getweight on a full small graph equals 1/sqrt(outdeg[src] * indeg[dst]) from bincounts
    ids = np.arange(30, dtype=np.int32)
    w = oracle.getweight(30, ids, ids, goff, grow)
    indeg = np.diff(goff)
    outdeg = np.bincount(grow, minlength=30)
    col = np.repeat(ids, indeg)
    np.testing.assert_allclose(w, 1.0 / np.sqrt(outdeg[grow].astype(np.float64) * indeg[col]), rtol=3e-7)


def test_csctocsr_readme_known_answer_and_dropped_sources():
    g = GOLD["csctocsr_readme_v4"]
    ids = np.arange(4, dtype=np.int32)
    r_o, c_i = oracle.csctocsr(np.array(g["column_offset"]), np.array(g["row_indices"]), ids, ids)
    assert r_o.tolist() == g["row_offset"] and c_i.tolist() == g["column_indices"]
    # a layer: dst ids are global, src lists only some of the row indices
    off = np.array([0, 2, 3, 6]); row = np.array([7, 9, 7, 4, 9, 5]); dst = np.array([20, 21, 22]); src = np.array([9, 7, 5])
    r_o, c_i = oracle.csctocsr(off, row, dst, src)
    assert r_o.tolist() == [0, 2, 4, 5]                      # 9: cols 20, 22; 7: cols 20, 21; 5: col 22; 4 dropped
    assert c_i.tolist() == [20, 22, 20, 21, 22, 0]


def test_sampleprocessing_invariants_and_uniformity():
    rng = np.random.default_rng(81)
    V = 60
    goff, grow = _global_csc(rng, V, 1500)
    dst = rng.permutation(V)[:40].astype(np.int32)
    for fanout in (-1, 3, 10, 1000):
        cnt = np.diff(goff)[dst] if fanout < 0 else np.minimum(np.diff(goff)[dst], fanout)
        loff = np.concatenate([[0], np.cumsum(cnt)]).astype(np.int32)
        a = oracle.sampleprocessing(fanout, dst, loff, goff, grow, seed=5)
        assert np.array_equal(a, oracle.sampleprocessing(fanout, dst, loff, goff, grow, seed=5))
        for i, d in enumerate(dst):
            nb = grow[goff[d]:goff[d + 1]]
            got = a[loff[i]:loff[i + 1]]
            if fanout < 0 or len(nb) <= fanout:
                assert np.array_equal(got, nb)                       # the copy branch of the reference, exactly
            else:
                # a sub-sequence of the neighbour list with `fanout` distinct positions
                pos, it = [], 0
                for v in got:
                    while nb[it] != v:
                        it += 1
                    pos.append(it)
                    it += 1
                assert len(pos) == fanout and len(set(pos)) == fanout
    # uniformity: one destination with 12 distinct neighbours, fanout 4, many seeds
    goff1 = np.array([0, 12], np.int32); grow1 = np.arange(100, 112, dtype=np.int32)
    hits = np.zeros(12)
    n = 6000
    for s in range(n):
        hits[oracle.sampleprocessing(4, np.array([0], np.int32), np.array([0, 4], np.int32), goff1, grow1, seed=s) - 100] += 1
    expect = n * 4 / 12
    assert np.all(np.abs(hits - expect) < 5 * np.sqrt(expect))
    assert len({tuple(oracle.sampleprocessing(4, np.array([0], np.int32), np.array([0, 4], np.int32), goff1, grow1,
                                              seed=s)) for s in range(300)}) > 150


def test_cross_entropy_closed_forms():
    from scipy.special import logsumexp
    rng = np.random.default_rng(21)
    V, C = 37, 11
    x = (rng.standard_normal((V, C)) * 3).astype(np.float32)
    y = rng.integers(0, C, V)
    loss, grad = oracle.cross_entropy_loss(x, y)
    want = np.mean(logsumexp(x.astype(np.float64), axis=1) - x[np.arange(V), y].astype(np.float64))
    assert abs(loss - want) < 1e-12
    # equal logits: log(C); adding a constant per row changes nothing
    assert abs(oracle.cross_entropy_loss(np.zeros((5, C)), np.arange(5))[0] - np.log(C)) < 1e-12
    shifted, gshift = oracle.cross_entropy_loss(x.astype(np.float64) + rng.standard_normal((V, 1)) * 50, y)
    assert abs(shifted - loss) < 1e-9 and np.allclose(gshift, grad, atol=1e-12)
    # the gradient: rows sum to zero, and it matches central differences
    assert np.allclose(grad.sum(axis=1), 0, atol=1e-15)
    x64 = x.astype(np.float64)
    for (i, c) in ((0, 0), (3, y[3]), (36, 10), (17, 4)):
        h = 1e-6
        xp, xm = x64.copy(), x64.copy()
        xp[i, c] += h
        xm[i, c] -= h
        fd = (oracle.cross_entropy_loss(xp, y)[0] - oracle.cross_entropy_loss(xm, y)[0]) / (2 * h)
        assert abs(fd - grad[i, c]) < 1e-8
    # labels outside [0, C) are left out of the mean and of the gradient
    y2 = y.copy()
    y2[[1, 5]] = (-100, C)
    loss2, grad2 = oracle.cross_entropy_loss(x, y2)
    keep = np.ones(V, bool)
    keep[[1, 5]] = False
    want2 = np.mean(logsumexp(x64[keep], axis=1) - x64[keep, y[keep]])
    assert abs(loss2 - want2) < 1e-12 and not grad2[[1, 5]].any()
    assert np.isnan(oracle.cross_entropy_loss(x, np.full(V, -1))[0])
    # very large logits stay finite
    big = np.array([[1e4, -1e4, 0.0]])
    assert abs(oracle.cross_entropy_loss(big, [1])[0] - 2e4) < 1e-6


# ------------------------------------- literal inputs of the reference's remaining tests ---
def test_reference_test_inputs_getweight_gpuinitco_fromtonodes_scatter():
    g = GOLD["getweight_v4"]
    w = oracle.getweight(g["vtx_size"], np.array(g["dst"]), np.array(g["src"]), np.array(g["column_offset"]),
                         np.array(g["row_indices"]))
    np.testing.assert_allclose(w, g["edge_weight"], rtol=2e-7)
    g = GOLD["gpuinitco_v4"]
    out = oracle.gpuinitco(g["dst_size"], g["fanout"], np.array(g["csc_layer_dst"]), np.array(g["csc_global_column_offset"]))
    assert out.tolist() == g["out"]
    g = GOLD["fromtonodes_v5"]
    a = oracle.from_nodes(g["column_offset"], g["row_indices"], g["nodes"])
    b = oracle.from_nodes(g["row_offset"], g["column_indices"], g["nodes"])
    assert a.tolist() == g["from_nodes"] and b.tolist() == g["to_nodes"]
    assert sorted(set(a.tolist())) == g["from_nodes_as_set"] and sorted(set(b.tolist())) == g["to_nodes_as_set"]
    g = GOLD["edgetovertex_v3"]
    out = oracle.edgetovertex(np.array(g["x"], np.float32), g["row_indices"], g["column_offset"], 1)
    assert out.tolist() == g["out"]
    g = GOLD["scatter_to_edge_v3"]
    x = np.array(g["x"], np.float32)
    assert oracle.scattertoedge(x, g["row_indices"], g["column_offset"], 1).tolist() == g["out_dst"]
    assert oracle.scattertoedge(x, g["row_indices"], g["column_offset"], 0).tolist() == g["out_src"]
