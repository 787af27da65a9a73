"""Per-graph plans (csrc/plan.hip) through the C ABI.

The reference's aggregate is one launch per call (ops/cpp/aggregate_op.cc:93-106); a plan holds
what the merge-path kernels otherwise work out per call from the offsets.  Checked here: the
plan's arrays against a numpy model of the partition rule (a chunk boundary inside a row of at
most chunk / 2 entries moves back to the row's first entry), the planned entry points bit for
bit against the unplanned ones and within tolerance against the oracle's loop
(aggregate_op.cc:42-58, edgesoftmax_op.cc:48-65), and that the Python wrappers rebuild a plan
when the offsets are written in place or rebound."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu

SPMM, GAT, TILES = 0, 1, 2
GROUP = 32


def lib():
    from jittorgeometric_amd import _lib
    return _lib, _lib.load()


def build_plan(off_g, R, E, kind):
    L, l = lib()
    nbytes = L.query(l.jgamd_csx_plan_bytes, R, E, kind)
    plan = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=dev())
    L.check(l.jgamd_csx_plan(L.ptr(off_g), R, E, kind, L.ptr(plan), nbytes, L.stream_ptr(dev())))
    n_fix, n_grp = ctypes.c_int32(-9), ctypes.c_int32(-9)
    if kind != TILES:
        L.check(l.jgamd_csx_plan_counts(L.ptr(plan), ctypes.byref(n_fix), ctypes.byref(n_grp), L.stream_ptr(dev())))
    return plan, n_fix.value, n_grp.value


def spmm_chunk(M):
    c = 512
    while c > 32 and M // c < 32768:
        c >>= 1
    return c


def gat_chunk(M):
    c = 128
    while c > 64 and M // c < 16384:
        c >>= 1
    return c


INLINE_GROUPS = 2      # the product's finishing kernel sums the groups of a row that crosses at most this many


def model_partition(off, R, E, chunk, inline_groups=0):
    """start[k] = (row, entry), the fix list and the group list, as the kernels define them."""
    M = R + E
    nchunks = max(-(-M // chunk), 1)
    first = off[:R].astype(np.int64) + np.arange(R)          # merged position of every row's first item
    start = np.zeros((nchunks + 1, 2), np.int64)
    for k in range(nchunks):
        p = k * chunk
        r = int(np.searchsorted(first, p, side="right")) - 1
        s, ln = int(off[r]), int(off[r + 1] - off[r])
        j = p - r
        if ln <= chunk // 2 and s + r < p:
            j = s
        start[k] = (r, j)
    start[nchunks] = (R, E)
    fix = [k for k in range(nchunks)
           if start[k, 0] < R and start[k + 1, 0] > start[k, 0] and start[k, 1] > off[start[k, 0]]]
    ngroups = -(-nchunks // GROUP)
    grp = [g for g in range(ngroups)
           if (g + 1) * GROUP < nchunks and start[(g + 1) * GROUP, 0] < R
           and start[(g + 1) * GROUP, 1] > off[start[(g + 1) * GROUP, 0]]]

    def crossings(g):     # group boundaries crossed by the row that continues past group g
        r = int(start[(g + 1) * GROUP, 0])
        return (int(off[r + 1]) + r) // chunk // GROUP - (int(off[r]) + r) // chunk // GROUP
    grp = [g for g in grp if crossings(g) > inline_groups]
    return nchunks, start, fix, grp


def read_plan(plan, nchunks):
    raw = plan.cpu().numpy()
    counts = raw[:16].view(np.int32)
    a256 = lambda n: (n + 255) // 256 * 256
    o = 256
    start = raw[o:o + 8 * (nchunks + 1)].view(np.int32).reshape(-1, 2)
    o += a256(8 * (nchunks + 1))
    fix = raw[o:o + 4 * nchunks].view(np.int32)
    o += a256(4 * nchunks)
    grp = raw[o:o + 4 * (-(-nchunks // GROUP))].view(np.int32)
    return counts, start, fix, grp


def csc_of(rng, V, E, hubs, hub_share=0.3):
    ei, w = rand_graph(rng, V, E, hubs, hub_share)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    return idx, off, wt


@pytest.mark.parametrize("V,E,hubs,share,kind,seed", [
    (3000, 20000, 0, 0.0, SPMM, 0),          # short rows only: nothing is ever cut
    (3000, 60000, 2, 0.4, SPMM, 1),          # two hubs of thousands of entries
    (500, 400000, 1, 0.7, SPMM, 2),          # one row across hundreds of chunks (several groups)
    (40000, 3000, 0, 0.0, SPMM, 3),          # mostly empty rows
    (3000, 60000, 2, 0.05, SPMM, 6),         # rows across a few dozen chunks: cut, but no group is listed
    (3000, 60000, 2, 0.4, GAT, 4),
    (200, 2000000, 1, 0.9, GAT, 5),          # chunk 128, a row across thousands of chunks
])
def test_plan_arrays_follow_the_partition_rule(V, E, hubs, share, kind, seed):
    rng = np.random.default_rng(seed)
    idx, off, wt = csc_of(rng, V, E, hubs, share)
    chunk = (spmm_chunk if kind == SPMM else gat_chunk)(V + E)
    nchunks, start, fix, grp = model_partition(off, V, E, chunk, INLINE_GROUPS if kind == SPMM else 0)
    plan, n_fix, n_grp = build_plan(to_gpu(off), V, E, kind)
    counts, g_start, g_fix, g_grp = read_plan(plan, nchunks)
    assert np.array_equal(g_start, start.astype(np.int32))
    assert (n_fix, n_grp) == (len(fix), len(grp)) == (int(counts[0]), int(counts[1]))
    assert g_fix[:n_fix].tolist() == fix and g_grp[:n_grp].tolist() == grp
    # no chunk is empty, none strays more than chunk / 2 items from its nominal size
    pos = start[:, 0] + start[:, 1]
    assert (np.diff(pos) > 0).all() and (np.abs(np.diff(pos)[:-1] - chunk) <= chunk // 2).all()
    if hubs == 0 and np.diff(off).max() <= chunk // 2:
        assert n_fix == 0 and n_grp == 0
    if seed == 6:
        assert n_grp == 0 and len(model_partition(off, V, E, chunk)[3]) > 0 and np.diff(off).max() > GROUP * chunk
    if seed in (1, 2):
        assert n_grp > 0


def planned(plan, tiles, hints, off, idx, w, x, R, beta=1.0, alpha=0.0, h=None, flags=0):
    L, l = lib()
    C, F = x.shape
    E = idx.shape[0] if idx is not None else C
    out = torch.full((R, F), float("nan"), dtype=torch.float32, device=dev())
    nbytes = L.query(l.jgamd_spmm_csx_planned_workspace, R, E, F)
    ws = L.workspace(nbytes, dev())
    h_rows = R if h is None or h.dim() == 2 else 1
    L.check(l.jgamd_spmm_csx_planned(L.ptr(plan), L.ptr(tiles), hints[0], hints[1], L.ptr(off), L.ptr(idx), L.ptr(w),
                                     L.ptr(x), L.ptr(out), beta, alpha, L.ptr(h), h_rows, flags, R, C, E, F, L.ptr(ws),
                                     nbytes, L.stream_ptr(dev())))
    return out


def unplanned(off, idx, w, x, R, beta=1.0, alpha=0.0, h=None):
    L, l = lib()
    C, F = x.shape
    E = idx.shape[0] if idx is not None else C
    out = torch.full((R, F), float("nan"), dtype=torch.float32, device=dev())
    nbytes = L.query(l.jgamd_spmm_csx_workspace, R, E, F)
    ws = L.workspace(nbytes, dev())
    h_rows = R if h is None or h.dim() == 2 else 1
    if h is None and beta == 1.0:
        L.check(l.jgamd_spmm_csx(L.ptr(off), L.ptr(idx), L.ptr(w), L.ptr(x), L.ptr(out), R, C, E, F, L.ptr(ws), nbytes,
                                 L.stream_ptr(dev())))
    else:
        L.check(l.jgamd_spmm_csx_axpby(L.ptr(off), L.ptr(idx), L.ptr(w), L.ptr(x), L.ptr(out), beta, alpha, L.ptr(h),
                                       h_rows, R, C, E, F, L.ptr(ws), nbytes, L.stream_ptr(dev())))
    return out


@pytest.mark.parametrize("F", [3, 16, 47, 64, 100, 128, 256, 300])
@pytest.mark.parametrize("V,E,hubs,share", [(3000, 20000, 0, 0.0), (3000, 90000, 2, 0.4), (400, 600000, 1, 0.8),
                                            (3000, 60000, 2, 0.05)])
def test_planned_product_equals_unplanned_and_oracle(V, E, hubs, share, F):
    rng = np.random.default_rng(F * 7 + V)
    idx, off, wt = csc_of(rng, V, E, hubs, share)
    x = rng.standard_normal((V, F)).astype(np.float32)
    off_g, idx_g, w_g, x_g = to_gpu(off), to_gpu(idx), to_gpu(wt), to_gpu(x)
    plan, n_fix, n_grp = build_plan(off_g, V, E, SPMM)
    base = unplanned(off_g, idx_g, w_g, x_g, V)
    for hints in ((n_fix, n_grp), (-1, -1), (n_fix + 5, n_grp + 3)):
        got = planned(plan, None, hints, off_g, idx_g, w_g, x_g, V)
        assert torch.equal(got, base), "hints %s" % (hints,)
    want, terms = oracle.aggregate_f64(x, idx, off, wt)
    assert_close(base.cpu().numpy(), want, terms, what="planned product F=%d" % F)
    # rows the partition never cuts are the oracle's own sequential sum whenever the compiler's
    # fused multiply-add does not change a bit: at least the sums of whole numbers are exact
    xi = rng.integers(-4, 5, (V, F)).astype(np.float32)
    wi = rng.integers(-3, 4, E).astype(np.float32)
    got = planned(plan, None, (n_fix, n_grp), off_g, idx_g, to_gpu(wi), to_gpu(xi), V).cpu().numpy()
    assert np.array_equal(got, oracle.aggregate(xi, idx, off, wi))


def test_planned_product_with_row_finish_and_without_indices():
    rng = np.random.default_rng(5)
    V, E, F = 2500, 70000, 96
    idx, off, wt = csc_of(rng, V, E, 2, 0.5)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((V, F)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    off_g, idx_g, w_g, x_g = to_gpu(off), to_gpu(idx), to_gpu(wt), to_gpu(x)
    plan, n_fix, n_grp = build_plan(off_g, V, E, SPMM)
    assert n_fix > 0
    for hh in (to_gpu(h), to_gpu(b)):
        got = planned(plan, None, (n_fix, n_grp), off_g, idx_g, w_g, x_g, V, 0.9, 0.1, hh)
        assert torch.equal(got, unplanned(off_g, idx_g, w_g, x_g, V, 0.9, 0.1, hh))
    # the row clamped at zero in the row store (a layer's relu): exactly max(0, .) of the unclamped call
    for hh in (to_gpu(h), to_gpu(b), None):
        got = planned(plan, None, (n_fix, n_grp), off_g, idx_g, w_g, x_g, V, 1.0, 1.0 if hh is not None else 0.0, hh, flags=1)
        ref = planned(plan, None, (n_fix, n_grp), off_g, idx_g, w_g, x_g, V, 1.0, 1.0 if hh is not None else 0.0, hh)
        assert torch.equal(got, torch.relu(ref)) and (got == 0).any()
    # per-entry rows summed per column (ScatterToVertex): idx = NULL, w = NULL
    xe = to_gpu(rng.standard_normal((E, F)).astype(np.float32))
    got = planned(plan, None, (n_fix, n_grp), off_g, None, None, xe, V)
    assert torch.equal(got, unplanned(off_g, None, None, xe, V))
    want = np.add.reduceat(np.vstack([xe.cpu().numpy().astype(np.float64), np.zeros((1, F))]),
                           np.minimum(off[:-1], E), axis=0)
    want[np.diff(off) == 0] = 0
    terms = np.add.reduceat(np.vstack([np.abs(xe.cpu().numpy()).astype(np.float64), np.zeros((1, F))]),
                            np.minimum(off[:-1], E), axis=0)
    assert_close(got.cpu().numpy(), want, terms, what="column sums of per-entry rows")


@pytest.mark.parametrize("F", [1, 2, 4, 8])
@pytest.mark.parametrize("case", ["hubs", "empty_columns", "no_entries_in_most", "tile_edges"])
def test_narrow_rows_with_a_tile_plan(case, F):
    """Rows of 1, 2, 4 or 8 floats go through the tile kernels; empty columns (before the first
    entry, between tiles, after the last entry) must come out as zeros without a zeroing pass."""
    rng = np.random.default_rng(F + len(case))
    if case == "hubs":
        V, E = 3000, 90000
        idx, off, wt = csc_of(rng, V, E, 2, 0.4)
    elif case == "empty_columns":
        V, E = 50000, 9000                       # most columns empty, everywhere
        idx, off, wt = csc_of(rng, V, E, 0)
    elif case == "no_entries_in_most":
        V, E = 9000, 5000                        # entries only in columns 3000..3999
        ei, w = rand_graph(rng, 1000, E)
        ei[1] += 3000
        idx, off, wt = oracle.cootocsc(ei, w, V)
    else:
        V = 40                                   # columns that end exactly on tile edges (1024 / 2048)
        deg = np.zeros(V, np.int64)
        deg[[3, 4, 9, 10, 30]] = [1024, 1024, 2048, 2048, 4096]
        deg[20] = 7
        E = int(deg.sum())
        dst = np.repeat(np.arange(V), deg).astype(np.int32)
        ei = np.stack([rng.integers(0, V, E).astype(np.int32), dst])
        w = rng.standard_normal(E).astype(np.float32)
        idx, off, wt = oracle.cootocsc(ei, w, V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    off_g, idx_g, w_g, x_g = to_gpu(off), to_gpu(idx), to_gpu(wt), to_gpu(x)
    tiles, _, _ = build_plan(off_g, V, E, TILES)
    got = planned(None, tiles, (-1, -1), off_g, idx_g, w_g, x_g, V)
    assert torch.equal(got, unplanned(off_g, idx_g, w_g, x_g, V))
    want, terms = oracle.aggregate_f64(x, idx, off, wt)
    assert_close(got.cpu().numpy(), want, terms, what="%s F=%d" % (case, F))
    assert (got.cpu().numpy()[np.diff(off) == 0] == 0).all()


@pytest.mark.parametrize("F", [1, 2, 4, 8])
def test_narrow_rows_with_a_row_finish_take_the_chunk_kernels(F):
    """The tile kernels have no row finish: beta * A x + alpha * h (a layer's bias, an APPNP hop, a
    fused relu) at 1, 2, 4 or 8 floats per row goes through the chunk kernels, through the
    wrappers on the first use of the offsets (no plan yet) and on the second (planned); a planned
    call that brings only the tile plan for such a product is refused with a message, before
    anything is enqueued."""
    from jittorgeometric_amd.ops._common import spmm, spmm_axpby
    L, l = lib()
    rng = np.random.default_rng(20 + F)
    V, E = 3000, 90000
    idx, off, wt = csc_of(rng, V, E, 2, 0.4)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((V, F)).astype(np.float32)
    off_g, idx_g, w_g, x_g, h_g = to_gpu(off), to_gpu(idx), to_gpu(wt), to_gpu(x), to_gpu(h)
    want, terms = oracle.aggregate_f64(x, idx, off, wt)
    for use in range(3):
        got = spmm_axpby(off_g, idx_g, w_g, x_g, V, 0.9, 0.1, h_g).cpu().numpy()
        assert_close(got, 0.9 * want + 0.1 * h, 0.9 * terms + 0.1 * np.abs(h), what="axpby F=%d, use %d" % (F, use))
        got = spmm_axpby(off_g, idx_g, w_g, x_g, V, 1.0, 1.0, h_g[0], relu=True).cpu().numpy()
        assert_close(got, np.maximum(want + h[0], 0), terms + np.abs(h[0]), what="relu F=%d, use %d" % (F, use))
        assert_close(spmm(off_g, idx_g, w_g, x_g, V).cpu().numpy(), want, terms, what="plain F=%d, use %d" % (F, use))
    tiles, _, _ = build_plan(off_g, V, E, TILES)
    out = torch.empty((V, F), device=dev())
    nbytes = L.query(l.jgamd_spmm_csx_planned_workspace, V, E, F)
    ws = L.workspace(nbytes, dev())
    rc = l.jgamd_spmm_csx_planned(None, L.ptr(tiles), -1, -1, L.ptr(off_g), L.ptr(idx_g), L.ptr(w_g), L.ptr(x_g), L.ptr(out),
                                  0.9, 0.1, L.ptr(h_g), V, 0, V, V, E, F, L.ptr(ws), nbytes, L.stream_ptr(dev()))
    assert rc == -1 and b"chunk plan" in l.jgamd_last_error()


@pytest.mark.parametrize("H", [1, 2, 4, 8])
def test_planned_edge_softmax_equals_unplanned(H):
    L, l = lib()
    rng = np.random.default_rng(H)
    V, E = 4000, 120000
    idx, off, wt = csc_of(rng, V, E, 2, 0.4)
    x = to_gpu((3 * rng.standard_normal((E, H))).astype(np.float32))
    g = to_gpu(rng.standard_normal((E, H)).astype(np.float32))
    off_g = to_gpu(off)
    tiles, _, _ = build_plan(off_g, V, E, TILES)
    nbytes = L.query(l.jgamd_edge_softmax_workspace, V, E)
    ws = L.workspace(nbytes, dev())
    s = L.stream_ptr(dev())
    y0, y1, d0, d1 = (torch.full((E, H), float("nan"), device=dev()) for _ in range(4))
    L.check(l.jgamd_edge_softmax_fwd(L.ptr(off_g), L.ptr(x), L.ptr(y0), V, E, H, L.ptr(ws), nbytes, s))
    L.check(l.jgamd_edge_softmax_fwd_planned(L.ptr(tiles), L.ptr(off_g), L.ptr(x), L.ptr(y1), V, E, H, L.ptr(ws), nbytes, s))
    L.check(l.jgamd_edge_softmax_bwd(L.ptr(off_g), L.ptr(y0), L.ptr(g), L.ptr(d0), V, E, H, L.ptr(ws), nbytes, s))
    L.check(l.jgamd_edge_softmax_bwd_planned(L.ptr(tiles), L.ptr(off_g), L.ptr(y0), L.ptr(g), L.ptr(d1), V, E, H,
                                             L.ptr(ws), nbytes, s))
    assert torch.equal(y0, y1) and torch.equal(d0, d1)
    # against the exact softmax (the oracle's sequential fp32 denominator has itself drifted on the
    # hub columns of this graph; tests/test_gpu_edge_ops.py compares with it at its own allowance)
    seg = np.repeat(np.arange(V), np.diff(off))
    x64 = x.cpu().numpy().astype(np.float64)
    mx = np.full((V, H), -np.inf)
    np.maximum.at(mx, seg, x64)
    p64 = np.exp(x64 - mx[seg])
    den = np.zeros((V, H))
    np.add.at(den, seg, p64)
    assert_close(y1.cpu().numpy(), p64 / den[seg], rtol=1e-5, atol=1e-7, what="softmax H=%d vs float64" % H)


def test_wrappers_keep_one_plan_per_offsets_and_rebuild_it_when_they_change():
    from jittorgeometric_amd import CSC
    from jittorgeometric_amd.ops import aggregateWithWeight
    from jittorgeometric_amd.ops._common import PLAN_SPMM, csc_arrays, csx_plan
    rng = np.random.default_rng(11)
    V, E, F = 2000, 50000, 64
    idx, off, wt = csc_of(rng, V, E, 1, 0.5)
    csc = CSC(to_gpu(idx), to_gpu(off), to_gpu(wt))
    x = to_gpu(rng.standard_normal((V, F)).astype(np.float32))
    out1 = aggregateWithWeight(x, csc, None)
    off_g = csc_arrays(csc)[0]
    # the first call partitions on the fly; the plan is built when the same offsets come again
    assert "_jgamd_plans" in off_g.__dict__ and PLAN_SPMM not in off_g._jgamd_plans
    assert torch.equal(aggregateWithWeight(x, csc, None), out1)
    assert PLAN_SPMM in off_g._jgamd_plans
    p1 = csx_plan(off_g, V, E, PLAN_SPMM)
    assert p1[0] is not None and csx_plan(off_g, V, E, PLAN_SPMM)[0] is p1[0]      # kept
    assert torch.equal(aggregateWithWeight(x, csc, None), out1)
    # the same arrays regrouped: column 0 gives its entries to column 1 (offsets written in place)
    new_off = off.copy()
    new_off[1] = 0
    csc.column_offset.copy_(to_gpu(new_off))
    out2 = aggregateWithWeight(x, csc, None)
    assert torch.equal(aggregateWithWeight(x, csc, None), out2)         # without a plan, then with the new one
    p2 = csx_plan(csc_arrays(csc)[0], V, E, PLAN_SPMM, now=True)
    assert p2[0] is not None and p2[0] is not p1[0]                     # rebuilt
    want, terms = oracle.aggregate_f64(x.cpu().numpy(), idx, new_off, wt)
    assert_close(out2.cpu().numpy(), want, terms, what="after the offsets changed in place")
    # a rebound attribute is another tensor with its own plan
    csc.column_offset = to_gpu(off)
    assert torch.equal(aggregateWithWeight(x, csc, None), out1)


def test_plan_entry_points_reject_bad_arguments():
    L, l = lib()
    n = ctypes.c_size_t(0)
    bad = ctypes.c_void_p(256)
    assert l.jgamd_csx_plan_bytes(10, 20, 3, ctypes.byref(n)) == -2          # no such kind
    assert l.jgamd_csx_plan_bytes(-1, 20, 0, ctypes.byref(n)) == -2
    assert l.jgamd_csx_plan_bytes(10, 20, 0, None) == -1
    assert l.jgamd_csx_plan(None, 10, 20, 0, bad, 1 << 20, None) == -1
    assert l.jgamd_csx_plan(bad, 10, 20, 0, bad, 8, None) == -3             # plan too small
    assert l.jgamd_csx_plan(bad, 10, 20, 0, ctypes.c_void_p(260), 1 << 20, None) == -5
    assert l.jgamd_spmm_csx_planned(None, None, -1, -1, bad, bad, bad, bad, bad, 1.0, 0.0, None, 1, 0, 4, 4, 5, 16, bad,
                                    1 << 20, None) == -1
    assert l.jgamd_spmm_csx_planned(bad, None, -1, -1, bad, bad, bad, bad, bad, 1.0, 0.0, None, 1, 2, 4, 4, 5, 16, bad,
                                    1 << 20, None) == -2                        # unknown flag
    assert l.jgamd_edge_softmax_fwd_planned(None, bad, bad, bad, 4, 5, 1, bad, 1 << 20, None) == -1


@pytest.mark.parametrize("F,wide", [(47, 64), (33, 64), (100, 128), (130, 160), (64, 96)])
def test_rows_of_x_padded_apart(F, wide):
    """x as a [C,F] view of rows `wide` floats apart: gathered in place, the same bits as from a
    dense copy, with and without a row finish."""
    from jittorgeometric_amd.ops._common import csx_plan, spmm, spmm_axpby
    rng = np.random.default_rng(F)
    V, E = 3000, 90000
    idx, off, wt = csc_of(rng, V, E, 2, 0.4)
    off_g, idx_g, w_g = to_gpu(off), to_gpu(idx), to_gpu(wt)
    buf = torch.full((V, wide), float("nan"), dtype=torch.float32, device=dev())
    x = buf[:, :F]
    x.copy_(to_gpu(rng.standard_normal((V, F)).astype(np.float32)))
    assert x.stride(0) == wide and not x.is_contiguous()
    dense = x.contiguous()
    h = to_gpu(rng.standard_normal((V, F)).astype(np.float32))
    csx_plan(off_g, V, E, SPMM, now=True)                 # the planned entry point is the one that takes a stride
    assert torch.equal(spmm(off_g, idx_g, w_g, x, V), spmm(off_g, idx_g, w_g, dense, V))
    assert torch.equal(spmm_axpby(off_g, idx_g, w_g, x, V, 0.7, 0.3, h, relu=True),
                       spmm_axpby(off_g, idx_g, w_g, dense, V, 0.7, 0.3, h, relu=True))
    want, terms = oracle.aggregate_f64(dense.cpu().numpy(), idx, off, wt)
    assert_close(spmm(off_g, idx_g, w_g, x, V).cpu().numpy(), want, terms, what="padded rows F=%d" % F)
    # offsets without a plan yet (first use): the wrapper falls back to a dense copy, same result
    off2 = off_g.clone()
    assert torch.equal(spmm(off2, idx_g, w_g, x, V), spmm(off_g, idx_g, w_g, dense, V))
    # through the C ABI: a stride below F, or not a multiple of 4 floats, is refused
    L, l = lib()
    plan, n_fix, n_grp = build_plan(off_g, V, E, SPMM)
    out = torch.empty((V, F), dtype=torch.float32, device=dev())
    nbytes = L.query(l.jgamd_spmm_csx_planned_workspace, V, E, F)
    ws = L.workspace(nbytes, dev())
    for bad in (F - 1 if (F - 1) % 4 == 0 else F - (F % 4) - 4, wide + 2):
        rc = l.jgamd_spmm_csx_planned(L.ptr(plan), None, n_fix, n_grp, L.ptr(off_g), L.ptr(idx_g), L.ptr(w_g), L.ptr(x),
                                      L.ptr(out), 1.0, 0.0, None, V, bad << 8, V, V, E, F, L.ptr(ws), nbytes,
                                      L.stream_ptr(dev()))
        assert rc == -2 and b"stride" in l.jgamd_last_error(), bad


def test_blas_route_writes_padded_rows():
    from jittorgeometric_amd.nn.dense import padded_width, rows_times
    assert [padded_width(n) for n in (7, 32, 33, 40, 41, 47, 64, 80, 100, 128, 130)] == [7, 32, 33, 40, 64, 64, 64, 80, 100, 128, 130]
    rng = np.random.default_rng(3)
    x = to_gpu(rng.standard_normal((5000, 256)).astype(np.float32))
    w = to_gpu(rng.standard_normal((256, 47)).astype(np.float32))
    b = to_gpu(rng.standard_normal(47).astype(np.float32))
    for bias in (None, b):
        got = rows_times(x, w, bias=bias, pad_rows=True)
        assert got.shape == (5000, 47) and got.stride() == (64, 1)
        ref = rows_times(x, w, bias=bias)
        assert ref.is_contiguous() and torch.allclose(got, ref, rtol=1e-5, atol=1e-5)
    assert rows_times(x, to_gpu(rng.standard_normal((256, 128)).astype(np.float32)), pad_rows=True).is_contiguous()
