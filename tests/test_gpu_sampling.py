"""Sampled-subgraph operators on the GPU against the CPU oracle: gpuinitco, getweight,
csctocsr (bit-exact / fp32-exact), and sampleprocessing, whose sampled branch has no
reference answer (the reference draws with rand() / clock-seeded curand): it is compared
with the oracle's seeded restatement of the same algorithm, bit for bit."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def global_csc(rng, V, E, hubs=0):
    ei, w = rand_graph(rng, V, E, hubs)
    row, off, _ = oracle.cootocsc(ei, w, V)
    return off, row


@pytest.mark.parametrize("V,E,n_dst,fanout,seed", [(50, 400, 20, 5, 0), (5000, 90000, 3000, 10, 1),
                                                   (5000, 90000, 5000, -1, 2), (300, 60000, 300, 25, 3),
                                                   (2000, 30000, 1, 1, 4), (2000, 30000, 700, 1000, 5)])
def test_sampleprocessing_matches_seeded_oracle(V, E, n_dst, fanout, seed):
    from jittorgeometric_amd.ops import gpuinitco, sampleprocessing
    rng = np.random.default_rng(seed)
    goff, grow = global_csc(rng, V, E, hubs=2)
    dst = rng.permutation(V)[:n_dst].astype(np.int32)
    deg = np.diff(goff)[dst]
    cnt = deg if fanout < 0 else np.minimum(deg, fanout)
    loff = np.concatenate([[0], np.cumsum(cnt)]).astype(np.int32)
    if fanout >= 0:
        co = gpuinitco(n_dst, fanout, to_gpu(dst), to_gpu(goff)).cpu().numpy()
        assert np.array_equal(co, oracle.gpuinitco(n_dst, fanout, dst, goff))
        assert np.array_equal(np.cumsum(co), loff)
    got = sampleprocessing(fanout, to_gpu(dst), to_gpu(loff), to_gpu(goff), to_gpu(grow), seed=1234 + seed).cpu().numpy()
    want = oracle.sampleprocessing(fanout, dst, loff, goff, grow, seed=1234 + seed)
    assert np.array_equal(got, want)
    other = sampleprocessing(fanout, to_gpu(dst), to_gpu(loff), to_gpu(goff), to_gpu(grow), seed=99).cpu().numpy()
    if fanout >= 0 and (deg > fanout).sum() > 5:
        assert not np.array_equal(other, got)            # another seed, another sample
    # without a seed the draw follows torch's seed: the same after manual_seed, and it moves on per call
    import sys
    sp_mod = sys.modules["jittorgeometric_amd.ops.sampleprocessing"]   # the package attribute is the function
    torch.manual_seed(7)
    sp_mod._calls = 0
    a = sampleprocessing(fanout, to_gpu(dst), to_gpu(loff), to_gpu(goff), to_gpu(grow)).cpu().numpy()
    torch.manual_seed(7)
    sp_mod._calls = 0
    b = sampleprocessing(fanout, to_gpu(dst), to_gpu(loff), to_gpu(goff), to_gpu(grow)).cpu().numpy()
    assert np.array_equal(a, b)


@pytest.mark.parametrize("V,E,seed", [(40, 300, 0), (3000, 50000, 1), (20000, 30000, 2)])
def test_getweight_full_graph(V, E, seed):
    from jittorgeometric_amd.ops import getweight
    rng = np.random.default_rng(seed)
    goff, grow = global_csc(rng, V, E, hubs=1)
    ids = np.arange(V, dtype=np.int32)
    got = getweight(V, to_gpu(ids), to_gpu(ids), to_gpu(goff), to_gpu(grow)).cpu().numpy()
    indeg = np.diff(goff).astype(np.float32)
    outdeg = np.bincount(grow, minlength=V).astype(np.float32)
    col = np.repeat(ids, np.diff(goff))
    want = np.float32(1) / (np.sqrt(outdeg[grow]) * np.sqrt(indeg[col]))        # the oracle's arithmetic, vectorised
    if V <= 3000:
        assert np.array_equal(want, oracle.getweight(V, ids, ids, goff, grow))
    assert np.array_equal(got.view(np.int32), want.view(np.int32))


def test_getweight_layer_with_global_ids():
    from jittorgeometric_amd.ops import getweight
    off = np.array([0, 2, 3, 6], np.int32)
    row = np.array([7, 9, 7, 4, 9, 5], np.int32)
    dst = np.array([20, 21, 22], np.int32)
    got = getweight(30, to_gpu(dst), to_gpu(dst), to_gpu(off), to_gpu(row)).cpu().numpy()
    assert np.array_equal(got.view(np.int32), oracle.getweight(30, dst, dst, off, row).view(np.int32))


def test_getweight_repeated_destinations_and_ids_out_of_range():
    """A destination listed twice adds both of its columns to its in-degree (getweight_op.cc:56-57);
    an id outside [0, vtx_size), which the reference would use as an index out of bounds, is
    skipped wherever it would be one: its entries get weight 0, the other entries are as if the id
    were a valid one that nothing else names."""
    from jittorgeometric_amd.ops import getweight
    off = np.array([0, 3, 5, 9], np.int32)
    row = np.array([1, 2, 3, 1, 4, 2, 2, 5, 1], np.int32)
    dst = np.array([6, 7, 6], np.int32)
    got = getweight(8, to_gpu(dst), to_gpu(dst), to_gpu(off), to_gpu(row)).cpu().numpy()
    assert np.array_equal(got.view(np.int32), oracle.getweight(8, dst, dst, off, row).view(np.int32))
    ins6 = np.float32(7)                                  # 3 + 4 entries
    assert got[0] == np.float32(1) / (np.sqrt(np.float32(3)) * np.sqrt(ins6))     # source 1 appears 3 times
    bad_row = row.copy()
    bad_row[4] = 100
    bad_dst = np.array([6, -1, 6], np.int32)
    got = getweight(8, to_gpu(bad_dst), to_gpu(bad_dst), to_gpu(off), to_gpu(bad_row)).cpu().numpy()
    assert got[3] == 0 and got[4] == 0                    # column of destination -1; row index 100
    keep = np.array([0, 1, 2, 5, 6, 7, 8])
    stand_in = bad_row.copy()
    stand_in[4] = 0                                       # ids 0 and 7 appear nowhere else
    want = oracle.getweight(8, np.array([6, 7, 6], np.int32), None, off, stand_in)
    assert np.array_equal(got[keep].view(np.int32), want[keep].view(np.int32))


def test_getweight_at_the_size_of_the_benchmark_graph():
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import getweight
    ei, V = synthetic.make("powerlaw_1m")
    row, off, _ = oracle.cootocsc(np.ascontiguousarray(ei.astype(np.int32)), np.ones(ei.shape[1], np.float32), V)
    ids = np.arange(V, dtype=np.int32)
    got = getweight(V, to_gpu(ids), to_gpu(ids), to_gpu(off), to_gpu(row)).cpu().numpy()
    indeg = np.diff(off).astype(np.float32)
    outdeg = np.bincount(row, minlength=V).astype(np.float32)
    want = np.float32(1) / (np.sqrt(outdeg[row]) * np.sqrt(indeg[np.repeat(ids, np.diff(off))]))
    assert np.array_equal(got.view(np.int32), want.view(np.int32))


def test_gpuinitco_edge_cases():
    from jittorgeometric_amd.ops import gpuinitco
    goff = np.array([0, 0, 4, 4, 9, 10], np.int32)
    dst = np.array([3, 0, 1, 4, 3, 2], np.int32)
    for fanout in (0, 1, 3, 5, 100):
        for n in (0, 1, 6):
            got = gpuinitco(n, fanout, to_gpu(dst), to_gpu(goff)).cpu().numpy()
            assert np.array_equal(got, oracle.gpuinitco(n, fanout, dst[:n], goff)), (fanout, n)
    from jittorgeometric_amd import JgamdError
    with pytest.raises(JgamdError):
        gpuinitco(7, 3, to_gpu(dst), to_gpu(goff))


def test_csctocsr_layer_and_full_graph():
    from jittorgeometric_amd.ops import csctocsr
    g = GOLD["csctocsr_readme_v4"]
    ids = torch.arange(4, dtype=torch.int32, device=dev())
    r_o, c_i = csctocsr(torch.tensor(g["column_offset"], device=dev()), torch.tensor(g["row_indices"], device=dev()), ids, ids)
    assert r_o.tolist() == g["row_offset"] and c_i.tolist() == g["column_indices"]
    off = np.array([0, 2, 3, 6], np.int32); row = np.array([7, 9, 7, 4, 9, 5], np.int32)
    dst = np.array([20, 21, 22], np.int32); src = np.array([9, 7, 5], np.int32)
    r_o, c_i = csctocsr(to_gpu(off), to_gpu(row), to_gpu(dst), to_gpu(src))
    wr, wc = oracle.csctocsr(off, row, dst, src)
    assert np.array_equal(r_o.cpu().numpy(), wr) and np.array_equal(c_i.cpu().numpy(), wc)
    rng = np.random.default_rng(9)
    V = 1500
    goff, grow = global_csc(rng, V, 20000, hubs=2)
    idsn = np.arange(V, dtype=np.int32)
    r_o, c_i = csctocsr(to_gpu(goff), to_gpu(grow), to_gpu(idsn), to_gpu(idsn))
    wr, wc = oracle.csctocsr(goff, grow, idsn, idsn)
    assert np.array_equal(r_o.cpu().numpy(), wr) and np.array_equal(c_i.cpu().numpy(), wc)


def test_two_layer_sampled_subgraph_end_to_end():
    """The steps of the reference's sample_one (examples/minibatch_example.py:232-278) for one
    layer: counts -> offsets -> sampled row indices -> CSR of the layer -> weights."""
    from jittorgeometric_amd.ops import csctocsr, getweight, gpuinitco, sampleprocessing
    rng = np.random.default_rng(12)
    V = 4000
    goff, grow = global_csc(rng, V, 80000, hubs=3)
    dst = rng.permutation(V)[:512].astype(np.int32)
    co = gpuinitco(512, 10, to_gpu(dst), to_gpu(goff))
    loff = torch.cumsum(co, 0).to(torch.int32)
    rows = sampleprocessing(10, to_gpu(dst), loff, to_gpu(goff), to_gpu(grow), seed=3)
    src = torch.unique(rows)
    r_o, c_i = csctocsr(loff, rows, to_gpu(dst), src.to(torch.int32))
    wr, wc = oracle.csctocsr(loff.cpu().numpy(), rows.cpu().numpy(), dst, src.cpu().numpy())
    assert np.array_equal(r_o.cpu().numpy(), wr) and np.array_equal(c_i.cpu().numpy(), wc)
    w = getweight(V, to_gpu(dst), src.to(torch.int32), loff, rows).cpu().numpy()
    want = oracle.getweight(V, dst, src.cpu().numpy(), loff.cpu().numpy(), rows.cpu().numpy())
    assert np.array_equal(w.view(np.int32), want.view(np.int32))


def test_from_nodes_and_to_nodes():
    from jittorgeometric_amd.ops import cootocsc, cootocsr, from_nodes, to_nodes
    rng = np.random.default_rng(21)
    V = 3000
    ei, w = rand_graph(rng, V, 40000, 2)
    csc, csr = cootocsc(to_gpu(ei), to_gpu(w), V), cootocsr(to_gpu(ei), to_gpu(w), V)
    row, coff, _ = oracle.cootocsc(ei, w, V)
    col, roff, _ = oracle.cootocsr(ei, w, V)
    nodes = np.concatenate([rng.integers(0, V, 500), [0, 0, V - 1]]).astype(np.int32)     # hubs, repeats, last node
    assert np.array_equal(from_nodes(csc, to_gpu(nodes)).cpu().numpy(), oracle.from_nodes(coff, row, nodes))
    assert np.array_equal(to_nodes(csr, to_gpu(nodes)).cpu().numpy(), oracle.from_nodes(roff, col, nodes))
    assert from_nodes(csc, to_gpu(np.zeros(0, np.int32))).numel() == 0
    many = rng.integers(0, V, 70000).astype(np.int32)                                    # more than one scan tile
    assert np.array_equal(from_nodes(csc, to_gpu(many)).cpu().numpy(), oracle.from_nodes(coff, row, many))
    with pytest.raises(ValueError):
        from_nodes(None, to_gpu(nodes))


def test_reference_test_inputs():
    """The literal tensors of the reference's own tests of these operators
    (tests/test_getweight.py, test_gpuinitco.py, test_fromtonodes.py, test_edgetovertex.py,
    test_scatter_to_edge.py) with the expected values the committed fixture file holds."""
    from jittorgeometric_amd.data import CSC, CSR
    from jittorgeometric_amd.ops import ScatterToEdge, ScatterToVertex, from_nodes, getweight, gpuinitco, to_nodes
    i32 = lambda a: to_gpu(np.asarray(a, np.int32))
    g = GOLD["getweight_v4"]
    w = getweight(g["vtx_size"], i32(g["dst"]), i32(g["src"]), i32(g["column_offset"]), i32(g["row_indices"]))
    np.testing.assert_allclose(w.cpu().numpy(), g["edge_weight"], rtol=2e-7)
    g = GOLD["gpuinitco_v4"]
    out = gpuinitco(g["dst_size"], g["fanout"], i32(g["csc_layer_dst"]), i32(g["csc_global_column_offset"]))
    assert out.cpu().tolist() == g["out"]
    g = GOLD["fromtonodes_v5"]
    csc = CSC(i32(g["row_indices"]), i32(g["column_offset"]), None)
    csr = CSR(i32(g["column_indices"]), i32(g["row_offset"]), None)
    assert from_nodes(csc, i32(g["nodes"])).cpu().tolist() == g["from_nodes"]
    assert to_nodes(csr, i32(g["nodes"])).cpu().tolist() == g["to_nodes"]
    g = GOLD["edgetovertex_v3"]
    csc = CSC(i32(g["row_indices"]), i32(g["column_offset"]), to_gpu(np.ones(4, np.float32)))
    assert ScatterToVertex(to_gpu(np.array(g["x"], np.float32)), csc, "src").cpu().tolist() == g["out"]
    g = GOLD["scatter_to_edge_v3"]
    x = to_gpu(np.array(g["x"], np.float32))
    assert ScatterToEdge(x, csc, "dst").cpu().tolist() == g["out_dst"]
    assert ScatterToEdge(x, csc, "src").cpu().tolist() == g["out_src"]
