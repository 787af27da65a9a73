"""COO -> CSR/CSC on the GPU against the CPU oracle: bit-exact, through the
C ABI (jittorgeometric_amd.ops -> ctypes -> libjgamd.so)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def run_both(ei, w, V):
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    csr = cootocsr(to_gpu(ei), to_gpu(w), V)
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    torch.cuda.synchronize()
    return csr, csc


def check_exact(ei, w, V):
    csr, csc = run_both(ei, w, V)
    col, roff, rw = oracle.cootocsr(ei, w, V)
    row, coff, cw = oracle.cootocsc(ei, w, V)
    assert np.array_equal(csr.row_offset.cpu().numpy(), roff)
    assert np.array_equal(csr.column_indices.cpu().numpy(), col)
    assert np.array_equal(csr.edge_weight.cpu().numpy().view(np.int32), rw.view(np.int32))
    assert np.array_equal(csc.column_offset.cpu().numpy(), coff)
    assert np.array_equal(csc.row_indices.cpu().numpy(), row)
    assert np.array_equal(csc.edge_weight.cpu().numpy().view(np.int32), cw.view(np.int32))
    assert csr.column_indices.dtype == torch.int32 and csr.edge_weight.dtype == torch.float32


@pytest.mark.parametrize("name", ["csr_v4", "mp_spmm_v10"])
def test_reference_fixtures(name):
    g = GOLD[name]
    ei = np.array(g["edge_index"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    csr, csc = run_both(ei, w, g["v_num"])
    assert csr.column_indices.tolist() == g["csr"]["column_indices"]
    assert csr.row_offset.tolist() == g["csr"]["row_offset"]
    assert csr.edge_weight.tolist() == g["csr"]["edge_weight"]
    assert csc.row_indices.tolist() == g["csc"]["row_indices"]
    assert csc.column_offset.tolist() == g["csc"]["column_offset"]
    assert csc.edge_weight.tolist() == g["csc"]["edge_weight"]


@pytest.mark.parametrize("V,E,hubs,seed", [
    (1, 0, 0, 0), (1, 9, 0, 1), (5, 0, 0, 2), (4, 100, 0, 3), (1000, 1, 0, 4),
    (1024, 20000, 3, 5), (1025, 20000, 3, 6), (2708, 13264, 0, 7), (5000, 8191, 2, 8),
    (5000, 8192, 2, 9), (5000, 8193, 2, 10), (70001, 300000, 5, 11), (300000, 1000000, 4, 12),
    (4194304, 600000, 3, 13), (2100000, 2500000, 2, 14),
    (4194305, 700000, 3, 15), (9000000, 3000000, 2, 16), (70000000, 100000, 1, 17),
])
def test_random_graphs_bit_exact(V, E, hubs, seed):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs)
    check_exact(ei, w, V)


def test_all_edges_one_row_and_sorted_and_reversed_inputs():
    rng = np.random.default_rng(20)
    V, E = 3000, 50000
    ei, w = rand_graph(rng, V, E)
    one = ei.copy()
    one[0, :] = 17                              # a single 50,000-edge row
    check_exact(one, w, V)
    order = np.argsort(ei[0], kind="stable")
    check_exact(ei[:, order], w[order], V)      # already sorted by source
    check_exact(ei[:, order[::-1]].copy(), w[order[::-1]].copy(), V)


def test_endpoints_of_any_size_come_through_unchanged():
    """The endpoint that is not the key is copied, never interpreted: negative values and values
    far above V (which do not fit the packed form the records take between the two passes, and
    are looked up again from the input) must arrive bit for bit, among ordinary ones."""
    rng = np.random.default_rng(77)
    for V in (700, 5000, 300_000, 2_000_000):
        E = 200_000
        ei, w = rand_graph(rng, V, E, hubs=2)
        odd = rng.random(E) < 0.3
        ei[1, odd] = rng.choice(np.array([-1, -2, -2 ** 31, 2 ** 31 - 1, 2 ** 30, 2 ** 22, 2 ** 21, 2 ** 21 - 1, V, V + 1],
                                         np.int64), odd.sum()).astype(np.int32)
        from jittorgeometric_amd.ops import cootocsr
        csr = cootocsr(to_gpu(ei), to_gpu(w), V)          # keyed on row 0: the odd values are the other endpoint
        col, roff, rw = oracle.cootocsr(ei, w, V)
        assert np.array_equal(csr.row_offset.cpu().numpy(), roff)
        assert np.array_equal(csr.column_indices.cpu().numpy(), col)
        assert np.array_equal(csr.edge_weight.cpu().numpy().view(np.int32), rw.view(np.int32))


def test_weights_are_copied_bitwise_including_nan_inf_and_negative_zero():
    rng = np.random.default_rng(21)
    V, E = 500, 4000
    ei, w = rand_graph(rng, V, E)
    w[:8] = [np.nan, np.inf, -np.inf, -0.0, 0.0, 1e-45, -1e38, 3.0]
    check_exact(ei, w, V)


def test_deterministic_across_runs():
    rng = np.random.default_rng(22)
    V, E = 20000, 400000
    ei, w = rand_graph(rng, V, E, hubs=3)
    a, _ = run_both(ei, w, V)
    b, _ = run_both(ei, w, V)
    assert torch.equal(a.column_indices, b.column_indices) and torch.equal(a.edge_weight, b.edge_weight)


def test_permutation_output_and_transpose():
    from jittorgeometric_amd.ops.cootocsr import _convert
    from jittorgeometric_amd.ops._common import transposed
    from jittorgeometric_amd import CSR
    rng = np.random.default_rng(23)
    V, E = 9000, 120000
    ei, w = rand_graph(rng, V, E, hubs=2)
    idx, off, wo, perm = _convert(to_gpu(ei), to_gpu(w), V, 0, with_perm=True)
    perm = perm.cpu().numpy()
    want = np.argsort(ei[0], kind="stable")
    assert np.array_equal(perm, want)
    assert np.array_equal(idx.cpu().numpy(), ei[1][want])
    # transpose of the CSR equals the CSC of the CSR-ordered edge list
    holder = CSR(idx, off, wo)
    off_t, idx_t, w_t, perm_t = transposed(holder, off, idx, wo, V, V)
    src_sorted = ei[0][want]
    dst_sorted = ei[1][want]
    row, coff, cw = oracle.cootocsc(np.stack([src_sorted, dst_sorted]), w[want], V)
    assert np.array_equal(off_t.cpu().numpy(), coff)
    assert np.array_equal(idx_t.cpu().numpy(), row)
    assert np.array_equal(w_t.cpu().numpy(), cw)
    assert np.array_equal(perm_t.cpu().numpy(), np.argsort(dst_sorted, kind="stable"))
    # the inverse map (original slot -> transposed slot), cached beside the transpose
    from jittorgeometric_amd.ops._common import transposed_inverse
    inv = transposed_inverse(holder, perm_t)
    assert transposed_inverse(holder, perm_t) is inv
    want_inv = np.empty(E, np.int32)
    want_inv[perm_t.cpu().numpy()] = np.arange(E, dtype=np.int32)
    assert np.array_equal(inv.cpu().numpy(), want_inv)


def test_int64_edge_index_is_narrowed_like_the_reference_data_class():
    from jittorgeometric_amd.ops import cootocsr
    g = GOLD["csr_v4"]
    ei = torch.tensor(g["edge_index"], dtype=torch.int64, device=dev())
    w = torch.tensor(g["edge_weight"], dtype=torch.float32, device=dev())
    csr = cootocsr(ei, w, 4)
    assert csr.column_indices.tolist() == g["csr"]["column_indices"]


def test_cpu_tensors_are_refused():
    from jittorgeometric_amd import _lib
    from jittorgeometric_amd.ops import cootocsr
    with pytest.raises(_lib.JgamdError):
        cootocsr(torch.zeros((2, 3), dtype=torch.int32), torch.zeros(3), 4)


def test_powerlaw_1m_full_size_bit_exact():
    """Benchmark configuration: 1M nodes, 16M power-law edges + self-loops,
    gcn_norm weights, edge order as generated (random)."""
    from jittorgeometric_amd import synthetic
    ei, V = synthetic.make("powerlaw_1m")
    ei, w = oracle.gcn_norm(ei, None, V)
    check_exact(ei.astype(np.int32), w, V)


def test_dense_233k_full_size_bit_exact():
    """Benchmark configuration 4: 232,965 nodes, ~115M lognormal-degree edges +
    self-loops (source-sorted input, so the CSR side is a pure copy and the CSC
    side a full sort)."""
    from jittorgeometric_amd import synthetic
    ei, V = synthetic.make("dense_233k")
    ei, w = oracle.gcn_norm(ei, None, V)
    check_exact(ei.astype(np.int32), w, V)


def test_one_hub_with_millions_of_edges_bit_exact():
    """A single key owning 3M of 8M edges: its bucket is cut into many
    sub-blocks (the uncapped power-law configuration has such a hub)."""
    rng = np.random.default_rng(77)
    V, E = 600000, 8000000
    ei, w = rand_graph(rng, V, E)
    ei[0, rng.random(E) < 0.38] = 31337
    ei[1, rng.random(E) < 0.38] = 4242
    check_exact(ei, w, V)


@pytest.mark.parametrize("norm", ["gcn", "sage"])
def test_conversion_after_a_normalisation_reuses_its_sort_and_stays_bit_exact(norm):
    """gcn_norm / sage_norm sort the edge list by destination to sum the degrees; the cootocsc the
    caller runs next on the same edges (examples/gcn_example.py:48-59) takes that order instead of
    sorting again.  Result: the oracle's arrays bit for bit, whichever way it was produced."""
    from jittorgeometric_amd.nn import gcn_norm, sage_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    rng = np.random.default_rng(31)
    V, E = 5000, 90000
    ei, _ = rand_graph(rng, V, E, 2)
    ei_g, w_g = (gcn_norm if norm == "gcn" else sage_norm)(to_gpu(ei), None, V)
    assert getattr(w_g, "_jgamd_order", None) is not None
    ei_h, w_h = ei_g.cpu().numpy(), w_g.cpu().numpy()
    want_c, want_r = oracle.cootocsc(ei_h, w_h, V), oracle.cootocsr(ei_h, w_h, V)

    def same(holder, names, want):
        for n, a in zip(names, want):
            got = getattr(holder, n).cpu().numpy()
            assert np.array_equal(got.view(np.int32), a.view(np.int32)), n
    csc = cootocsc(ei_g, w_g, V)                      # takes the remembered order
    assert getattr(w_g, "_jgamd_order", None) is None      # handed out once
    same(csc, ("row_indices", "column_offset", "edge_weight"), want_c)
    same(cootocsc(ei_g, w_g, V), ("row_indices", "column_offset", "edge_weight"), want_c)     # sorts
    same(cootocsr(ei_g, w_g, V), ("column_indices", "row_offset", "edge_weight"), want_r)

    # weights written in place after the normalisation, or another node count: the order is not used
    ei2, w2 = (gcn_norm if norm == "gcn" else sage_norm)(to_gpu(ei), None, V)
    w2.mul_(2.0)
    same(cootocsc(ei2, w2, V), ("row_indices", "column_offset", "edge_weight"),
         oracle.cootocsc(ei2.cpu().numpy(), w2.cpu().numpy(), V))
    ei3, w3 = (gcn_norm if norm == "gcn" else sage_norm)(to_gpu(ei), None, V)
    same(cootocsc(ei3, w3, V + 7), ("row_indices", "column_offset", "edge_weight"),
         oracle.cootocsc(ei3.cpu().numpy(), w3.cpu().numpy(), V + 7))


@pytest.mark.parametrize("V,E,extra,hubs", [(300, 5000, 40, 1), (4000, 90000, 0, 2), (1, 3000, 0, 0), (70000, 9000, 0, 0)])
def test_weights_scaled_in_compressed_order_equal_the_conversion_of_scaled_weights(V, E, extra, hubs):
    """jgamd_scale_csx_weights on the arrays of one conversion = the conversion of
    jgamd_scale_edge_weights's result, bit for bit, slots of dropped edges (keys outside [0, V))
    included; either factor array may be missing."""
    from jittorgeometric_amd import _lib
    from jittorgeometric_amd.ops.cootocsr import _convert
    lib = _lib.load()
    rng = np.random.default_rng(32 + V)
    ei, w = rand_graph(rng, V + extra, E, hubs)          # with extra > 0 some destinations are outside [0, V)
    ei_g, w_g = to_gpu(ei), to_gpu(w)
    N = V + extra
    a = to_gpu(rng.standard_normal(N).astype(np.float32))
    b = to_gpu(rng.standard_normal(N).astype(np.float32))
    idx, off, ws, _ = _convert(ei_g, w_g, V, 1)
    for fa, fb in ((a, b), (None, b), (a, None)):
        coo = torch.empty(E, device=dev())
        _lib.check(lib.jgamd_scale_edge_weights(_lib.ptr(ei_g), _lib.ptr(w_g), _lib.ptr(fa), _lib.ptr(fb), E, N,
                                                _lib.ptr(coo), _lib.stream_ptr(dev())))
        want = _convert(ei_g, coo, V, 1)[2]
        got = torch.full((E,), 7.0, device=dev())
        nbytes = _lib.query(lib.jgamd_scale_csx_weights_workspace, E)
        wsp = _lib.workspace(nbytes, dev())
        _lib.check(lib.jgamd_scale_csx_weights(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(ws), _lib.ptr(fa), _lib.ptr(fb), V, E,
                                               N, _lib.ptr(got), _lib.ptr(wsp), nbytes, _lib.stream_ptr(dev())))
        assert np.array_equal(got.cpu().numpy().view(np.int32), want.cpu().numpy().view(np.int32))
    # and the COO form against numpy
    ref = a.cpu().numpy()[ei[0]] * w * b.cpu().numpy()[ei[1]]
    coo = torch.empty(E, device=dev())
    _lib.check(lib.jgamd_scale_edge_weights(_lib.ptr(ei_g), _lib.ptr(w_g), _lib.ptr(a), _lib.ptr(b), E, N, _lib.ptr(coo),
                                            _lib.stream_ptr(dev())))
    assert np.array_equal(coo.cpu().numpy(), (a.cpu().numpy()[ei[0]] * w) * b.cpu().numpy()[ei[1]]) or \
        np.allclose(coo.cpu().numpy(), ref, rtol=1e-6)
