"""Weighted CSR/CSC SpMM on the GPU against the CPU oracle (fp32, 1e-5
relative / 1e-6 absolute, relative to the sum of absolute terms of each
output element since the summation order differs)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def gpu_csx(ei, w, V):
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    return cootocsc(to_gpu(ei), to_gpu(w), V), cootocsr(to_gpu(ei), to_gpu(w), V)


def abs_scale(x, idx, off, w):
    """sum_j |w_j| |x[idx_j]| per output element: the size the rounding error scales with."""
    return oracle.aggregate(np.abs(x), idx, off, np.abs(w)).astype(np.float64)


def check_fwd_bwd(ei, w, V, F, seed=0):
    from jittorgeometric_amd.ops import aggregateWithWeight
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    csc, csr = gpu_csx(ei, w, V)
    xt = to_gpu(x).requires_grad_(True)
    out = aggregateWithWeight(xt, csc, csr)
    out.backward(to_gpu(g))
    torch.cuda.synchronize()
    ocsc = oracle.cootocsc(ei, w, V)
    ocsr = oracle.cootocsr(ei, w, V)
    want = oracle.aggregate_with_weight(x, ocsc)
    wantg = oracle.aggregate_with_weight_grad(g, ocsr)
    assert_close(out.detach().cpu().numpy(), want, abs_scale(x, *ocsc), what="forward F=%d" % F)
    assert_close(xt.grad.cpu().numpy(), wantg, abs_scale(g, *ocsr), what="backward F=%d" % F)
    return out


def test_reference_fixture_integer_exact():
    from jittorgeometric_amd.ops import SpmmCsr, aggregateWithWeight
    g = GOLD["mp_spmm_v10"]
    ei = np.array(g["edge_index"], np.int32)
    w = np.array(g["edge_weight"], np.float32)
    x = np.array(g["x"], np.float32)
    csc, csr = gpu_csx(ei, w, 10)
    out = aggregateWithWeight(to_gpu(x), csc, csr).cpu().numpy()
    for r, vals in g["aggregate_rows"].items():
        assert out[int(r)].tolist() == [float(v) for v in vals]
    assert np.array_equal(out, oracle.aggregate_with_weight(x, oracle.cootocsc(ei, w, 10)))
    # SpmmCsr(x, csr) with its default trans_A=True is the same quantity (tests/test_mp_spmm.py:28-31)
    assert np.array_equal(SpmmCsr(to_gpu(x), csr).cpu().numpy(), out)


def test_spmmcsr_fixture_with_int64_indices():
    from jittorgeometric_amd import CSR
    from jittorgeometric_amd.ops import SpmmCsr
    g = GOLD["spmmcsr_v3"]
    csr = CSR(torch.tensor(g["column_indices"], dtype=torch.int64, device=dev()),
              torch.tensor(g["row_offset"], dtype=torch.int64, device=dev()),
              torch.tensor(g["edge_weight"], dtype=torch.float32, device=dev()))
    x = torch.tensor(g["x"], dtype=torch.float32, device=dev())
    assert SpmmCsr(x, csr).tolist() == g["out_trans_A"]
    assert SpmmCsr(x, csr, trans_A=False).tolist() == g["out_no_trans"]


@pytest.mark.parametrize("F", [1, 2, 3, 7, 8, 31, 32, 33, 41, 47, 64, 65, 100, 128, 130, 192, 256, 300, 320, 512, 602, 1024, 1030])
def test_feature_widths(F):
    rng = np.random.default_rng(100 + F)
    V, E = 700, 9000
    ei, w = rand_graph(rng, V, E, hubs=2)
    check_fwd_bwd(ei, w, V, F, seed=F)


@pytest.mark.parametrize("V,E,hubs,F,seed", [
    (1, 0, 0, 4, 0), (1, 50, 0, 128, 1), (3, 0, 0, 64, 2), (50, 7, 0, 128, 3),
    (4000, 200000, 2, 128, 4), (4000, 200000, 2, 32, 5), (100000, 50000, 0, 16, 6),
    (30000, 600000, 4, 64, 7), (20000, 300000, 1, 256, 8),
    # rows of 1-8 floats take the tile kernels: mostly empty rows (more rows than entries in a tile),
    # hubs that cross many tiles, entry counts around the tile sizes
    (200000, 5000, 0, 1, 9), (300000, 3000, 2, 8, 10), (4000, 200000, 2, 1, 11), (4000, 200000, 2, 4, 12),
    (500, 2048, 0, 2, 13), (500, 2049, 1, 8, 14), (3, 70000, 0, 1, 15), (1, 30000, 0, 8, 16),
])
def test_shapes_empty_rows_and_hubs(V, E, hubs, F, seed):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs, hub_share=0.5)
    check_fwd_bwd(ei, w, V, F, seed=seed)


def test_single_hub_row_spanning_many_wavefronts():
    rng = np.random.default_rng(40)
    V, E, F = 2000, 150000, 128
    ei, w = rand_graph(rng, V, E)
    ei[1, :140000] = 1234                     # one 140,000-entry destination
    check_fwd_bwd(ei, w, V, F)


def test_run_to_run_reproducible():
    from jittorgeometric_amd.ops import aggregateWithWeight
    rng = np.random.default_rng(41)
    V, E, F = 20000, 500000, 128
    ei, w = rand_graph(rng, V, E, hubs=3, hub_share=0.4)
    csc, csr = gpu_csx(ei, w, V)
    x = to_gpu(rng.standard_normal((V, F)).astype(np.float32))
    a = aggregateWithWeight(x, csc, csr)
    b = aggregateWithWeight(x, csc, csr)
    assert torch.equal(a, b)


def test_transpose_identity_at_full_size_and_oracle_on_a_row_sample():
    """Config 2 at full size: <A x, g> = <x, A^T g> ties forward (CSC) to
    backward (CSR); a sample of rows, hubs included, is checked against the oracle's
    sequential sums."""
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import aggregateWithWeight
    ei, V = synthetic.make("powerlaw_1m")
    ei, w = oracle.gcn_norm(ei, None, V)
    ei = ei.astype(np.int32)
    F = 128
    rng = np.random.default_rng(42)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    csc, csr = gpu_csx(ei, w, V)
    xt = to_gpu(x).requires_grad_(True)
    out = aggregateWithWeight(xt, csc, csr)
    out.backward(to_gpu(g))
    lhs = (out.detach().double() * to_gpu(g).double()).sum().item()
    rhs = (xt.grad.double() * to_gpu(x).double()).sum().item()
    assert abs(lhs - rhs) <= 1e-6 * (out.detach().abs().double() * to_gpu(g).abs().double()).sum().item()
    ocsc = oracle.cootocsc(ei, w, V)
    want = oracle.aggregate_with_weight(x, ocsc)
    assert_close(out.detach().cpu().numpy(), want, abs_scale(x, *ocsc), what="config 2 forward")


def test_hub_row_with_millions_of_entries_uses_grouped_piece_sums():
    """One destination with 2.5M in-edges: its row is cut into ~10^4 pieces
    whose sums are grouped before the final add."""
    rng = np.random.default_rng(78)
    V, E, F = 50000, 3000000, 32
    ei, w = rand_graph(rng, V, E)
    ei[1, :2500000] = 777
    ei[0, 2500000:2900000] = 5            # and a 400k-entry row for the backward direction
    check_fwd_bwd(ei, w, V, F)


def test_dense_233k_full_size_odd_width():
    """Benchmark configuration 4 at F=41 (rows of x are not line-aligned): forward over
    the CSC arrays against the oracle's sequential sums, backward through the
    transpose identity."""
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import aggregateWithWeight
    ei, V = synthetic.make("dense_233k")
    ei, w = oracle.gcn_norm(ei, None, V)
    ei = ei.astype(np.int32)
    F = 41
    rng = np.random.default_rng(44)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    csc, csr = gpu_csx(ei, w, V)
    xt = to_gpu(x).requires_grad_(True)
    out = aggregateWithWeight(xt, csc, csr)
    out.backward(to_gpu(g))
    ocsc = oracle.cootocsc(ei, w, V)
    want = oracle.aggregate_with_weight(x, ocsc)
    assert_close(out.detach().cpu().numpy(), want, abs_scale(x, *ocsc), what="config 4 forward F=41")
    lhs = (out.detach().double() * to_gpu(g).double()).sum().item()
    rhs = (xt.grad.double() * to_gpu(x).double()).sum().item()
    assert abs(lhs - rhs) <= 1e-6 * (out.detach().abs().double() * to_gpu(g).abs().double()).sum().item()


def test_wide_rows_take_the_64_bit_address_path():
    """x larger than 4 GiB: gathered rows are addressed with 64-bit arithmetic."""
    from jittorgeometric_amd.ops._common import spmm
    rng = np.random.default_rng(45)
    C, F, R, E = 4_300_000, 256, 3000, 40000          # C*F*4 = 4.4e9 bytes
    x = torch.empty((C, F), dtype=torch.float32, device=dev())
    x.normal_()
    src = np.concatenate([rng.integers(0, C, E - 8), np.arange(C - 8, C)]).astype(np.int32)   # reach the last rows
    dst = rng.integers(0, R, E).astype(np.int32)
    w = rng.standard_normal(E).astype(np.float32)
    row, off, cw = oracle.cootocsc(np.stack([src, dst]), w, R)
    out = spmm(to_gpu(off), to_gpu(row), to_gpu(cw), x, R).cpu().numpy()
    xs = x[torch.from_numpy(row.astype(np.int64)).to(dev())].cpu().numpy().astype(np.float64)   # [E,F] gathered rows
    want = np.zeros((R, F))
    seg = np.repeat(np.arange(R), np.diff(off))
    np.add.at(want, seg, xs * cw[:, None].astype(np.float64))
    scale = np.zeros((R, F))
    np.add.at(scale, seg, np.abs(xs) * np.abs(cw[:, None]))
    assert_close(out, want, scale, what="wide x")
