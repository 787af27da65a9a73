"""CSC / CSR holders that were not produced by the library: int64 indices and
float64 weights (what torch.tensor([...]) gives, and what the reference's own
test scripts build by hand), non-contiguous inputs, arrays written in place,
and arrays whose offsets stop short of the entries (keys dropped by the
conversion).  Every operator must give the oracle's answer on them."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def _graph(seed, V=500, E=6000, hubs=2):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs)
    return rng, ei, w, oracle.cootocsc(ei, w, V), oracle.cootocsr(ei, w, V)


def _wide_holders(ocsc, ocsr):
    """The same arrays as int64 / float64 tensors."""
    from jittorgeometric_amd import CSC, CSR
    t64 = lambda a: torch.from_numpy(np.asarray(a).astype(np.int64)).to(dev())
    f64 = lambda a: torch.from_numpy(np.asarray(a).astype(np.float64)).to(dev())
    return (CSC(t64(ocsc[0]), t64(ocsc[1]), f64(ocsc[2])), CSR(t64(ocsr[0]), t64(ocsr[1]), f64(ocsr[2])))


def _scale(x, idx, off, w):
    return oracle.aggregate(np.abs(x), idx, off, np.abs(w)).astype(np.float64)


def test_aggregate_with_int64_and_float64_holders():
    from jittorgeometric_amd.ops import aggregateWithWeight
    rng, ei, w, ocsc, ocsr = _graph(1)
    V, F = 500, 24
    csc, csr = _wide_holders(ocsc, ocsr)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    xt = to_gpu(x).requires_grad_(True)
    out = aggregateWithWeight(xt, csc, csr)
    out.backward(to_gpu(g))
    assert_close(out.detach().cpu().numpy(), oracle.aggregate_with_weight(x, ocsc), _scale(x, *ocsc), what="fwd")
    assert_close(xt.grad.cpu().numpy(), oracle.aggregate_with_weight_grad(g, ocsr), _scale(g, *ocsr), what="bwd")
    # an explicit weight tensor in float64 is narrowed the same way
    out2 = aggregateWithWeight(to_gpu(x), csc, csr, csc.edge_weight)
    assert torch.equal(out2, out.detach())


def test_edgesoftmax_and_scatter_ops_with_int64_holders():
    from jittorgeometric_amd.ops import EdgeSoftmax, ScatterToEdge, ScatterToVertex
    rng, ei, w, ocsc, ocsr = _graph(2)
    V, E, C = 500, 6000, 5
    csc, _ = _wide_holders(ocsc, ocsr)
    row, off, _ = ocsc
    x = rng.standard_normal(E).astype(np.float64)                 # float64 logits too
    xt = torch.from_numpy(x).to(dev()).requires_grad_(True)
    y = EdgeSoftmax(xt, csc)
    g = rng.standard_normal(E).astype(np.float32)
    y.backward(to_gpu(g))
    want = oracle.edgesoftmax(x.astype(np.float32), off)
    deg = np.diff(off)[np.repeat(np.arange(V), np.diff(off))].astype(np.float64)
    # against the oracle's own sequential fp32 denominator: good to about deg * 2^-24
    assert_close(y.detach().cpu().numpy(), want, want * (1 + deg * 6e-3), atol=1e-7, what="softmax")
    yh = y.detach().cpu().numpy()
    wantg = oracle.edgesoftmax_backward(g, yh, off)
    seg = np.repeat(np.arange(V), np.diff(off))
    dot_terms = np.zeros(V)
    np.add.at(dot_terms, seg, np.abs(yh.astype(np.float64) * g))
    assert_close(xt.grad.cpu().numpy(), wantg, np.abs(yh * g) + yh * dot_terms[seg], what="softmax grad")
    xv = rng.standard_normal((V, C)).astype(np.float32)
    for flow, flag in (("src", 0), ("dst", 1)):
        xg = to_gpu(xv).requires_grad_(True)
        e = ScatterToEdge(xg, csc, flow)
        assert np.array_equal(e.detach().cpu().numpy(), oracle.scattertoedge(xv, row, off, flag))
        ge = rng.standard_normal((E, C)).astype(np.float32)
        e.backward(to_gpu(ge))
        wantv = oracle.edgetovertex(ge, row, off, flag, V)
        assert_close(xg.grad.cpu().numpy(), wantv, oracle.edgetovertex(np.abs(ge), row, off, flag, V), what=flow)
    xe = rng.standard_normal((E, C)).astype(np.float32)
    v = ScatterToVertex(to_gpu(xe), csc, "src")
    assert_close(v.cpu().numpy(), oracle.edgetovertex(xe, row, off, 1, V),
                 oracle.edgetovertex(np.abs(xe), row, off, 1, V), what="scatter to vertex")


def test_spmmcsr_and_hops_with_int64_holders():
    from jittorgeometric_amd.ops import SpmmCsr, appnp_propagate
    rng, ei, w, ocsc, ocsr = _graph(3)
    V, F = 500, 16
    csc, csr = _wide_holders(ocsc, ocsr)
    x = rng.standard_normal((V, F)).astype(np.float32)
    out = SpmmCsr(to_gpu(x), csr)
    assert_close(out.cpu().numpy(), oracle.aggregate_with_weight(x, ocsc), _scale(x, *ocsc), what="SpmmCsr")
    got = appnp_propagate(to_gpu(x), csc, csr, 3, 0.1)
    want = oracle.appnp(x, ocsc, 3, 0.1)
    terms = oracle.appnp(np.abs(x), (ocsc[0], ocsc[1], np.abs(ocsc[2])), 3, 0.1)     # three hops, 1e-5 each
    assert_close(got.cpu().numpy(), want, terms, rtol=3e-5, what="appnp")


def test_gat_with_int64_holder_and_noncontiguous_float64_inputs():
    """h handed over as a transposed view in float64: forward and all three
    gradients against the fp64 model of the layer."""
    from test_gpu_gat import check_against_fp64, torch_reference
    from jittorgeometric_amd.ops import gat_aggregate
    rng, ei, w, ocsc, ocsr = _graph(4, V=400, E=5000)
    V, H, D = 400, 4, 8
    csc, _ = _wide_holders(ocsc, ocsr)
    row, off, _ = ocsc
    dst = np.repeat(np.arange(V), np.diff(off))
    h = rng.standard_normal((V, H, D))
    a_src, a_dst = rng.standard_normal((H, D)) / 4, rng.standard_normal((H, D)) / 4
    g = rng.standard_normal((V, H, D)).astype(np.float32)
    base = torch.from_numpy(np.ascontiguousarray(h.transpose(1, 0, 2))).to(dev()).requires_grad_(True)   # [H,V,D]
    ht = base.transpose(0, 1)                                    # [V,H,D] view, strides of [H,V,D]
    assert not ht.is_contiguous()
    a_s = torch.from_numpy(np.ascontiguousarray(a_src.T)).to(dev()).requires_grad_(True)                  # [D,H]
    a_d = torch.from_numpy(a_dst).to(dev()).requires_grad_(True)
    out = gat_aggregate(ht, csc, a_s.t(), a_d, 0.2)
    out.backward(to_gpu(g))
    h64, s64, d64 = (torch.from_numpy(t.astype(np.float32).astype(np.float64)).requires_grad_(True)
                     for t in (h, a_src, a_dst))
    ref, alpha = torch_reference(h64, s64, d64, torch.from_numpy(row.astype(np.int64)),
                                 torch.from_numpy(dst.astype(np.int64)), V)
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    assert base.grad.dtype == torch.float64 and base.grad.shape == base.shape
    check_against_fp64(None, out, base.grad.transpose(0, 1), a_s.grad.t(), a_d.grad, ref, alpha, h64, s64, d64, g, row,
                       dst, V)


def test_in_place_weight_update_reaches_the_cached_transpose():
    """SpmmCsr keeps the transposed arrays on the CSR object; writing the weights in
    place, or rebinding them, must not leave the product on the old ones."""
    from jittorgeometric_amd.ops import SpmmCsr, cootocsr
    rng, ei, w, ocsc, ocsr = _graph(5)
    V, F = 500, 8
    csr = cootocsr(to_gpu(ei), to_gpu(w), V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    first = SpmmCsr(to_gpu(x), csr)
    csr.edge_weight.mul_(2.0)
    second = SpmmCsr(to_gpu(x), csr)
    assert torch.equal(second, first * 2.0)
    csr.edge_weight = csr.edge_weight * 0.5
    third = SpmmCsr(to_gpu(x), csr)
    assert torch.equal(third, first)
    # the same for a holder whose arrays were converted (int64 -> int32 copies are kept on it)
    _, csr64 = _wide_holders(ocsc, ocsr)
    a = SpmmCsr(to_gpu(x), csr64)
    csr64.edge_weight.mul_(3.0)
    b = SpmmCsr(to_gpu(x), csr64)
    # (3w rounded to fp32) is not 3 * (w rounded to fp32): one rounding per term
    assert_close(b.cpu().numpy(), 3.0 * a.cpu().numpy(), 3.0 * _scale(x, *ocsc), what="converted holder")


def test_wrong_shapes_raise_instead_of_reading_out_of_bounds():
    from jittorgeometric_amd import CSC, JgamdError
    from jittorgeometric_amd.ops import EdgeSoftmax, aggregateWithWeight
    rng, ei, w, ocsc, ocsr = _graph(6)
    csc, csr = _wide_holders(ocsc, ocsr)
    x = to_gpu(rng.standard_normal((499, 4)).astype(np.float32))       # one row short of V
    with pytest.raises(JgamdError):
        aggregateWithWeight(x, csc, csr)
    bad = CSC(csc.row_indices, csc.column_offset, csc.edge_weight[:-1])
    with pytest.raises(JgamdError):
        aggregateWithWeight(to_gpu(rng.standard_normal((500, 4)).astype(np.float32)), bad, csr)
    with pytest.raises(JgamdError):
        EdgeSoftmax(torch.zeros(6000, 2, 2, device=dev()), csc)
    with pytest.raises(JgamdError):
        aggregateWithWeight(torch.zeros(500, 4), csc, csr)             # CPU tensor


def test_keys_out_of_range_are_dropped_and_the_rest_still_works():
    """Edges whose destination lies outside [0, V) are dropped by the conversion, so the
    offsets end below the length of the index arrays: the tail of the arrays is zero, and
    the degree sum (one float per entry), EdgeSoftmax and the wide product only see the
    entries the offsets cover."""
    from jittorgeometric_amd.ops import EdgeSoftmax, aggregateWithWeight, cootocsc, cootocsr
    from jittorgeometric_amd.ops._common import spmm
    rng = np.random.default_rng(7)
    V, E = 300, 9000
    ei, w = rand_graph(rng, V, E, 2)
    bad = rng.random(E) < 0.2
    ei[1, bad] = rng.choice([-1, -7, V, V + 5, 2 ** 30], bad.sum())
    keep = ~bad
    kept_ei, kept_w = np.ascontiguousarray(ei[:, keep]), w[keep]
    K = int(keep.sum())
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    orow, ooff, ow = oracle.cootocsc(kept_ei, kept_w, V)
    assert np.array_equal(csc.column_offset.cpu().numpy(), ooff)
    assert np.array_equal(csc.row_indices.cpu().numpy()[:K], orow)
    assert np.array_equal(csc.edge_weight.cpu().numpy()[:K], ow)
    assert not csc.row_indices[K:].any() and not csc.edge_weight[K:].any()
    # one float per entry: the degree sum of gcn_norm
    deg = spmm(csc.column_offset, None, None, csc.edge_weight.view(-1, 1), V).view(-1).cpu().numpy()
    want = np.array([ow[ooff[v]:ooff[v + 1]].astype(np.float64).sum() for v in range(V)])
    sc = np.array([np.abs(ow[ooff[v]:ooff[v + 1]]).astype(np.float64).sum() for v in range(V)])
    assert_close(deg, want, sc, what="degree")
    x = rng.standard_normal(E).astype(np.float32)
    y = EdgeSoftmax(to_gpu(x), csc).cpu().numpy()
    want_y = oracle.edgesoftmax(x[:K], ooff)
    deg = np.diff(ooff)[np.repeat(np.arange(V), np.diff(ooff))].astype(np.float64)
    assert_close(y[:K], want_y, want_y * (1 + deg * 6e-3), atol=1e-7, what="softmax")
    xv = rng.standard_normal((V, 12)).astype(np.float32)
    csr = cootocsr(to_gpu(kept_ei), to_gpu(kept_w), V)
    out = aggregateWithWeight(to_gpu(xv), csc, csr).cpu().numpy()
    assert_close(out, oracle.aggregate(xv, orow, ooff, ow), _scale(xv, orow, ooff, ow), what="wide product")
