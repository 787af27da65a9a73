"""GPU operators against the committed vectors of tests/golden (no oracle call)."""
import os

import numpy as np
import pytest
import torch

from util import assert_close, dev, to_gpu

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_vectors_v64.npz"))


def graph():
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    V = int(G["v_num"])
    return cootocsc(to_gpu(G["edge_index"]), to_gpu(G["edge_weight"]), V), \
        cootocsr(to_gpu(G["edge_index"]), to_gpu(G["edge_weight"]), V), V


def test_conversion_bit_exact():
    csc, csr, _ = graph()
    for got, key in ((csr.column_indices, "csr_col"), (csr.row_offset, "csr_off"), (csc.row_indices, "csc_row"),
                     (csc.column_offset, "csc_off")):
        assert np.array_equal(got.cpu().numpy(), G[key]), key
    assert np.array_equal(csr.edge_weight.cpu().numpy().view(np.int32), G["csr_w"].view(np.int32))
    assert np.array_equal(csc.edge_weight.cpu().numpy().view(np.int32), G["csc_w"].view(np.int32))


@pytest.mark.parametrize("F", [7, 8, 33])
def test_aggregate_forward_backward(F):
    from jittorgeometric_amd.ops import aggregateWithWeight
    csc, csr, _ = graph()
    x = to_gpu(G["x%d" % F]).requires_grad_(True)
    out = aggregateWithWeight(x, csc, csr)
    out.backward(to_gpu(G["x%d" % F]))
    assert_close(out.detach().cpu().numpy(), G["agg_fwd%d" % F], G["agg_fwd_terms%d" % F])
    assert_close(x.grad.cpu().numpy(), G["agg_bwd%d" % F], G["agg_bwd_terms%d" % F])


@pytest.mark.parametrize("H", [1, 2])
def test_edge_softmax(H):
    from jittorgeometric_amd.ops import EdgeSoftmax
    csc, _, _ = graph()
    x = to_gpu(G["sm_x%d" % H]).requires_grad_(True)
    y = EdgeSoftmax(x, csc)
    y.backward(to_gpu(G["sm_g%d" % H]))
    assert_close(y.detach().cpu().numpy(), G["sm_y%d" % H], rtol=1e-5, atol=1e-7)
    assert_close(x.grad.cpu().numpy(), G["sm_dx%d" % H], np.abs(G["sm_dx%d" % H]) + np.abs(G["sm_y%d" % H]))


def test_scatter_operators():
    from jittorgeometric_amd.ops import ScatterToEdge, ScatterToVertex
    csc, _, _ = graph()
    x = to_gpu(G["sc_x"]).requires_grad_(True)
    assert np.array_equal(ScatterToEdge(x, csc, "src").detach().cpu().numpy(), G["sc_src"])
    out = ScatterToEdge(x, csc, "dst")
    assert np.array_equal(out.detach().cpu().numpy(), G["sc_dst"])
    out.backward(to_gpu(G["sc_xe"]))
    assert_close(x.grad.cpu().numpy(), G["ev_dst"], G["ev_dst_terms"])
    x2 = to_gpu(G["sc_x"]).requires_grad_(True)
    ScatterToEdge(x2, csc, "src").backward(to_gpu(G["sc_xe"]))
    assert_close(x2.grad.cpu().numpy(), G["ev_src"], G["ev_src_terms"])
    assert_close(ScatterToVertex(to_gpu(G["sc_xe"]), csc, "src").cpu().numpy(), G["ev_dst"], G["ev_dst_terms"])


def test_fused_gat_forward():
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    csc, _, _ = graph()
    r2 = gat_forward_raw(to_gpu(G["gat_h"]), csc, to_gpu(G["gat_a_src"]), to_gpu(G["gat_a_dst"]), 0.2, want_alpha=True)
    assert_close(r2["alpha"].cpu().numpy(), G["gat_alpha2"], rtol=1e-5, atol=1e-7)
    assert_close(r2["out"].cpu().numpy(), G["gat_out2"], G["gat_terms2"])
    h1 = torch.from_numpy(np.ascontiguousarray(G["gat_h"][:, :1, :])).to(dev())
    r1 = gat_forward_raw(h1, csc, to_gpu(G["gat_a_src"][:1]), to_gpu(G["gat_a_dst"][:1]), 0.2, want_alpha=True)
    assert_close(r1["alpha"].cpu().numpy(), G["gat_alpha1"], rtol=1e-5, atol=1e-7)
    assert_close(r1["out"][:, 0, :].cpu().numpy(), G["gat_out1"], G["gat_terms2"][:, 0, :])
