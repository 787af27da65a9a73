"""Edge softmax (forward/backward) and the scatter operators on the GPU
against the CPU oracle, through the operator wrappers and the C ABI."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def make_csc(ei, w, V):
    from jittorgeometric_amd.ops import cootocsc
    return cootocsc(to_gpu(ei), to_gpu(w), V), oracle.cootocsc(ei, w, V)


def test_edgesoftmax_reference_fixture_and_gradient():
    from jittorgeometric_amd import CSC
    from jittorgeometric_amd.ops import EdgeSoftmax
    g = GOLD["edgesoftmax_v3"]
    csc = CSC(torch.tensor(g["row_indices"], dtype=torch.int32, device=dev()),
              torch.tensor(g["column_offset"], dtype=torch.int32, device=dev()),
              torch.ones(4, device=dev()))
    x = torch.tensor(g["x"], device=dev(), requires_grad=True)
    y = EdgeSoftmax(x, csc)
    np.testing.assert_allclose(y.detach().cpu().numpy(), np.array(g["y"]), rtol=1e-6)
    # the reference test feeds the output to BCELoss against ones (tests/test_edgesoftmax.py:31-33)
    loss = torch.nn.functional.binary_cross_entropy(y, torch.ones_like(y))
    loss.backward()
    yh = y.detach().cpu().numpy()
    gy = (-1.0 / yh / 4.0).astype(np.float32)
    want = oracle.edgesoftmax_backward(gy, yh, np.array(g["column_offset"], np.int32))
    assert_close(x.grad.cpu().numpy(), want, rtol=1e-5, atol=1e-6, what="BCE gradient")


@pytest.mark.parametrize("V,E,H,hubs,seed", [
    (1, 0, 1, 0, 0), (1, 300, 1, 0, 1), (300, 2000, 1, 2, 2), (300, 2000, 2, 2, 3), (5000, 40000, 8, 3, 4),
    (2000, 300000, 1, 2, 5), (2000, 100000, 4, 1, 6), (700, 9000, 3, 2, 7), (700, 9000, 16, 2, 8),
    (20000, 30000, 64, 0, 9), (100, 5000, 128, 1, 10),
    # tile edge cases of the 1/2/4/8-head path: E a multiple of the tile (2048 and 1024 entries),
    # one entry more, mostly empty columns (more columns than entries in a tile), one column only
    (300, 4096, 1, 1, 11), (300, 4097, 2, 1, 12), (50, 3072, 4, 0, 13), (50, 2049, 8, 1, 14),
    (200000, 5000, 1, 0, 15), (300000, 3000, 8, 2, 16), (1, 70000, 2, 0, 17), (3, 40000, 8, 0, 18),
])
def test_edgesoftmax_forward_backward(V, E, H, hubs, seed):
    from jittorgeometric_amd.ops import EdgeSoftmax
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs, hub_share=0.5)
    csc, (row, off, _) = make_csc(ei, w, V)
    x = (3 * rng.standard_normal((E, H))).astype(np.float32)
    g = rng.standard_normal((E, H)).astype(np.float32)
    xt = to_gpu(x).requires_grad_(True)
    y = EdgeSoftmax(xt, csc)
    y.backward(to_gpu(g))
    want = oracle.edgesoftmax(x, off).reshape(E, H)
    seg = np.repeat(np.arange(V), np.diff(off))
    deg = np.diff(off)[seg].reshape(E, 1).astype(np.float64)
    # the reference adds a column's exp terms one after the other in fp32: its own
    # denominator is only good to about deg * 2^-24 relative, which is what the
    # comparison with it is allowed; against the exact (fp64) softmax the kernel
    # has to meet the plain 1e-5
    assert_close(y.detach().cpu().numpy(), want, scale=want * (1 + deg * 6e-3), rtol=1e-5, atol=1e-7,
                 what="softmax vs oracle")
    x64 = x.astype(np.float64)
    mx = np.full((V, H), -np.inf)
    np.maximum.at(mx, seg, x64)
    p64 = np.exp(x64 - mx[seg])
    den = np.zeros((V, H))
    np.add.at(den, seg, p64)
    assert_close(y.detach().cpu().numpy(), p64 / den[seg], rtol=1e-5, atol=1e-7, what="softmax vs fp64")
    # backward: compare on the oracle's own y so that only the backward kernel is judged
    wantg = oracle.edgesoftmax_backward(g, y.detach().cpu().numpy(), off).reshape(E, H)
    scale = np.zeros((V, H))
    np.add.at(scale, seg, np.abs(want.astype(np.float64) * g))
    assert_close(xt.grad.cpu().numpy(), wantg, scale=np.abs(wantg) + want * scale[seg], what="softmax backward")


def _column_layouts():
    """Column lengths whose first entries fall on the places the tile kernels treat differently:
    lane edges (a lane holds 8 or 4 consecutive entries), tile edges (2048 / 1024 entries),
    every entry a column of its own, columns inside one lane, columns over many lanes, runs of
    empty columns (more than a block has threads, more than a tile has entries)."""
    rng = np.random.default_rng(77)
    lay = {
        "lane_edges": [8] * 300 + [4] * 100 + [16] * 50 + [3, 5] * 80 + [1] * 64 + [7, 9] * 60,
        "tile_edges": [2048, 1024, 1024, 2047, 1, 2049, 1023, 1, 1024, 4096, 5, 3, 2040],
        "singles": [1] * 5000,
        "empties": [0] * 700 + [3] + [0] * 3000 + [2, 0, 0, 5] * 300 + [0] * 2500 + [2048] + [0] * 10,
        "long_inside": [1, 700, 2, 1300, 45, 2048 - 45, 6, 2000, 42],
        "mixed": list(rng.integers(0, 40, 800)) + [5000] + list(rng.integers(0, 6, 3000)) + [1, 9000, 1],
    }
    return lay


@pytest.mark.parametrize("layout", sorted(_column_layouts()))
@pytest.mark.parametrize("H", [1, 2, 4, 8])
def test_edgesoftmax_and_narrow_sums_on_built_columns(layout, H):
    from jittorgeometric_amd import CSC
    from jittorgeometric_amd.ops import EdgeSoftmax
    from jittorgeometric_amd.ops._common import spmm
    lens = np.asarray(_column_layouts()[layout], dtype=np.int64)
    V, E = len(lens), int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(len(lens) + H)
    row = rng.integers(0, V, E).astype(np.int32)
    w = rng.standard_normal(E).astype(np.float32)
    csc = CSC(to_gpu(row), to_gpu(off), to_gpu(w))
    x = (4 * rng.standard_normal((E, H))).astype(np.float32)
    g = rng.standard_normal((E, H)).astype(np.float32)
    xt = to_gpu(x).requires_grad_(True)
    y = EdgeSoftmax(xt, csc)
    y.backward(to_gpu(g))
    seg = np.repeat(np.arange(V), lens)
    x64 = x.astype(np.float64)
    mx = np.full((V, H), -np.inf)
    np.maximum.at(mx, seg, x64)
    p64 = np.exp(x64 - mx[seg])
    den = np.zeros((V, H))
    np.add.at(den, seg, p64)
    y64 = p64 / den[seg]
    assert_close(y.detach().cpu().numpy(), y64, rtol=1e-5, atol=1e-7, what="softmax vs fp64")
    dot = np.zeros((V, H))
    np.add.at(dot, seg, y64 * g)
    absdot = np.zeros((V, H))
    np.add.at(absdot, seg, np.abs(y64 * g))
    assert_close(xt.grad.cpu().numpy(), y64 * (g - dot[seg]), scale=np.abs(y64 * g) + y64 * absdot[seg],
                 what="softmax backward vs fp64")
    # the gather-sum over the same columns at the same widths (rows of H floats)
    feat = rng.standard_normal((V, H)).astype(np.float32)
    out = spmm(csc.column_offset, csc.row_indices, csc.edge_weight, to_gpu(feat), V).cpu().numpy()
    terms = w.astype(np.float64)[:, None] * feat.astype(np.float64)[row]
    want = np.zeros((V, H))
    np.add.at(want, seg, terms)
    mag = np.zeros((V, H))
    np.add.at(mag, seg, np.abs(terms))
    assert_close(out, want, scale=mag, what="narrow gather-sum vs fp64")


def test_edgesoftmax_reference_shapes_E_and_E1():
    from jittorgeometric_amd.ops import EdgeSoftmax
    rng = np.random.default_rng(30)
    V, E = 400, 5000
    ei, w = rand_graph(rng, V, E, 2)
    csc, (row, off, _) = make_csc(ei, w, V)
    x = rng.standard_normal(E).astype(np.float32)
    y1 = EdgeSoftmax(to_gpu(x), csc)
    y2 = EdgeSoftmax(to_gpu(x.reshape(E, 1)), csc)
    assert y1.shape == (E,) and y2.shape == (E, 1)
    assert torch.equal(y1, y2[:, 0])
    assert_close(y1.cpu().numpy(), oracle.edgesoftmax(x, off), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("H", [1, 4])
@pytest.mark.parametrize("variant", ["misaligned", "groups", "stage0", "stage1"])
def test_edgesoftmax_code_paths_agree(H, variant, monkeypatch):
    """Arrays that are not 16-byte aligned, the lane-group kernels, and both ways of
    moving a tile (direct / through LDS) give the default path's results."""
    from jittorgeometric_amd.ops import EdgeSoftmax
    rng = np.random.default_rng(40 + H)
    V, E = 3000, 50000
    ei, w = rand_graph(rng, V, E, 2)
    csc, (row, off, _) = make_csc(ei, w, V)
    x = rng.standard_normal((E, H)).astype(np.float32)
    g = rng.standard_normal((E, H)).astype(np.float32)
    xt = to_gpu(x).requires_grad_(True)
    y = EdgeSoftmax(xt, csc)
    y.backward(to_gpu(g))
    if variant == "misaligned":
        pad = torch.zeros(E * H + 1, device=dev())
        pad[1:] = to_gpu(x).reshape(-1)
        x2 = pad[1:].reshape(E, H).requires_grad_(True)
        assert x2.data_ptr() % 16 != 0
        gpad = torch.zeros(E * H + 1, device=dev())
        gpad[1:] = to_gpu(g).reshape(-1)
        g2 = gpad[1:].reshape(E, H)
    else:
        if variant == "groups":
            monkeypatch.setenv("JGAMD_SOFTMAX", "groups")
        else:
            monkeypatch.setenv("JGAMD_SOFTMAX_STAGE", variant[-1])
        x2 = to_gpu(x).requires_grad_(True)
        g2 = to_gpu(g)
    y2 = EdgeSoftmax(x2, csc)
    y2.backward(g2)
    assert_close(y2.detach().cpu().numpy(), y.detach().cpu().numpy(), rtol=2e-6, atol=1e-8, what=variant)
    gref = xt.grad.cpu().numpy()
    assert_close(x2.grad.cpu().numpy(), gref, scale=np.abs(gref) + 1e-3, rtol=1e-5, what=variant + " backward")


def test_edgesoftmax_large_logits_stay_finite():
    from jittorgeometric_amd.ops import EdgeSoftmax
    rng = np.random.default_rng(31)
    V, E = 100, 3000
    ei, w = rand_graph(rng, V, E)
    csc, (row, off, _) = make_csc(ei, w, V)
    x = (200 * rng.standard_normal(E)).astype(np.float32)      # exp(x) alone would overflow
    y = EdgeSoftmax(to_gpu(x), csc).cpu().numpy()
    assert np.isfinite(y).all()
    assert_close(y, oracle.edgesoftmax(x, off), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("V,E,F,seed", [(1, 0, 4, 0), (60, 500, 5, 1), (3000, 50000, 16, 2), (500, 20000, 128, 3),
                                        (5000, 3000, 33, 4)])
def test_scatter_ops_and_their_gradients(V, E, F, seed):
    from jittorgeometric_amd.ops import ScatterToEdge, ScatterToVertex
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs=2 if V > 10 else 0, hub_share=0.4)
    csc, (row, off, _) = make_csc(ei, w, V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    xe = rng.standard_normal((E, F)).astype(np.float32)
    for flow, flag in (("src", 0), ("dst", 1)):
        xt = to_gpu(x).requires_grad_(True)
        out = ScatterToEdge(xt, csc, flow)
        assert np.array_equal(out.detach().cpu().numpy(), oracle.scattertoedge(x, row, off, flag))
        out.backward(to_gpu(xe))
        want = oracle.edgetovertex(xe, row, off, flag)
        scale = oracle.edgetovertex(np.abs(xe), row, off, flag)
        assert_close(xt.grad.cpu().numpy(), want, scale, what="ScatterToEdge grad %s" % flow)
    et = to_gpu(xe).requires_grad_(True)
    out = ScatterToVertex(et, csc, "src")
    want = oracle.edgetovertex(xe, row, off, 1)
    assert_close(out.detach().cpu().numpy(), want, oracle.edgetovertex(np.abs(xe), row, off, 1), what="ScatterToVertex")
    out.backward(to_gpu(x))
    assert np.array_equal(et.grad.cpu().numpy(), oracle.scattertoedge(x, row, off, 1))
