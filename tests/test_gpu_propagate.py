"""Callers either side of the SpMM path on the GPU against the CPU oracle: the
product with a fused row finish, the propagation layers built on it (APPNP, SGConv,
GPRGNN, LightGCNConv, GCN2Conv, EvenNet, ChebNetII, BernNet), SpmmCoo and
toUndirected.  fp32, 1e-5 relative to the sum of absolute terms for one product,
1e-4 for the layers of several hops."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")))


def graphs(V, E, hubs, seed):
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    rng = np.random.default_rng(seed)
    ei, _ = rand_graph(rng, V, E, hubs)
    ei = ei[:, ei[0] != ei[1]]
    ei, w = oracle.gcn_norm(ei, None, V)
    ei = ei.astype(np.int32)
    csc_o, csr_o = oracle.cootocsc(ei, w, V), oracle.cootocsr(ei, w, V)
    return rng, ei, w, csc_o, csr_o, cootocsc(to_gpu(ei), to_gpu(w), V), cootocsr(to_gpu(ei), to_gpu(w), V)


def abs_prod(x, csx):
    """sum_j |w_j| |x[idx_j]| per output element, widened for long rows: the oracle adds a row's
    terms one after the other in fp32, so its own sum carries about deg * 2^-24 of this."""
    deg = np.diff(csx[1]).reshape(-1, 1).astype(np.float64)
    return oracle.aggregate(np.abs(x), csx[0], csx[1], np.abs(csx[2])).astype(np.float64) * (1 + deg * 6e-3)


@pytest.mark.parametrize("V,E,F,hubs,seed", [(1, 0, 4, 0, 0), (50, 0, 3, 0, 1), (300, 4000, 7, 0, 2),
                                             (3000, 60000, 64, 2, 3), (2000, 150000, 128, 1, 4),
                                             (5000, 40000, 33, 3, 5), (800, 30000, 256, 2, 6)])
def test_product_with_row_finish(V, E, F, hubs, seed):
    """beta * A x + alpha * h in one call; hub rows are cut into pieces, so the finish must be
    applied exactly once to them too."""
    from jittorgeometric_amd.ops._common import spmm_axpby
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, E, hubs, seed)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((V, F)).astype(np.float32)
    base = oracle.aggregate_with_weight(x, csc_o).astype(np.float64)
    scale = abs_prod(x, csc_o)
    args = (csc.column_offset, csc.row_indices, csc.edge_weight, to_gpu(x), V)
    for beta, alpha, hh in ((0.9, 0.1, h), (1.0, 0.0, None), (-2.0, 0.5, h), (0.25, 0.0, h), (1.0, 1.0, x)):
        got = spmm_axpby(*args, beta, alpha, None if hh is None else to_gpu(hh)).cpu().numpy()
        want = beta * base + (alpha * hh.astype(np.float64) if hh is not None else 0.0)
        assert_close(got, want, scale=abs(beta) * scale + (abs(alpha) * np.abs(hh) if hh is not None else 0.0) + 1e-30,
                     what="beta=%g alpha=%g" % (beta, alpha))


def test_row_finish_with_unaligned_h():
    from jittorgeometric_amd.ops._common import spmm_axpby
    V, F = 700, 64
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, 9000, 1, 11)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((V, F)).astype(np.float32)
    pad = torch.zeros(V * F + 1, device=dev())
    pad[1:] = to_gpu(h).reshape(-1)
    h_dev = pad[1:].reshape(V, F)
    assert h_dev.data_ptr() % 16 != 0
    got = spmm_axpby(csc.column_offset, csc.row_indices, csc.edge_weight, to_gpu(x), V, 0.8, 0.2, h_dev).cpu().numpy()
    want = 0.8 * oracle.aggregate_with_weight(x, csc_o).astype(np.float64) + 0.2 * h
    assert_close(got, want, scale=0.8 * abs_prod(x, csc_o) + 0.2 * np.abs(h))


@pytest.mark.parametrize("spmm", [True, False])
@pytest.mark.parametrize("V,E,F,K,hubs,seed", [(400, 5000, 16, 1, 0, 20), (3000, 50000, 41, 4, 2, 21),
                                               (1500, 80000, 128, 10, 1, 22)])
def test_appnp_forward_backward(V, E, F, K, hubs, seed, spmm):
    from jittorgeometric_amd.nn import APPNP
    alpha = 0.1
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, E, hubs, seed)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    want = oracle.appnp(x, csc_o, K, alpha)
    # magnitude of the terms: the same recursion on absolute values
    mag = oracle.appnp(np.abs(x), (csc_o[0], csc_o[1], np.abs(csc_o[2])), K, alpha).astype(np.float64)
    mag = mag * (1 + np.diff(csc_o[1]).reshape(-1, 1) * 6e-3)
    outs = []
    for fused in (True, False):
        xt = to_gpu(x).requires_grad_(True)
        layer = APPNP(K, alpha, spmm=spmm, fused=fused)
        out = layer(xt, csc, csr)
        out.backward(to_gpu(g))
        assert_close(out.detach().cpu().numpy(), want, scale=mag, rtol=3e-5, what="forward fused=%s" % fused)
        outs.append((out.detach().cpu().numpy(), xt.grad.cpu().numpy()))
    # gradient: the transposed recursion, g_x = M^K g + alpha * sum_{i<K} M^i g with M = (1-alpha) A^T,
    # restated with the oracle's CSR aggregation in fp64
    v = g.astype(np.float64)
    gmag = np.abs(g).astype(np.float64)
    for _ in range(K):
        v = (1 - alpha) * oracle.aggregate(v.astype(np.float32), *csr_o).astype(np.float64) + alpha * g
        gmag = (1 - alpha) * oracle.aggregate(gmag.astype(np.float32), csr_o[0], csr_o[1], np.abs(csr_o[2])) + alpha * np.abs(g)
    for (_, grad), name in zip(outs, ("fused", "chain")):
        assert_close(grad, v, scale=gmag, rtol=5e-5, what="gradient " + name)
    assert_close(outs[0][0], outs[1][0], scale=mag, rtol=2e-5, what="fused vs chain")


def test_propagate_axpby_gradients():
    from jittorgeometric_amd.ops import propagate_axpby
    V, F = 500, 24
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, 6000, 1, 30)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    xt, ht = to_gpu(x).requires_grad_(True), to_gpu(h).requires_grad_(True)
    out = propagate_axpby(xt, ht, csc, csr, beta=0.7, alpha=0.3)
    out.backward(to_gpu(g))
    assert_close(out.detach().cpu().numpy(), 0.7 * oracle.aggregate_with_weight(x, csc_o).astype(np.float64) + 0.3 * h,
                 scale=0.7 * abs_prod(x, csc_o) + 0.3 * np.abs(h))
    assert_close(xt.grad.cpu().numpy(), 0.7 * oracle.aggregate_with_weight_grad(g, csr_o).astype(np.float64),
                 scale=0.7 * abs_prod(g, csr_o) + 1e-30)
    assert_close(ht.grad.cpu().numpy(), 0.3 * g.astype(np.float64))
    # only one of the two orders given: the other is the cached transpose
    out2 = propagate_axpby(to_gpu(x), to_gpu(h), None, csr, beta=0.7, alpha=0.3)
    assert_close(out2.cpu().numpy(), out.detach().cpu().numpy(), scale=0.7 * abs_prod(x, csc_o) + 0.3 * np.abs(h))


@pytest.mark.parametrize("spmm", [True, False])
def test_sgconv_forward_backward(spmm):
    from jittorgeometric_amd.nn import SGConv
    V, Fin, Fout, K = 1200, 48, 7, 3
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, 20000, 1, 40)
    x = rng.standard_normal((V, Fin)).astype(np.float32)
    layer = SGConv(Fin, Fout, K=K, spmm=spmm).to(dev())
    with torch.no_grad():
        layer.bias.copy_(to_gpu(rng.standard_normal(Fout).astype(np.float32)))
    W, b = layer.weight.detach().cpu().numpy(), layer.bias.detach().cpu().numpy()
    xt = to_gpu(x).requires_grad_(True)
    out = layer(xt, csc, csr)
    want = oracle.sgconv(x, csc_o, K, W, b)
    # K products and one dense product in a row, each good to 1e-5 of its sum of absolute
    # terms; the bound is carried through the chain by running it on absolute values
    steps = (K + 1) * 1e-5
    abs_csc = (csc_o[0], csc_o[1], np.abs(csc_o[2]))
    abs_csr = (csr_o[0], csr_o[1], np.abs(csr_o[2]))
    assert_close(out.detach().cpu().numpy(), want, scale=oracle.sgconv(np.abs(x), abs_csc, K, np.abs(W), np.abs(b)),
                 rtol=steps)
    g = rng.standard_normal((V, Fout)).astype(np.float32)
    out.backward(to_gpu(g))
    # d/dx = (A^T)^K (g W^T), d/dW = (A^K x)^T g
    v = (g.astype(np.float64) @ W.T.astype(np.float64)).astype(np.float32)
    va = (np.abs(g).astype(np.float64) @ np.abs(W).T.astype(np.float64)).astype(np.float32)
    ak, aka = x, np.abs(x)
    for _ in range(K):
        v = oracle.aggregate_with_weight_grad(v, csr_o)
        va = oracle.aggregate_with_weight_grad(va, abs_csr)
        ak = oracle.aggregate_with_weight(ak, csc_o)
        aka = oracle.aggregate_with_weight(aka, abs_csc)
    assert_close(xt.grad.cpu().numpy(), v, scale=va, rtol=steps)
    gw = ak.astype(np.float64).T @ g.astype(np.float64)
    assert_close(layer.weight.grad.cpu().numpy(), gw, scale=aka.astype(np.float64).T @ np.abs(g).astype(np.float64),
                 rtol=steps)
    assert_close(layer.bias.grad.cpu().numpy(), g.astype(np.float64).sum(0), scale=np.abs(g).sum(0), rtol=1e-5)


def test_spmmcoo_reference_fixture_and_random():
    from jittorgeometric_amd.ops import SpmmCoo
    f = GOLD["spmmcoo_v3"]
    x = torch.tensor(f["x"], device=dev())
    ei = torch.tensor(f["edge_index"], dtype=torch.int32, device=dev())
    w = torch.tensor(f["edge_weight"], device=dev())
    assert SpmmCoo(x, ei, w).tolist() == f["out"]
    assert SpmmCoo(x, ei, w, trans_A=False).tolist() == f["out_no_trans"]
    rng = np.random.default_rng(50)
    V, E, F = 4000, 70000, 40
    ein, wn = rand_graph(rng, V, E, 2)
    xn = rng.standard_normal((V, F)).astype(np.float32)
    gn = rng.standard_normal((V, F)).astype(np.float32)
    for trans in (True, False):
        xt = to_gpu(xn).requires_grad_(True)
        out = SpmmCoo(xt, to_gpu(ein), to_gpu(wn), trans_A=trans)
        out.backward(to_gpu(gn))
        want = oracle.spmmcoo(xn, ein, wn, trans_A=trans)
        scale = oracle.spmmcoo(np.abs(xn), ein, np.abs(wn), trans_A=trans).astype(np.float64)
        # the oracle adds in edge order, one fp32 rounding per edge: hub rows carry deg * 2^-24
        deg = np.bincount(ein[1] if trans else ein[0], minlength=V).reshape(V, 1)
        assert_close(out.detach().cpu().numpy(), want, scale=scale * (1 + deg * 6e-3), what="trans_A=%s" % trans)
        wantg = oracle.spmmcoo(gn, ein, wn, trans_A=not trans)
        gscale = oracle.spmmcoo(np.abs(gn), ein, np.abs(wn), trans_A=not trans).astype(np.float64)
        degg = np.bincount(ein[0] if trans else ein[1], minlength=V).reshape(V, 1)
        assert_close(xt.grad.cpu().numpy(), wantg, scale=gscale * (1 + degg * 6e-3), what="grad trans_A=%s" % trans)
    with pytest.raises(Exception):
        SpmmCoo(x, ei, w, trans_B=True)


@pytest.mark.parametrize("V,E,seed", [(3, 0, 0), (1, 5, 1), (8, 40, 2), (2000, 30000, 3), (50000, 200000, 4)])
def test_toundirected(V, E, seed):
    from jittorgeometric_amd.ops import toUndirected
    rng = np.random.default_rng(seed)
    ei = rng.integers(0, V, (2, E)).astype(np.int32)
    attr = rng.standard_normal(E).astype(np.float32)
    ni, na = toUndirected(to_gpu(ei), to_gpu(attr), V)
    wi, wa = oracle.toundirected(ei, attr)
    assert np.array_equal(ni.cpu().numpy(), wi)
    assert np.array_equal(na.cpu().numpy().view(np.int32), wa.view(np.int32))
    assert tuple(na.shape) == (1, wi.shape[1])


def test_toundirected_reference_fixture():
    from jittorgeometric_amd.ops import toUndirected
    f = GOLD["toundirected_v3"]
    ni, na = toUndirected(torch.tensor(f["edge_index"], device=dev()), torch.tensor(f["edge_attr"], device=dev()),
                          f["num_nodes"])
    assert ni.tolist() == f["new_edge_index"] and na.tolist() == f["new_edge_attr"]


def test_row_finish_on_wide_rows_runs_as_its_own_pass():
    """x larger than 4 GiB: the product takes the 64-bit address kernels, which have no fused
    finish; the blend then runs as a separate pass with the same result."""
    from jittorgeometric_amd.ops._common import spmm, spmm_axpby
    rng = np.random.default_rng(46)
    C, F, R, E = 4_300_000, 256, 3000, 40000
    x = torch.empty((C, F), dtype=torch.float32, device=dev())
    x.normal_()
    src = rng.integers(0, C, E).astype(np.int32)
    dst = rng.integers(0, R, E).astype(np.int32)
    w = rng.standard_normal(E).astype(np.float32)
    row, off, cw = oracle.cootocsc(np.stack([src, dst]), w, R)
    h = torch.randn(R, F, device=dev())
    plain = spmm(to_gpu(off), to_gpu(row), to_gpu(cw), x, R)
    got = spmm_axpby(to_gpu(off), to_gpu(row), to_gpu(cw), x, R, 0.75, 0.25, h)
    want = 0.75 * plain.double() + 0.25 * h.double()
    assert_close(got.cpu().numpy(), want.cpu().numpy(), scale=(0.75 * plain.abs() + 0.25 * h.abs()).cpu().numpy() + 1e-6)


@pytest.mark.parametrize("F", [7, 64, 130])
def test_aggregate_with_bias_row(F):
    """One row of h added to every output row (a layer's bias), and its gradients."""
    from jittorgeometric_amd.ops import aggregate_bias
    V = 2500
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, 40000, 2, 60 + F)
    x = rng.standard_normal((V, F)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    xt, bt = to_gpu(x).requires_grad_(True), to_gpu(b).requires_grad_(True)
    out = aggregate_bias(xt, bt, csc, csr)
    out.backward(to_gpu(g))
    want = oracle.aggregate_with_weight(x, csc_o).astype(np.float64) + b
    assert_close(out.detach().cpu().numpy(), want, scale=abs_prod(x, csc_o) + np.abs(b))
    assert_close(xt.grad.cpu().numpy(), oracle.aggregate_with_weight_grad(g, csr_o), scale=abs_prod(g, csr_o) + 1e-30)
    assert_close(bt.grad.cpu().numpy(), g.astype(np.float64).sum(0), scale=np.abs(g).sum(0))


@pytest.mark.parametrize("init", ["PPR", "SGC", "NPPR", "WS"])
def test_gprgnn_forward_backward(init):
    from jittorgeometric_amd.nn import GPRGNN
    V, F, K = 1500, 20, 4
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, 25000, 1, 80)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    layer = GPRGNN(K, 0.1, init, spmm=False, Gamma=[0.5, -0.2, 0.1, 0.3, 0.05]).to(dev())
    temp = layer.temp.detach().cpu().numpy()
    if init == "PPR":
        assert np.allclose(temp, [0.1, 0.09, 0.081, 0.0729, 0.6561])
    xt = to_gpu(x).requires_grad_(True)
    out = layer(xt, csc, csr)
    out.backward(to_gpu(g))
    want = oracle.gprgnn(x, csc_o, temp)
    mag = oracle.gprgnn(np.abs(x), (csc_o[0], csc_o[1], np.abs(csc_o[2])), np.abs(temp)).astype(np.float64)
    mag = mag * (1 + np.diff(csc_o[1]).reshape(-1, 1) * 6e-3)
    assert_close(out.detach().cpu().numpy(), want, scale=mag + 1e-30, rtol=3e-5)
    # d/dtemp[k] = <g, A^k x>;  d/dx = sum_k temp[k] (A^T)^k g
    xs, gs = [x], [g]
    for _ in range(K):
        xs.append(oracle.aggregate_with_weight(xs[-1], csc_o))
        gs.append(oracle.aggregate_with_weight_grad(gs[-1], csr_o))
    gt = np.array([(g.astype(np.float64) * xk).sum() for xk in xs])
    gts = np.array([(np.abs(g).astype(np.float64) * np.abs(xk)).sum() for xk in xs])
    assert_close(layer.temp.grad.cpu().numpy(), gt, scale=gts, rtol=1e-4)
    gx = sum(float(temp[k]) * gs[k].astype(np.float64) for k in range(K + 1))
    gxs = sum(abs(float(temp[k])) * np.abs(gs[k]).astype(np.float64) for k in range(K + 1))
    assert_close(xt.grad.cpu().numpy(), gx, scale=gxs + 1e-3, rtol=1e-4)


# ------------------------------------------- polynomial layers built on the fused hop ---
def _dense64(ei, w, V):
    A = torch.zeros((V, V), dtype=torch.float64)
    A.index_put_((torch.from_numpy(ei[1].astype(np.int64)), torch.from_numpy(ei[0].astype(np.int64))),
                 torch.from_numpy(w.astype(np.float64)), accumulate=True)
    return A


def _check_layer(run_gpu, model, A_list, x_list, params, what, rtol=1e-4):
    """Forward and every gradient of a layer on the GPU against a float64 dense model of it.
    model(As, xs, ps, sub) is written with sub(a, b) for every subtraction, so that the same
    expression on absolute values (sub = add) bounds the size of the terms that were added."""
    rng = np.random.default_rng(5)
    xs_g = [to_gpu(x).requires_grad_(True) for x in x_list]
    out = run_gpu(xs_g)
    g = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    out.backward(to_gpu(g))
    xs64 = [torch.from_numpy(x).double().requires_grad_(True) for x in x_list]
    ps64 = [p.detach().cpu().double().requires_grad_(True) for p in params]
    want = model(A_list, xs64, ps64, lambda a, b: a - b)
    want.backward(torch.from_numpy(g).double())
    mag = model([A.abs() for A in A_list], [x.detach().abs() for x in xs64], [p.detach().abs() for p in ps64],
                lambda a, b: a + b).detach().numpy()
    assert_close(out.detach().cpu().numpy(), want.detach().numpy(), scale=mag + 1e-30, rtol=rtol, what=what + " forward")
    # gradients: the size of their terms comes from the same model run on |g| through the transposes
    for got, ref64, name in [(t.grad, r.grad, "x%d" % i) for i, (t, r) in enumerate(zip(xs_g, xs64))] + \
                            [(p.grad, r.grad, "param%d" % i) for i, (p, r) in enumerate(zip(params, ps64))]:
        if ref64 is None:
            assert got is None or float(got.abs().max()) == 0.0
            continue
        ref = ref64.numpy()
        bound = np.abs(ref).max() + 1e-30
        assert got is not None, name
        err = np.abs(got.cpu().numpy().astype(np.float64) - ref).max()
        # a coefficient's gradient is one sum over all V * F products, whose terms cancel: looser
        tol = 1e-4 if name.startswith("x") else 2e-3
        assert err <= tol * bound, "%s gradient of %s: err %g against max %g" % (what, name, err, bound)
    return out.detach().cpu().numpy()


def _poly_graph(V=1500, E=25000, seed=90):
    rng, ei, w, csc_o, csr_o, csc, csr = graphs(V, E, 1, seed)
    return rng, ei, w, csc_o, csc, csr, _dense64(ei, w, V)


@pytest.mark.parametrize("spmm", [True, False])
def test_lightgcn_and_gcn2conv(spmm):
    from jittorgeometric_amd.nn import GCN2Conv, LightGCNConv
    V, F = 1500, 24
    rng, ei, w, csc_o, csc, csr, A = _poly_graph()
    x = rng.standard_normal((V, F)).astype(np.float32)
    x0 = rng.standard_normal((V, F)).astype(np.float32)
    layer = LightGCNConv(spmm=spmm)
    got = _check_layer(lambda xs: layer(xs[0], csc, csr), lambda As, xs, ps, sub: As[0] @ xs[0], [A], [x], [], "LightGCNConv")
    assert_close(got, oracle.lightgcn(x, csc_o), scale=abs_prod(x, csc_o) + 1e-30)
    a, b = 0.1, 0.35
    for fused in (True, False):
        conv = GCN2Conv(F, F, spmm=spmm, fused=fused).to(dev())

        def model(As, xs, ps, sub):
            support = (1 - b) * (1 - a) * xs[0] + b * xs[0] @ ps[0]
            return As[0] @ support + (1 - b) * a * xs[1] + b * xs[1] @ ps[1]
        got = _check_layer(lambda xs: conv(xs[0], xs[1], csc, csr, a, b), model, [A], [x, x0], [conv.weight1, conv.weight2],
                           "GCN2Conv fused=%s" % fused)
        want = oracle.gcn2conv(x, x0, csc_o, conv.weight1.detach().cpu().numpy(), conv.weight2.detach().cpu().numpy(), a, b)
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("K", [1, 2, 3, 4, 7])
def test_evennet(K):
    from jittorgeometric_amd.nn import EvenNet
    V, F, alpha = 1500, 20, 0.2
    rng, ei, w, csc_o, csc, csr, A = _poly_graph(seed=91)
    x = rng.standard_normal((V, F)).astype(np.float32)
    t = oracle.evennet_temp(K, alpha)

    def model(As, xs, ps, sub):
        out, v = t[0] * xs[0], xs[0]
        for k in range(K):
            v = As[0] @ v
            if k // 2 == 1:
                out = out + t[k + 1] * v
        return out
    want = oracle.evennet(x, csc_o, K, alpha)
    for fused, spmm in ((True, True), (True, False), (False, False)):
        layer = EvenNet(K, alpha, spmm=spmm, fused=fused)
        assert np.allclose(layer.temp, t)
        got = _check_layer(lambda xs: layer(xs[0], csc, csr), model, [A], [x], [], "EvenNet K=%d fused=%s" % (K, fused))
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("K", [1, 2, 5])
def test_chebnet2(K):
    from jittorgeometric_amd.nn import ChebNetII
    from jittorgeometric_amd.nn.conv.chebnet2_conv import node_table
    V, F = 1500, 20
    rng, ei, w, csc_o, csc, csr, A = _poly_graph(seed=92)
    x = rng.standard_normal((V, F)).astype(np.float32)
    temp0 = (rng.random(K + 1) * 2 - 0.4).astype(np.float32)       # some below zero: clamped
    table = torch.from_numpy(node_table(K) * (2.0 / (K + 1)))

    def model(As, xs, ps, sub):
        # the run on absolute values (sub adds) takes the table's absolute values too
        coe = (table.abs() if sub(1.0, 1.0) == 2.0 else table) @ torch.relu(ps[0])
        t0 = xs[0]
        t1 = As[0] @ t0
        out = coe[0] / 2 * t0 + coe[1] * t1
        for i in range(2, K + 1):
            t2 = sub(2 * (As[0] @ t1), t0)
            out = out + coe[i] * t2
            t0, t1 = t1, t2
        return out
    with pytest.raises(ValueError):
        ChebNetII(0)
    for fused, spmm in ((True, True), (True, False), (False, False)):
        layer = ChebNetII(K, spmm=spmm, fused=fused).to(dev())
        assert torch.equal(layer.temp.detach().cpu(), torch.ones(K + 1))
        with torch.no_grad():
            layer.temp.copy_(to_gpu(temp0))
        np.testing.assert_allclose(layer.coefficients().detach().cpu().numpy(), oracle.chebnet2_coefficients(temp0),
                                   rtol=1e-5, atol=1e-6)
        got = _check_layer(lambda xs: layer(xs[0], csc, csr), model, [A], [x], [layer.temp], "ChebNetII K=%d fused=%s" % (K, fused))
        want = oracle.chebnet2(x, csc_o, temp0)
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("K", [1, 2, 4])
def test_bernnet(K):
    from math import comb
    from jittorgeometric_amd.nn import BernNet
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    V, F = 1200, 16
    rng, ei, w, csc_o, csc, csr, A = _poly_graph(V=V, E=20000, seed=93)
    loops = np.stack([np.arange(V), np.arange(V)]).astype(np.int32)
    ei2 = np.concatenate([ei, loops], axis=1)
    w1 = np.concatenate([-w, np.ones(V, np.float32)])              # L = I - A
    w2 = np.concatenate([w, np.ones(V, np.float32)])               # 2I - L = I + A
    csc1, csr1 = cootocsc(to_gpu(ei2), to_gpu(w1), V), cootocsr(to_gpu(ei2), to_gpu(w1), V)
    csc2, csr2 = cootocsc(to_gpu(ei2), to_gpu(w2), V), cootocsr(to_gpu(ei2), to_gpu(w2), V)
    A1, A2 = _dense64(ei2, w1, V), _dense64(ei2, w2, V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    temp0 = (rng.random(K + 1) * 2 - 0.3).astype(np.float32)

    def model(As, xs, ps, sub):
        t = torch.relu(ps[0])
        tmp = [xs[0]]
        for _ in range(K):
            tmp.append(As[1] @ tmp[-1])
        out = 0
        for i in range(K + 1):
            v = tmp[K - i]
            for _ in range(i):
                v = As[0] @ v
            out = out + comb(K, i) / 2 ** K * t[i] * v
        return out
    want = oracle.bernnet(x, oracle.cootocsc(ei2, w1, V), oracle.cootocsc(ei2, w2, V), temp0)
    for fused, spmm in ((True, True), (True, False), (False, False)):
        layer = BernNet(K, spmm=spmm, fused=fused).to(dev())
        with torch.no_grad():
            layer.temp.copy_(to_gpu(temp0))
        got = _check_layer(lambda xs: layer(xs[0], csc1, csr1, csc2, csr2), model, [A1, A2], [x], [layer.temp],
                           "BernNet K=%d fused=%s" % (K, fused))
        scale = np.abs(model([A1.abs(), A2.abs()], [torch.from_numpy(np.abs(x)).double()], [torch.from_numpy(np.abs(temp0)).double()],
                             None).numpy())
        assert_close(got, want, scale=scale + 1e-30, rtol=1e-4, what="BernNet against the oracle's order of products")
    # all weights one on (L, 2I - L): the binomial theorem gives x back
    layer = BernNet(3).to(dev())
    out = layer(to_gpu(x), csc1, csr1, csc2, csr2).cpu().detach().numpy()
    assert np.abs(out - x).max() < 1e-4
