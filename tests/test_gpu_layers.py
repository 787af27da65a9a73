"""Layer-level parity: GCNConv / SAGEConv forward and backward on the GPU
against a dense fp64 PyTorch model (the small Cora-like configuration is small
enough for a dense adjacency), and the two propagation routes against each
other."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, to_gpu

pytestmark = pytest.mark.gpu


def cora_like():
    from jittorgeometric_amd import synthetic
    ei, V = synthetic.make("cora_like")
    rng = np.random.default_rng(1)
    x = (rng.random((V, 1433)) < 0.013).astype(np.float32)
    x = x / np.maximum(x.sum(1, keepdims=True), 1)
    y = rng.integers(0, 7, V)
    return ei, V, x, y


def dense_adj(ei, w, V):
    A = torch.zeros((V, V), dtype=torch.float64)
    A.index_put_((torch.from_numpy(ei[1].astype(np.int64)), torch.from_numpy(ei[0].astype(np.int64))),
                 torch.from_numpy(w.astype(np.float64)), accumulate=True)
    return A


@pytest.mark.parametrize("spmm", [False, True])
def test_two_layer_gcn_forward_backward_config1(spmm):
    from jittorgeometric_amd.nn import GCNConv, gcn_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    ei, V, x, y = cora_like()
    eit, wt = gcn_norm(to_gpu(ei), None, V)
    oei, ow = oracle.gcn_norm(ei, None, V)
    assert np.array_equal(eit.cpu().numpy(), oei)
    assert_close(wt.cpu().numpy(), ow, rtol=1e-6, atol=0)
    assert eit.shape[1] == 13264
    csc, csr = cootocsc(eit, wt, V), cootocsr(eit, wt, V)
    torch.manual_seed(0)
    l1, l2 = GCNConv(1433, 256, spmm=spmm).to(dev()), GCNConv(256, 7, spmm=spmm).to(dev())
    xt = to_gpu(x)
    yt = to_gpu(y)
    out = l2(torch.relu(l1(xt, csc, csr)), csc, csr)
    loss = torch.nn.functional.cross_entropy(out, yt)
    loss.backward()

    A = dense_adj(oei, ow, V)
    W1, b1, W2, b2 = (p.detach().cpu().double().requires_grad_(True) for p in (l1.weight, l1.bias, l2.weight, l2.bias))
    x64 = torch.from_numpy(x.astype(np.float64))
    ref = A @ (torch.relu(A @ (x64 @ W1) + b1) @ W2) + b2
    rloss = torch.nn.functional.cross_entropy(ref, torch.from_numpy(y))
    rloss.backward()
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=1e-5, what="logits")
    assert abs(loss.item() - rloss.item()) < 1e-5
    for got, want, name in ((l1.weight.grad, W1.grad, "W1"), (l1.bias.grad, b1.grad, "b1"),
                            (l2.weight.grad, W2.grad, "W2"), (l2.bias.grad, b2.grad, "b2")):
        want = want.numpy()
        assert_close(got.cpu().numpy(), want, np.abs(want) + np.abs(want).max() * 1e-2, rtol=1e-4, atol=1e-8,
                     what="grad " + name)


@pytest.mark.parametrize("spmm,root", [(False, True), (True, True), (False, False)])
def test_sage_layer_asymmetric_weights(spmm, root):
    """sage_norm weights are not symmetric, so backward must be the true
    transpose of forward (CSR arrays), not a second forward product."""
    from jittorgeometric_amd.nn import SAGEConv, sage_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from jittorgeometric_amd import synthetic
    V = 3000
    ei = synthetic.chung_lu(V, 40000, 2.1, max_degree=800, seed=9)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((V, 100)).astype(np.float32)
    g = rng.standard_normal((V, 47)).astype(np.float32)
    eit, wt = sage_norm(to_gpu(ei), None, V)
    oei, ow = oracle.sage_norm(ei, None, V)
    assert np.array_equal(eit.cpu().numpy(), oei)
    assert_close(wt.cpu().numpy(), ow, rtol=1e-6, atol=0)
    csc, csr = cootocsc(eit, wt, V), cootocsr(eit, wt, V)
    torch.manual_seed(0)
    layer = SAGEConv(100, 47, root_weight=root, spmm=spmm).to(dev())
    xt = to_gpu(x).requires_grad_(True)
    out = layer(xt, csc=csc, csr=csr)
    out.backward(to_gpu(g))
    # same layer fed the COO list converts internally and must agree
    out2 = layer(to_gpu(x), to_gpu(ei), None)
    assert torch.allclose(out.detach(), out2.detach(), rtol=1e-5, atol=1e-6)

    A = dense_adj(oei, ow, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W1 = layer.weight1.detach().cpu().double().requires_grad_(True)
    ref = (A @ x64) @ W1 + layer.bias.detach().cpu().double()
    if root:
        ref = ref + x64 @ layer.root_weight.detach().cpu().double()
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=1e-5, what="out")
    want = x64.grad.numpy()
    assert_close(xt.grad.cpu().numpy(), want, np.abs(want) + np.abs(want).mean(), rtol=1e-4, what="grad x")
    want = W1.grad.numpy()
    assert_close(layer.weight1.grad.cpu().numpy(), want, np.abs(want) + np.abs(want).max() * 1e-2, rtol=1e-4,
                 what="grad W1")


def test_spmmcsr_reference_grad_switch():
    from jittorgeometric_amd.ops import SpmmCsr, cootocsr, spmmcsr
    from util import rand_graph
    rng = np.random.default_rng(5)
    V, E, F = 500, 6000, 16
    ei, w = rand_graph(rng, V, E)
    csr = cootocsr(to_gpu(ei), to_gpu(w), V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    g = rng.standard_normal((V, F)).astype(np.float32)
    ocsr, ocsc = oracle.cootocsr(ei, w, V), oracle.cootocsc(ei, w, V)
    try:
        for flag, arrays in ((False, ocsr), (True, ocsc)):
            want = oracle.aggregate(g, *arrays)
            terms = oracle.aggregate(np.abs(g), arrays[0], arrays[1], np.abs(arrays[2]))
            spmmcsr.REFERENCE_GRAD = flag
            xt = to_gpu(x).requires_grad_(True)
            SpmmCsr(xt, csr).backward(to_gpu(g))
            assert_close(xt.grad.cpu().numpy(), want, terms, what="REFERENCE_GRAD=%s" % flag)
    finally:
        spmmcsr.REFERENCE_GRAD = False


@pytest.mark.parametrize("R,F", [(1, 1), (5000, 47), (100000, 7), (70000, 128), (3000, 602), (0, 16), (2049, 256)])
def test_bias_gradient_column_sum(R, F):
    from jittorgeometric_amd.nn.dense import add_bias, column_sum
    rng = np.random.default_rng(R + F)
    g = rng.standard_normal((R, F)).astype(np.float32)
    got = column_sum(to_gpu(g)).cpu().numpy() if R > 0 else column_sum(torch.empty((0, F), device=dev())).cpu().numpy()
    want = g.astype(np.float64).sum(0)
    assert_close(got, want, np.abs(g).astype(np.float64).sum(0), what="column sum")
    if R > 0:
        b = torch.zeros(F, device=dev(), requires_grad=True)
        x = to_gpu(g).requires_grad_(True)
        add_bias(x, b).backward(to_gpu(g))
        assert_close(b.grad.cpu().numpy(), (g.astype(np.float64) ** 1).sum(0), np.abs(g).astype(np.float64).sum(0))
        assert torch.equal(x.grad, to_gpu(g))


def test_gcn_norm_with_hub_destination_matches_oracle():
    from jittorgeometric_amd.nn import gcn_norm, sage_norm
    from util import rand_graph
    rng = np.random.default_rng(91)
    V, E = 20000, 400000
    ei, _ = rand_graph(rng, V, E, hubs=1, hub_share=0.6)
    # several self-loops on one node make "which weight becomes the loop weight" order-dependent
    # in the reference too (utils/loop.py:130-132); keep at most none
    ei = ei[:, ei[0] != ei[1]]
    w = rng.random(ei.shape[1]).astype(np.float32) + 0.5
    for fn, ofn in ((gcn_norm, oracle.gcn_norm), (sage_norm, oracle.sage_norm)):
        gi, gw = fn(to_gpu(ei), to_gpu(w), V)
        oi, ow = ofn(ei, w, V)
        assert np.array_equal(gi.cpu().numpy(), oi)
        # degrees of 10^5-edge hubs are float sums in different orders
        assert_close(gw.cpu().numpy(), ow, rtol=2e-4, atol=0, what=fn.__name__)


@pytest.mark.parametrize("V,E,with_w,fill,seed", [(4, 0, True, 1.0, 0), (7, 30, True, 1.0, 1), (7, 30, False, 2.0, 2),
                                                  (5000, 80000, True, 2.0, 3), (3000, 2048, True, 1.0, 4),
                                                  (3000, 2049, False, 1.0, 5), (1, 5, True, 1.0, 6)])
def test_add_remaining_self_loops_kernels(V, E, with_w, fill, seed):
    """Kept edges in input order, one loop per node appended, a dropped loop's weight kept (at most
    one loop per node in the input: with several the reference keeps whichever its indexed assignment
    writes last)."""
    from jittorgeometric_amd.utils import add_remaining_self_loops
    rng = np.random.default_rng(seed)
    ei = rng.integers(0, V, (2, E)).astype(np.int32)
    ei = ei[:, ei[0] != ei[1]]
    loops = rng.permutation(V)[:max(V // 3, 1)].astype(np.int32)          # distinct nodes with a loop
    ei = np.concatenate([ei, np.stack([loops, loops])], axis=1)
    ei = ei[:, rng.permutation(ei.shape[1])]
    w = (rng.random(ei.shape[1]).astype(np.float32) + 0.5) if with_w else None
    gi, gw = add_remaining_self_loops(to_gpu(ei), to_gpu(w) if with_w else None, fill, V)
    oi, ow = oracle.add_remaining_self_loops(ei, w, fill, V)
    assert gi.dtype == torch.int32 and np.array_equal(gi.cpu().numpy(), oi)
    if with_w:
        assert np.array_equal(gw.cpu().numpy().view(np.int32), ow.view(np.int32))
    else:
        assert gw is None and ow is None
    # int64 indices come back as int64
    gi64, _ = add_remaining_self_loops(to_gpu(ei).long(), None, fill, V)
    assert gi64.dtype == torch.int64 and np.array_equal(gi64.cpu().numpy(), oi)


def test_norms_with_existing_weighted_loops_and_flags():
    from jittorgeometric_amd.nn import gcn_norm, sage_norm
    rng = np.random.default_rng(17)
    V, E = 3000, 50000
    ei = rng.integers(0, V, (2, E)).astype(np.int32)
    ei = ei[:, ei[0] != ei[1]]
    loops = rng.permutation(V)[:700].astype(np.int32)
    ei = np.concatenate([ei[:, :20000], np.stack([loops, loops]), ei[:, 20000:]], axis=1)
    w = rng.random(ei.shape[1]).astype(np.float32) + 0.5
    for kwargs in ({}, {"improved": True}, {"add_self_loops": False}):
        for fn, ofn in ((gcn_norm, oracle.gcn_norm), (sage_norm, oracle.sage_norm)):
            gi, gw = fn(to_gpu(ei), to_gpu(w), V, **kwargs)
            oi, ow = ofn(ei, w, V, **kwargs)
            assert np.array_equal(gi.cpu().numpy(), oi)
            assert_close(gw.cpu().numpy(), ow, rtol=2e-5, atol=1e-7, what="%s %s" % (fn.__name__, kwargs))


def test_preprocessing_refuses_cpu_tensors():
    from jittorgeometric_amd import _lib
    from jittorgeometric_amd.nn import gcn_norm, sage_norm
    from jittorgeometric_amd.utils import add_remaining_self_loops
    ei = torch.tensor([[0, 1], [1, 0]], dtype=torch.int32)
    for fn in (lambda: gcn_norm(ei, None, 2), lambda: sage_norm(ei, None, 2), lambda: add_remaining_self_loops(ei, None, 1.0, 2)):
        with pytest.raises(_lib.JgamdError):
            fn()


def test_layers_honour_the_reference_grad_switch():
    """With REFERENCE_GRAD set, a layer on its spmm=True route back-propagates through the forward
    product again, as ops/spmmcsr.py:35-39 does; the fused layer paths step aside for it."""
    from jittorgeometric_amd.nn import SAGEConv, sage_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr, spmmcsr
    from jittorgeometric_amd import synthetic
    V = 2000
    ei = synthetic.chung_lu(V, 30000, 2.1, max_degree=500, seed=4)
    eit, wt = sage_norm(to_gpu(ei), None, V)
    oei, ow = oracle.sage_norm(ei, None, V)
    csc, csr = cootocsc(eit, wt, V), cootocsr(eit, wt, V)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((V, 32)).astype(np.float32)
    g = rng.standard_normal((V, 16)).astype(np.float32)
    torch.manual_seed(1)
    layer = SAGEConv(32, 16, root_weight=False, bias=False, spmm=True).to(dev())
    A = dense_adj(oei, ow, V).numpy()
    gW = g.astype(np.float64) @ layer.weight1.detach().cpu().double().numpy().T
    try:
        for flag, want in ((False, A.T @ gW), (True, A @ gW)):
            spmmcsr.REFERENCE_GRAD = flag
            xt = to_gpu(x).requires_grad_(True)
            layer(xt, csc=csc, csr=csr).backward(to_gpu(g))
            assert_close(xt.grad.cpu().numpy(), want, np.abs(want) + np.abs(want).mean(), rtol=1e-4,
                         what="REFERENCE_GRAD=%s" % flag)
    finally:
        spmmcsr.REFERENCE_GRAD = False


@pytest.mark.parametrize("spmm", [False, True])
def test_gcn_aggregate_first_is_the_same_layer(spmm):
    """(A x) W + b against A (x W) + b, the reference's order (gcn_conv.py:95-101): same
    output and gradients up to rounding, checked against a float64 dense model."""
    from jittorgeometric_amd.nn import GCNConv, gcn_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from jittorgeometric_amd import synthetic
    V = 5000
    ei = synthetic.chung_lu(V, 70000, 2.1, max_degree=900, seed=12)
    eit, wt = gcn_norm(to_gpu(ei), None, V)
    csc, csr = cootocsc(eit.contiguous(), wt, V), cootocsr(eit.contiguous(), wt, V)
    oei, ow = oracle.gcn_norm(ei, None, V)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((V, 100)).astype(np.float32)
    g = rng.standard_normal((V, 256)).astype(np.float32)
    torch.manual_seed(2)
    ref_layer = GCNConv(100, 256, spmm=spmm).to(dev())
    with torch.no_grad():
        ref_layer.bias.normal_(0, 0.2)
    layer = GCNConv(100, 256, spmm=spmm, aggregate_first=True).to(dev())
    layer.load_state_dict(ref_layer.state_dict())
    A = dense_adj(oei, ow, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W = layer.weight.detach().cpu().double().requires_grad_(True)
    b = layer.bias.detach().cpu().double().requires_grad_(True)
    (A @ (x64 @ W) + b).backward(torch.from_numpy(g.astype(np.float64)))
    want_out = (A @ (x64 @ W) + b).detach().numpy()
    for lay in (ref_layer, layer):
        xt = to_gpu(x).requires_grad_(True)
        out = lay(xt, csc, csr)
        out.backward(to_gpu(g))
        assert_close(out.detach().cpu().numpy(), want_out, rtol=1e-4, atol=1e-5, what="out")
        for got, want, name in ((xt.grad, x64.grad, "x"), (lay.weight.grad, W.grad, "W"), (lay.bias.grad, b.grad, "b")):
            want = want.numpy()
            assert_close(got.cpu().numpy(), want, np.abs(want) + np.abs(want).mean(), rtol=1e-4, what="grad " + name)


@pytest.mark.parametrize("root,bias", [(True, True), (False, True), (False, False), (True, False)])
def test_sage_transform_first_is_the_same_layer(root, bias):
    """A (x W1) + x W_root + b against the reference's (A x) W1 + x W_root + b
    (sage_conv.py:172-190): same output and gradients up to rounding, both against a float64
    dense model; the weights are not symmetric, so this also checks the transposed product."""
    from jittorgeometric_amd.nn import SAGEConv, sage_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from jittorgeometric_amd import synthetic
    V = 5000
    ei = synthetic.chung_lu(V, 70000, 2.1, max_degree=900, seed=13)
    eit, wt = sage_norm(to_gpu(ei), None, V)
    csc, csr = cootocsc(eit.contiguous(), wt, V), cootocsr(eit.contiguous(), wt, V)
    oei, ow = oracle.sage_norm(ei, None, V)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((V, 256)).astype(np.float32)
    g = rng.standard_normal((V, 48)).astype(np.float32)
    torch.manual_seed(3)
    ref_layer = SAGEConv(256, 48, root_weight=root, bias=bias, spmm=False).to(dev())
    if bias:
        with torch.no_grad():
            ref_layer.bias.normal_(0, 0.2)
    layer = SAGEConv(256, 48, root_weight=root, bias=bias, spmm=False, transform_first=True).to(dev())
    layer.load_state_dict(ref_layer.state_dict())
    A = dense_adj(oei, ow, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W1 = layer.weight1.detach().cpu().double().requires_grad_(True)
    Wr = layer.root_weight.detach().cpu().double().requires_grad_(True) if root else None
    b = layer.bias.detach().cpu().double().requires_grad_(True) if bias else None
    ref = (A @ x64) @ W1
    if root:
        ref = ref + x64 @ Wr
    if bias:
        ref = ref + b
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    for lay in (ref_layer, layer):
        xt = to_gpu(x).requires_grad_(True)
        out = lay(xt, csc=csc, csr=csr)
        out.backward(to_gpu(g))
        assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=1e-5, what="out")
        pairs = [(xt.grad, x64.grad, "x"), (lay.weight1.grad, W1.grad, "W1")]
        if root:
            pairs.append((lay.root_weight.grad, Wr.grad, "W_root"))
        if bias:
            pairs.append((lay.bias.grad, b.grad, "b"))
        for got, want, name in pairs:
            want = want.numpy()
            assert_close(got.cpu().numpy(), want, np.abs(want) + np.abs(want).mean(), rtol=1e-4, what="grad " + name)


@pytest.mark.parametrize("spmm", [False, True])
@pytest.mark.parametrize("f_in,f_out", [(40, 96), (96, 40), (64, 64)])
def test_gcn_layer_weight_gradient_with_and_without_input_gradient(spmm, f_in, f_out):
    """A layer whose input needs no gradient (the first of a model) may take
    g_W = (A x)^T g instead of x^T (A^T g) when it widens: both against a dense float64
    model, and against each other, on a directed graph with asymmetric weights."""
    from jittorgeometric_amd.nn import GCNConv
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from util import rand_graph
    rng = np.random.default_rng(41)
    V, E = 6000, 70000                       # above the row count from which the matrix-core kernel is used
    ei, w = rand_graph(rng, V, E, hubs=3)
    x = rng.standard_normal((V, f_in)).astype(np.float32)
    g = rng.standard_normal((V, f_out)).astype(np.float32)
    csc, csr = cootocsc(to_gpu(ei), to_gpu(w), V), cootocsr(to_gpu(ei), to_gpu(w), V)
    torch.manual_seed(3)
    layer = GCNConv(f_in, f_out, spmm=spmm).to(dev())
    with torch.no_grad():
        layer.bias.normal_(0, 0.1)
    grads = []
    for needs in (True, False):
        layer.zero_grad(set_to_none=True)
        xt = to_gpu(x).requires_grad_(needs)
        out = layer(xt, csc, csr)
        out.backward(to_gpu(g))
        grads.append((layer.weight.grad.clone(), layer.bias.grad.clone(), xt.grad))
    A = dense_adj(ei, w, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W = layer.weight.detach().cpu().double().requires_grad_(True)
    b = layer.bias.detach().cpu().double().requires_grad_(True)
    ref = A @ (x64 @ W) + b
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    # sums of absolute terms of the same chain, for the tolerance
    Aa = A.abs()
    gw_scale = (x64.detach().abs().t() @ (Aa.t() @ torch.from_numpy(np.abs(g).astype(np.float64)))).numpy()
    gx_scale = ((Aa.t() @ torch.from_numpy(np.abs(g).astype(np.float64))) @ W.detach().abs().t()).numpy()
    out_scale = (Aa @ (x64.detach().abs() @ W.detach().abs()) + b.detach().abs()).numpy()
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), out_scale, rtol=2e-5, what="out")
    for (gw, gb, gx), needs in zip(grads, (True, False)):
        assert_close(gw.cpu().numpy(), W.grad.numpy(), gw_scale, rtol=2e-5, what="grad W (input gradient %s)" % needs)
        assert_close(gb.cpu().numpy(), b.grad.numpy(), np.abs(g).sum(0), rtol=2e-5, what="grad b")
        if needs:
            assert_close(gx.cpu().numpy(), x64.grad.numpy(), gx_scale, rtol=2e-5, what="grad x")
        else:
            assert gx is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_gcn_layer_without_bias_on_a_small_graph(dtype):
    """No bias row, fewer rows than the matrix-core kernel takes, and float64 features (narrowed to
    float32 like every other input): the same layer against a dense float64 model."""
    from jittorgeometric_amd.nn import GCNConv
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from util import rand_graph
    rng = np.random.default_rng(43)
    V, E, f_in, f_out = 500, 4000, 24, 40
    ei, w = rand_graph(rng, V, E, hubs=2)
    x = rng.standard_normal((V, f_in)).astype(np.float32)
    g = rng.standard_normal((V, f_out)).astype(np.float32)
    csc, csr = cootocsc(to_gpu(ei), to_gpu(w), V), cootocsr(to_gpu(ei), to_gpu(w), V)
    torch.manual_seed(4)
    layer = GCNConv(f_in, f_out, bias=False, spmm=False).to(dev())
    assert layer.bias is None
    xt = to_gpu(x).to(dtype).requires_grad_(True)
    out = layer(xt, csc, csr)
    assert out.dtype == torch.float32
    out.backward(to_gpu(g))
    assert xt.grad.dtype == dtype
    A = dense_adj(ei, w, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W = layer.weight.detach().cpu().double().requires_grad_(True)
    ref = A @ (x64 @ W)
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    g64 = torch.from_numpy(np.abs(g).astype(np.float64))
    Aa = A.abs()
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), (Aa @ (x64.detach().abs() @ W.detach().abs())).numpy(),
                 rtol=2e-5, what="out")
    assert_close(layer.weight.grad.cpu().numpy(), W.grad.numpy(), (x64.detach().abs().t() @ (Aa.t() @ g64)).numpy(),
                 rtol=2e-5, what="grad W")
    assert_close(xt.grad.cpu().numpy(), x64.grad.numpy(), ((Aa.t() @ g64) @ W.detach().abs().t()).numpy(), rtol=2e-5,
                 what="grad x")


def test_training_loop_follows_a_dense_float64_model():
    """The training loop of examples/gcn_example.py:48-59,96-115 (two GCN layers, relu, mean
    cross-entropy, Adam with weight decay) for 25 steps on the small configuration: the loss
    of every step follows a dense float64 model started from the same parameters.  The graph
    structures are built once and reused while the optimiser updates the parameters in place."""
    from jittorgeometric_amd.nn import GCNConv, cross_entropy_loss, gcn_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    ei, V, x, y = cora_like()
    eit, wt = gcn_norm(to_gpu(ei), None, V)
    oei, ow = oracle.gcn_norm(ei, None, V)
    csc, csr = cootocsc(eit, wt, V), cootocsr(eit, wt, V)
    torch.manual_seed(11)
    l1, l2 = GCNConv(1433, 64).to(dev()), GCNConv(64, 7).to(dev())
    params = list(l1.parameters()) + list(l2.parameters())
    ref_params = [p.detach().cpu().double().requires_grad_(True) for p in params]
    opt = torch.optim.Adam(params, lr=0.01, weight_decay=5e-4)
    ref_opt = torch.optim.Adam(ref_params, lr=0.01, weight_decay=5e-4)
    A = dense_adj(oei, ow, V)
    xt, yt = to_gpu(x), to_gpu(y)
    x64, y64 = torch.from_numpy(x.astype(np.float64)), torch.from_numpy(y)
    losses, ref_losses = [], []
    for _ in range(25):
        opt.zero_grad(set_to_none=True)
        loss = cross_entropy_loss(l2(torch.relu(l1(xt, csc, csr)), csc, csr), yt)
        loss.backward()
        opt.step()
        losses.append(loss.item())
        ref_opt.zero_grad(set_to_none=True)
        W1, b1, W2, b2 = ref_params
        ref = torch.nn.functional.cross_entropy(A @ (torch.relu(A @ (x64 @ W1) + b1) @ W2) + b2, y64)
        ref.backward()
        ref_opt.step()
        ref_losses.append(ref.item())
    assert losses[-1] < losses[0], losses                     # random labels: slowly, but it goes down
    assert np.allclose(losses, ref_losses, rtol=2e-4, atol=0), (losses, ref_losses)
    # (single parameters are not compared: Adam divides by the running gradient magnitude, so an
    # entry whose gradient is rounding noise moves by the learning rate in either model)


@pytest.mark.parametrize("root", [False, True])
def test_sage_training_loop_through_the_edge_list_route(root):
    """The model of examples/sage_example.py:57-69 (two SAGEConv layers called with the edge list,
    cached=True so that normalisation and conversion happen once, relu between, log-softmax +
    nll loss), 15 plain gradient steps against a dense float64 model.  Both layers narrow, so
    their backward passes take the transposed product at the output width."""
    from jittorgeometric_amd.nn import SAGEConv, nll_loss
    from jittorgeometric_amd import synthetic
    V, f_in, hid, C = 6000, 96, 48, 7                  # above the row count from which the matrix-core kernel is used
    ei = synthetic.chung_lu(V, 60000, 2.1, max_degree=900, seed=31)
    rng = np.random.default_rng(32)
    x = rng.standard_normal((V, f_in)).astype(np.float32)
    y = rng.integers(0, C, V)
    oei, ow = oracle.sage_norm(ei, None, V)
    A = dense_adj(oei, ow, V)
    torch.manual_seed(33)
    l1 = SAGEConv(f_in, hid, cached=True, root_weight=root).to(dev())
    l2 = SAGEConv(hid, C, cached=True, root_weight=root).to(dev())
    params = list(l1.parameters()) + list(l2.parameters())
    names = [n for n, _ in l1.named_parameters()]
    ref_params = [p.detach().cpu().double().requires_grad_(True) for p in params]
    opt, ref_opt = torch.optim.SGD(params, lr=0.3), torch.optim.SGD(ref_params, lr=0.3)
    xt, yt, eit = to_gpu(x), to_gpu(y), to_gpu(ei)
    x64, y64 = torch.from_numpy(x.astype(np.float64)), torch.from_numpy(y)
    n = len(names)

    def ref_layer(h, ps):
        p = dict(zip(names, ps))
        out = (A @ h) @ p["weight1"]
        if root:
            out = out + h @ p["root_weight"]
        return out + p["bias"]

    losses, ref_losses = [], []
    for _ in range(15):
        opt.zero_grad(set_to_none=True)
        out = l2(torch.relu(l1(xt, eit)), eit)
        loss = nll_loss(torch.log_softmax(out, dim=1), yt)
        loss.backward()
        opt.step()
        losses.append(loss.item())
        ref_opt.zero_grad(set_to_none=True)
        ref_out = ref_layer(torch.relu(ref_layer(x64, ref_params[:n])), ref_params[n:])
        ref = torch.nn.functional.nll_loss(torch.log_softmax(ref_out, dim=1), y64)
        ref.backward()
        ref_opt.step()
        ref_losses.append(ref.item())
    assert l1._cached_edge_index is not None and losses[-1] < losses[0], losses
    assert np.allclose(losses, ref_losses, rtol=1e-4, atol=0), (losses, ref_losses)
    for p, q in zip(params, ref_params):
        q = q.detach().numpy()
        assert_close(p.detach().cpu().numpy(), q, np.abs(q) + np.abs(q).mean(), rtol=1e-4, what="parameters after 15 steps")


@pytest.mark.parametrize("spmm,bias", [(False, True), (True, True), (False, False)])
@pytest.mark.parametrize("f_in,f_out", [(48, 96), (96, 47)])
def test_gcn_layer_with_the_activation_in_its_row_store_is_relu_of_the_layer(spmm, bias, f_in, f_out):
    """GCNConv(activation="relu") = relu(GCNConv(...)) as examples/gcn_example.py:84-90 writes it:
    same output and same gradients bit for bit (the clamp and its mask are exact operations), and
    both within tolerance of a dense float64 model."""
    from jittorgeometric_amd.nn import GCNConv, gcn_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from util import rand_graph
    rng = np.random.default_rng(f_in + 3 * f_out)
    V, E = 6000, 90000
    ei, _ = rand_graph(rng, V, E, 2)
    ei_g, w_g = gcn_norm(to_gpu(ei), None, V)
    csc, csr = cootocsc(ei_g, w_g, V), cootocsr(ei_g, w_g, V)
    torch.manual_seed(3)
    plain = GCNConv(f_in, f_out, bias=bias, spmm=spmm).to(dev())
    fused = GCNConv(f_in, f_out, bias=bias, spmm=spmm, activation="relu").to(dev())
    fused.load_state_dict(plain.state_dict())
    if bias:
        with torch.no_grad():
            plain.bias.copy_(torch.randn(f_out, device=dev()) * 0.1)
            fused.bias.copy_(plain.bias)
    x = rng.standard_normal((V, f_in)).astype(np.float32)
    g = rng.standard_normal((V, f_out)).astype(np.float32)
    xa, xb = to_gpu(x).requires_grad_(True), to_gpu(x).requires_grad_(True)
    out_a = torch.relu(plain(xa, csc, csr))
    out_b = fused(xb, csc, csr)
    assert torch.equal(out_a, out_b) and (out_b >= 0).all() and (out_b == 0).any()
    out_a.backward(to_gpu(g))
    out_b.backward(to_gpu(g))
    assert torch.equal(xa.grad, xb.grad) and torch.equal(plain.weight.grad, fused.weight.grad)
    if bias:
        assert torch.equal(plain.bias.grad, fused.bias.grad)
    # dense float64 model of relu(A (x W) + b)
    A = dense_adj(ei_g.cpu().numpy(), w_g.cpu().numpy(), V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W64 = plain.weight.detach().cpu().double().requires_grad_(True)
    pre = A @ (x64 @ W64) + (plain.bias.detach().cpu().double() if bias else 0)
    torch.relu(pre).backward(torch.from_numpy(g.astype(np.float64)))
    scale = (A.abs() @ (x64.detach().abs() @ W64.detach().abs())).numpy() + 1
    near_zero = np.abs(pre.detach().numpy()) < 1e-4 * scale       # the mask may flip where the pre-activation is ~0
    assert_close(np.where(near_zero, 0, out_b.detach().cpu().numpy()), np.where(near_zero, 0, torch.relu(pre).detach().numpy()),
                 scale, what="activated output")
    if not near_zero.any():
        assert_close(fused.weight.grad.cpu().numpy(), W64.grad.numpy(), rtol=1e-4, atol=1e-4, what="weight gradient")


@pytest.mark.parametrize("R,F", [(1, 1), (5000, 47), (70000, 128), (3000, 602), (2049, 256)])
def test_relu_backward_with_column_sum_in_one_pass(R, F):
    from jittorgeometric_amd.nn.dense import column_sum, relu_backward_column_sum
    rng = np.random.default_rng(R + F)
    g = to_gpu(rng.standard_normal((R, F)).astype(np.float32))
    y = to_gpu(np.maximum(rng.standard_normal((R, F)), 0).astype(np.float32))
    masked, gb = relu_backward_column_sum(g, y)
    want = g * (y > 0)
    assert torch.equal(masked, want)
    assert torch.equal(gb, column_sum(want))                       # the same sums in the same order
    assert_close(gb.cpu().numpy(), want.double().sum(0).cpu().numpy(), want.abs().double().sum(0).cpu().numpy(),
                 what="bias gradient behind a relu")


@pytest.mark.parametrize("root,f_in,f_out", [(True, 64, 96), (False, 100, 48)])
def test_sage_layer_with_the_activation_in_its_store_is_relu_of_the_layer(root, f_in, f_out):
    """SAGEConv(activation="relu") = relu(SAGEConv(...)), outputs and gradients bit for bit."""
    from jittorgeometric_amd.nn import SAGEConv, sage_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from util import rand_graph
    rng = np.random.default_rng(f_in + f_out)
    V, E = 6000, 80000
    ei, _ = rand_graph(rng, V, E, 2)
    ei_g, w_g = sage_norm(to_gpu(ei), None, V)
    csc, csr = cootocsc(ei_g, w_g, V), cootocsr(ei_g, w_g, V)
    torch.manual_seed(4)
    plain = SAGEConv(f_in, f_out, root_weight=root, spmm=False).to(dev())
    fused = SAGEConv(f_in, f_out, root_weight=root, spmm=False, activation="relu").to(dev())
    fused.load_state_dict(plain.state_dict())
    x = rng.standard_normal((V, f_in)).astype(np.float32)
    g = to_gpu(rng.standard_normal((V, f_out)).astype(np.float32))
    xa, xb = to_gpu(x).requires_grad_(True), to_gpu(x).requires_grad_(True)
    out_a = torch.relu(plain(xa, None, None, csc, csr))
    out_b = fused(xb, None, None, csc, csr)
    assert torch.equal(out_a, out_b) and (out_b == 0).any()
    out_a.backward(g)
    out_b.backward(g)
    assert torch.equal(xa.grad, xb.grad) and torch.equal(plain.weight1.grad, fused.weight1.grad)
    assert torch.equal(plain.bias.grad, fused.bias.grad)
    if root:
        assert torch.equal(plain.root_weight.grad, fused.root_weight.grad)


@pytest.mark.parametrize("spmm,lam,weighted", [(True, 0.0, False), (False, 0.3, False), (True, 0.3, True)])
def test_clustergcn_layer(spmm, lam, weighted):
    """clustergcn_norm's weights are asymmetric on an irregular graph (scaled by the source's
    degree only), so the backward must be the true transpose, as for SAGEConv."""
    from jittorgeometric_amd.nn import ClusterGCNConv, clustergcn_norm
    from jittorgeometric_amd import synthetic
    V = 3000
    ei = synthetic.chung_lu(V, 40000, 2.1, max_degree=800, seed=19)
    rng = np.random.default_rng(3)
    w = (rng.random(ei.shape[1]) + 0.5).astype(np.float32) if weighted else None
    x = rng.standard_normal((V, 64)).astype(np.float32)
    g = rng.standard_normal((V, 24)).astype(np.float32)
    eit, wt = clustergcn_norm(to_gpu(ei), None if w is None else to_gpu(w), V, diag_lambda=lam)
    oei, ow = oracle.clustergcn_norm(ei, w, V, diag_lambda=lam)
    assert np.array_equal(eit.cpu().numpy(), oei)
    assert_close(wt.cpu().numpy(), ow, rtol=2e-6, atol=0)
    torch.manual_seed(1)
    layer = ClusterGCNConv(64, 24, diag_lambda=lam, spmm=spmm, cached=True).to(dev())
    with torch.no_grad():
        layer.bias.copy_(to_gpu(rng.standard_normal(24).astype(np.float32)))
    xt = to_gpu(x).requires_grad_(True)
    out = layer(xt, to_gpu(ei), None if w is None else to_gpu(w))
    out.backward(to_gpu(g))
    again = layer(to_gpu(x), None, None)                      # from the cached arrays
    assert torch.equal(again, out.detach())
    params = [p.detach().cpu().numpy() for p in (layer.weight_out, layer.weight_root, layer.bias)]
    want = oracle.clustergcn_conv(x, oracle.cootocsc(oei, ow, V), *params)
    assert_close(out.detach().cpu().numpy(), want, rtol=1e-4, atol=1e-5, what="against the oracle")

    A = dense_adj(oei, ow, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    Wo, Wr, b = [torch.from_numpy(p.astype(np.float64)).requires_grad_(True) for p in params]
    ref = (A @ x64) @ Wo + x64 @ Wr + b
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=1e-5, what="out")
    for got, want, name in ((xt.grad, x64.grad, "x"), (layer.weight_out.grad, Wo.grad, "W_out"),
                            (layer.weight_root.grad, Wr.grad, "W_root"), (layer.bias.grad, b.grad, "bias")):
        want = want.numpy()
        assert_close(got.cpu().numpy(), want, np.abs(want) + np.abs(want).max() * 1e-2, rtol=1e-4, what="grad " + name)


@pytest.mark.parametrize("normalization", [None, "sym", "rw"])
def test_get_laplacian(normalization):
    from jittorgeometric_amd.utils import get_laplacian
    from jittorgeometric_amd import synthetic
    V = 4000
    ei = synthetic.chung_lu(V, 50000, 2.1, max_degree=900, seed=29)
    rng = np.random.default_rng(4)
    loops = np.stack([rng.integers(0, V, 50)] * 2).astype(ei.dtype)          # a few self-loops: dropped
    ei = np.concatenate([ei[:, :20000], loops, ei[:, 20000:]], axis=1)
    ei[:, 100:110] = V - 1 - np.arange(10)[None, :]                          # more loops, in the middle
    for w in (None, (rng.random(ei.shape[1]) + 0.5).astype(np.float32)):
        gi, gw = get_laplacian(to_gpu(ei), None if w is None else to_gpu(w), normalization, num_nodes=V)
        oi, ow = oracle.get_laplacian(ei, w, normalization, V)
        assert np.array_equal(gi.cpu().numpy(), oi)
        # the degree is a sum of up to 900 weights: fixed order here, numpy's own order in the oracle
        assert_close(gw.cpu().numpy(), ow, rtol=1e-5 if w is not None else 2e-6, atol=0)
    # nodes without an outgoing edge: D^-1/2 = inf becomes 0
    few = np.array([[0, 1, 2], [1, 2, 0]], np.int32)
    gi, gw = get_laplacian(to_gpu(few), None, normalization, num_nodes=6)
    oi, ow = oracle.get_laplacian(few, None, normalization, 6)
    assert np.array_equal(gi.cpu().numpy(), oi) and np.array_equal(gw.cpu().numpy(), ow)


@pytest.mark.parametrize("K,normalization,lam", [(1, "sym", None), (2, "sym", None), (4, "sym", 2.5), (3, "rw", None),
                                                 (3, None, 40.0)])
def test_cheb_conv(K, normalization, lam):
    """The reference sends norm_e * x[src] messages; here the scaled Laplacian is a compressed
    matrix and every recurrence step one product with `2 * ... - T_{k-2}` in its row store."""
    from jittorgeometric_amd.nn import ChebConv
    from jittorgeometric_amd import synthetic
    V, Fin, Fout = 2500, 32, 12
    ei = synthetic.chung_lu(V, 30000, 2.1, max_degree=600, seed=39)
    rng = np.random.default_rng(6)
    w = (rng.random(ei.shape[1]) + 0.5).astype(np.float32)
    x = rng.standard_normal((V, Fin)).astype(np.float32)
    g = rng.standard_normal((V, Fout)).astype(np.float32)
    torch.manual_seed(2)
    layer = ChebConv(Fin, Fout, K, normalization=normalization).to(dev())
    with torch.no_grad():
        layer.bias.copy_(to_gpu(rng.standard_normal(Fout).astype(np.float32)))
    ei_g, w_g = to_gpu(ei), to_gpu(w)
    xt = to_gpu(x).requires_grad_(True)
    out = layer(xt, ei_g, w_g, None, lam)
    out.backward(to_gpu(g))
    assert torch.equal(layer(to_gpu(x), ei_g, w_g, None, lam), out.detach())           # from the kept conversion
    Ws = [lin.weight.detach().cpu().numpy().T for lin in layer.lins]                     # [in, out]
    b = layer.bias.detach().cpu().numpy()
    want = oracle.cheb_conv(x, ei, Ws, b, w, normalization, lam)
    assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-4 * np.abs(want).max()

    ni, nw = oracle.cheb_norm(ei, V, w, normalization, lam)
    L = dense_adj(ni, nw, V)
    x64 = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    W64 = [torch.from_numpy(W.astype(np.float64)).requires_grad_(True) for W in Ws]
    b64 = torch.from_numpy(b.astype(np.float64)).requires_grad_(True)
    t0 = t1 = x64
    ref = t0 @ W64[0]
    if K > 1:
        t1 = L @ x64
        ref = ref + t1 @ W64[1]
    for k in range(2, K):
        t0, t1 = t1, 2 * (L @ t1) - t0
        ref = ref + t1 @ W64[k]
    ref = ref + b64
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    scale = np.abs(ref.detach().numpy()).max()
    assert np.abs(out.detach().cpu().numpy() - ref.detach().numpy()).max() <= 1e-4 * scale
    pairs = [(xt.grad, x64.grad, "x"), (layer.bias.grad, b64.grad, "bias")] + \
            [(lin.weight.grad.t(), W.grad, "W%d" % k) for k, (lin, W) in enumerate(zip(layer.lins, W64))]
    for got, ref_g, name in pairs:
        ref_g = ref_g.numpy()
        assert np.abs(got.cpu().numpy() - ref_g).max() <= 2e-4 * np.abs(ref_g).max(), name
    # other edge tensors: the conversion is redone
    ei2 = to_gpu(ei[:, :20000].copy())
    out2 = layer(to_gpu(x), ei2, to_gpu(w[:20000].copy()), None, lam)
    want2 = oracle.cheb_conv(x, ei[:, :20000], Ws, b, w[:20000], normalization, lam)
    assert np.abs(out2.detach().cpu().numpy() - want2).max() <= 1e-4 * np.abs(want2).max()
