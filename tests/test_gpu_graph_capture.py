"""The entry points neither allocate, nor synchronise, nor clear memory with memset calls, so a
sequence of them can be recorded into a HIP graph and replayed.  Every replay is checked against
the eager result, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def test_two_layer_gcn_and_appnp_replay_as_a_graph():
    from jittorgeometric_amd.nn import APPNP, GCNConv
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    rng = np.random.default_rng(5)
    V, F = 2708, 64
    ei, _ = rand_graph(rng, V, 10556, 1)
    ei = ei[:, ei[0] != ei[1]]
    ei, w = oracle.gcn_norm(ei, None, V)
    csc = cootocsc(to_gpu(ei.astype(np.int32)), to_gpu(w), V)
    csr = cootocsr(to_gpu(ei.astype(np.int32)), to_gpu(w), V)
    l1, l2 = GCNConv(F, 32, spmm=False).to(dev()), GCNConv(32, 7, spmm=False).to(dev())
    prop = APPNP(4, 0.1, spmm=False)

    def model(x):
        with torch.no_grad():
            return prop(l2(torch.relu(l1(x, csc, csr)), csc, csr), csc, csr)

    static_x = torch.randn(V, F, device=dev())
    # warm-up on a side stream, as graph capture requires
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            model(static_x)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = model(static_x)
    for trial in range(4):
        x = torch.randn(V, F, device=dev())
        want = model(x)                      # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, want), "replay %d differs from the eager result" % trial
    # the eager result itself against the oracle
    W1, b1 = l1.weight.detach().cpu().numpy(), l1.bias.detach().cpu().numpy()
    W2, b2 = l2.weight.detach().cpu().numpy(), l2.bias.detach().cpu().numpy()
    csc_o = oracle.cootocsc(ei.astype(np.int32), w, V)
    xh = x.cpu().numpy()
    h = np.maximum(oracle.aggregate_with_weight((xh @ W1).astype(np.float32), csc_o) + b1, 0).astype(np.float32)
    z = (oracle.aggregate_with_weight((h @ W2).astype(np.float32), csc_o) + b2).astype(np.float32)
    ref = oracle.appnp(z, csc_o, 4, 0.1)
    # eight operators in a row (2 dense products, 2 aggregations, 4 hops), each good to 1e-5 of
    # its sum of absolute terms; the same chain on absolute values carries that bound to the end
    abs_csc = (csc_o[0], csc_o[1], np.abs(csc_o[2]))
    ha = (oracle.aggregate_with_weight((np.abs(xh) @ np.abs(W1)).astype(np.float32), abs_csc) + np.abs(b1))
    za = (oracle.aggregate_with_weight((ha @ np.abs(W2)).astype(np.float32), abs_csc) + np.abs(b2)).astype(np.float32)
    assert_close(want.cpu().numpy(), ref, scale=oracle.appnp(za, abs_csc, 4, 0.1), rtol=8e-5)


def test_training_step_replays_as_a_graph():
    """Forward, the library's loss and backward of a 2-layer GCN (the step of
    examples/gcn_example.py:96-115) recorded once and replayed: loss and every gradient of every
    replay equal the eager step's, with eager steps and synchronisations in between."""
    from jittorgeometric_amd.nn import GCNConv, cross_entropy_loss
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    rng = np.random.default_rng(6)
    V, F, C = 2708, 96, 7
    ei, _ = rand_graph(rng, V, 10556, 1)
    ei = ei[:, ei[0] != ei[1]]
    ei, w = oracle.gcn_norm(ei, None, V)
    csc = cootocsc(to_gpu(ei.astype(np.int32)), to_gpu(w), V)
    csr = cootocsr(to_gpu(ei.astype(np.int32)), to_gpu(w), V)
    torch.manual_seed(7)
    l1, l2 = GCNConv(F, 32, spmm=False).to(dev()), GCNConv(32, C, spmm=False).to(dev())
    params = list(l1.parameters()) + list(l2.parameters())
    static_x = torch.randn(V, F, device=dev())
    static_y = torch.randint(0, C, (V,), device=dev())

    def step(x, y):
        for p in params:
            p.grad = None
        loss = cross_entropy_loss(l2(torch.relu(l1(x, csc, csr)), csc, csr), y)
        loss.backward()
        return loss

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            step(static_x, static_y)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_loss = step(static_x, static_y)
    static_grads = [p.grad for p in params]          # written in place by every replay
    for trial in range(4):
        x = torch.randn(V, F, device=dev())
        y = torch.randint(0, C, (V,), device=dev())
        want_loss = step(x, y).clone()               # eager work between the replays
        want = [p.grad.clone() for p in params]
        torch.cuda.synchronize()
        static_x.copy_(x)
        static_y.copy_(y)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_loss, want_loss), "loss of replay %d differs from the eager step" % trial
        for got, ref, p in zip(static_grads, want, params):
            assert torch.equal(got, ref), "a gradient of shape %s differs in replay %d" % (tuple(p.shape), trial)
    assert all(torch.isfinite(g).all() for g in static_grads)
