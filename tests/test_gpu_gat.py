"""Fused GAT kernels against (a) the oracle's composition of the reference's
CPU loops (forward), (b) a plain PyTorch fp64 model of the same layer
(forward and gradients), (c) the unfused operator chain on the GPU."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def torch_reference(h, a_src, a_dst, src, dst, V, slope=0.2):
    """fp64 CPU model: logits, segment softmax by destination, weighted sum."""
    z = (h[src] * a_src).sum(-1) + (h[dst] * a_dst).sum(-1)            # [E,H]
    z = torch.nn.functional.leaky_relu(z, slope)
    H = z.shape[1]
    idx = dst.view(-1, 1).expand(-1, H)
    zmax = torch.full((V, H), -float("inf"), dtype=z.dtype).scatter_reduce(0, idx, z, "amax", include_self=True)
    p = torch.exp(z - zmax[dst])
    den = torch.zeros((V, H), dtype=z.dtype).index_add(0, dst, p)
    alpha = p / den[dst]
    out = torch.zeros_like(h).index_add(0, dst, alpha.unsqueeze(-1) * h[src])
    return out, alpha


def alpha_weighted_abs(alpha, h, row, dst, V):
    """sum over a destination's in-edges of alpha * |h[src]| (fp64): the sum of absolute
    terms of every element of the layer's output."""
    a = torch.from_numpy(np.asarray(alpha, dtype=np.float64))
    habs = torch.from_numpy(np.abs(h).astype(np.float64))
    out = torch.zeros((V,) + tuple(habs.shape[1:]), dtype=torch.float64)
    return out.index_add(0, torch.from_numpy(dst.astype(np.int64)),
                         a.unsqueeze(-1) * habs[torch.from_numpy(row.astype(np.int64))]).numpy()


def grad_term_sums(h64, a_src, a_dst, alpha, g, row, dst, V, slope=0.2):
    """Sums of the absolute values of the terms that make up each gradient element
    (fp64, from the fp64 model's own quantities): what a rounding error of the fp32
    kernels scales with when the signed terms cancel.
      g_h[u]   = sum_{e: src=u} alpha_e g[dst_e]  +  a_src * sum_{e: src=u} dz_e  +  a_dst * sum_{e: dst=u} dz_e
      g_a_src  = sum_e dz_e h[src_e],   g_a_dst = sum_e dz_e h[dst_e]
      dz_e     = leaky'(z_e) * alpha_e * (g[dst_e].h[src_e] - sum_e' alpha_e' g[dst].h[src_e'])
    """
    h = h64.detach()
    g = torch.from_numpy(g.astype(np.float64))
    gh_dot = (g[dst] * h[row]).sum(-1)                                  # [E,H]
    gh_abs = (g[dst].abs() * h[row].abs()).sum(-1)
    mix = torch.zeros((V, gh_dot.shape[1]), dtype=torch.float64).index_add(0, dst, alpha * gh_abs)
    dz_abs = alpha * (gh_abs + mix[dst])                                # |leaky'| <= 1
    terms_h = torch.zeros_like(h).index_add(0, row, alpha.unsqueeze(-1) * g[dst].abs())
    terms_h += a_src.detach().abs() * torch.zeros((V, dz_abs.shape[1]), dtype=torch.float64).index_add(
        0, row, dz_abs).unsqueeze(-1)
    terms_h += a_dst.detach().abs() * torch.zeros((V, dz_abs.shape[1]), dtype=torch.float64).index_add(
        0, dst, dz_abs).unsqueeze(-1)
    terms_as = (dz_abs.unsqueeze(-1) * h[row].abs()).sum(0)
    terms_ad = (dz_abs.unsqueeze(-1) * h[dst].abs()).sum(0)
    return terms_h.numpy(), terms_as.numpy(), terms_ad.numpy()


def check_against_fp64(alpha, out, g_h, g_as, g_ad, ref, ref_alpha, h64, as64, ad64, g, row, dst, V):
    """Forward and the three gradients against the fp64 model at 1e-5 relative to the
    sums of absolute terms, 1e-6 absolute (1e-7 for attention values, which lie in (0, 1])."""
    row_t, dst_t = torch.from_numpy(row.astype(np.int64)), torch.from_numpy(dst.astype(np.int64))
    ra = ref_alpha.detach()
    hs = torch.zeros_like(h64.detach()).index_add(0, dst_t, ra.unsqueeze(-1) * h64.detach().abs()[row_t]).numpy()
    if alpha is not None:
        assert_close(alpha.cpu().numpy(), ra.numpy(), rtol=1e-5, atol=1e-7, what="alpha")
    assert_close(out.detach().cpu().numpy(), ref.detach().numpy(), hs, what="out")
    th, tas, tad = grad_term_sums(h64, as64, ad64, ra, g, row_t, dst_t, V)
    assert_close(g_h.cpu().numpy(), h64.grad.numpy(), th, what="grad h")
    assert_close(g_as.cpu().numpy(), as64.grad.numpy(), tas, what="grad a_src")
    assert_close(g_ad.cpu().numpy(), ad64.grad.numpy(), tad, what="grad a_dst")


def run_case(V, E, H, D, hubs, seed, check_oracle=True):
    from jittorgeometric_amd.ops import cootocsc, gat_aggregate
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs, hub_share=0.5)
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    row, off, _ = oracle.cootocsc(ei, w, V)
    dst = np.repeat(np.arange(V), np.diff(off))
    h = rng.standard_normal((V, H, D)).astype(np.float32)
    a_src = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    a_dst = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    g = rng.standard_normal((V, H, D)).astype(np.float32)

    ht, ast, adt = (to_gpu(t).requires_grad_(True) for t in (h, a_src, a_dst))
    out = gat_aggregate(ht, csc, ast, adt, 0.2)
    out.backward(to_gpu(g))
    raw = gat_forward_raw(to_gpu(h), csc, to_gpu(a_src), to_gpu(a_dst), 0.2, want_alpha=True)
    torch.cuda.synchronize()

    h64, as64, ad64 = (torch.from_numpy(t.astype(np.float64)).requires_grad_(True) for t in (h, a_src, a_dst))
    ref, ref_alpha = torch_reference(h64, as64, ad64, torch.from_numpy(row.astype(np.int64)),
                                     torch.from_numpy(dst.astype(np.int64)), V)
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    # forward: alpha in (0,1]; out is a convex combination of |h| rows
    hs = torch.zeros((V, H, D), dtype=torch.float64).index_add(
        0, torch.from_numpy(dst.astype(np.int64)), ref_alpha.detach().unsqueeze(-1) * h64.detach().abs()[row]).numpy()
    check_against_fp64(raw["alpha"], out, ht.grad, ast.grad, adt.grad, ref, ref_alpha, h64, as64, ad64, g, row, dst, V)
    # the forward alone, as a caller without a backward pass runs it: no el / er arrays, the scores
    # are taken inside the aggregation kernel where its lane layout allows (else in a workspace)
    inf = gat_forward_raw(to_gpu(h), csc, to_gpu(a_src), to_gpu(a_dst), 0.2)
    assert inf["el"] is None and inf["er"] is None and raw["el"] is not None
    assert_close(inf["out"].cpu().numpy(), ref.detach().numpy(), hs, what="out of the forward without el / er")
    finite = lambda t: np.nan_to_num(t.cpu().numpy(), neginf=-1e30)       # destinations without entries hold -inf
    assert_close(finite(inf["smax"]), finite(raw["smax"]), rtol=1e-5, atol=1e-6, what="smax")
    assert_close(inf["ssum"].cpu().numpy(), raw["ssum"].cpu().numpy(), rtol=1e-4, atol=1e-6, what="ssum")
    with torch.no_grad():
        out_ng = gat_aggregate(to_gpu(h), csc, to_gpu(a_src), to_gpu(a_dst), 0.2)
    assert torch.equal(out_ng, inf["out"])
    if check_oracle:
        # the reference's loops add a destination's terms one by one in fp32, so the
        # oracle itself is only good to about deg * 2^-24 relative on long columns
        o_out, o_alpha = oracle.gat_forward_heads(h, (row, off, None), a_src, a_dst, 0.2)
        slack = 1 + np.diff(off).astype(np.float64) * 6e-3
        assert_close(raw["alpha"].cpu().numpy(), o_alpha, o_alpha * slack[dst][:, None], atol=1e-7,
                     what="alpha vs oracle")
        assert_close(out.detach().cpu().numpy(), o_out, hs * slack[:, None, None], what="out vs oracle")


@pytest.mark.parametrize("V,E,H,D,hubs,seed", [
    (1, 0, 1, 4, 0, 0), (1, 40, 1, 8, 0, 1), (50, 400, 1, 6, 1, 2), (300, 4000, 1, 7, 2, 3),
    (300, 4000, 1, 64, 2, 4), (500, 6000, 1, 256, 2, 5), (400, 5000, 8, 16, 2, 6), (400, 5000, 2, 16, 2, 7),
    (400, 5000, 4, 32, 2, 8), (3000, 100000, 8, 16, 2, 9), (200, 3000, 1, 300, 1, 10), (5000, 2000, 8, 16, 0, 11),
    (300, 3000, 16, 8, 1, 12), (300, 3000, 1, 1, 1, 13),
])
def test_fused_forward_backward(V, E, H, D, hubs, seed):
    run_case(V, E, H, D, hubs, seed)


def test_single_hub_destination_spanning_many_wavefronts():
    from jittorgeometric_amd.ops import cootocsc
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    rng = np.random.default_rng(50)
    V, E, H, D = 1500, 60000, 8, 16
    ei, w = rand_graph(rng, V, E)
    ei[1, :50000] = 7
    ei[0, 50000:58000] = 9                       # and one hub source for the backward pass
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    row, off, _ = oracle.cootocsc(ei, w, V)
    h = rng.standard_normal((V, H, D)).astype(np.float32)
    a_src = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    a_dst = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    raw = gat_forward_raw(to_gpu(h), csc, to_gpu(a_src), to_gpu(a_dst), 0.2, want_alpha=True)
    o_out, o_alpha = oracle.gat_forward_heads(h, (row, off, None), a_src, a_dst, 0.2)
    slack = 1 + np.diff(off).astype(np.float64) * 6e-3
    dst = np.repeat(np.arange(V), np.diff(off))
    assert_close(raw["alpha"].cpu().numpy(), o_alpha, o_alpha * slack[dst][:, None], atol=1e-8, what="alpha")
    assert_close(raw["out"].cpu().numpy(), o_out, alpha_weighted_abs(o_alpha, h, row, dst, V) * slack[:, None, None],
                 what="out")
    run_case(V, E, H, D, 1, 51, check_oracle=False)


def test_gatconv_fused_equals_operator_chain_and_oracle():
    """GATConv with the reference's single head: the fused path, the unfused
    ScatterToEdge/EdgeSoftmax/ScatterToVertex chain and the oracle agree, in
    value and in the gradients of x, W and the attention vector."""
    from jittorgeometric_amd.nn import GATConv
    from jittorgeometric_amd.ops import cootocsc
    rng = np.random.default_rng(60)
    V, E, Fin, C = 800, 9000, 24, 16
    ei, w = rand_graph(rng, V, E, 2)
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    row, off, _ = oracle.cootocsc(ei, w, V)
    x = rng.standard_normal((V, Fin)).astype(np.float32)
    g = rng.standard_normal((V, C)).astype(np.float32)
    torch.manual_seed(1)
    fused = GATConv(Fin, C, E, fused=True).to(dev())
    chain = GATConv(Fin, C, E, fused=False).to(dev())
    chain.load_state_dict(fused.state_dict())
    res = []
    for layer in (fused, chain):
        xt = to_gpu(x).requires_grad_(True)
        out = layer(xt, csc)
        out.backward(to_gpu(g))
        res.append((out.detach().cpu().numpy(), xt.grad.cpu().numpy(), layer.weight.grad.cpu().numpy(),
                    layer.edge_weight.grad.cpu().numpy()))
    hW = np.maximum(x @ fused.weight.detach().cpu().numpy(), 0).astype(np.float32)
    o_out, _, _ = oracle.gat_forward(hW, (row, off, None), fused.edge_weight.detach().cpu().numpy().reshape(-1))
    dst = np.repeat(np.arange(V), np.diff(off))
    _, o_alpha, _ = oracle.gat_forward(hW, (row, off, None), fused.edge_weight.detach().cpu().numpy().reshape(-1))
    terms = alpha_weighted_abs(o_alpha.reshape(-1, 1), hW.reshape(V, 1, C), row, dst, V).reshape(V, C)
    slack = 1 + np.diff(off).astype(np.float64)[:, None] * 6e-3      # the oracle's own sequential fp32 sums
    assert_close(res[0][0], o_out, terms * slack, what="fused vs oracle")
    assert_close(res[1][0], o_out, terms * slack, what="chain vs oracle")
    for a, b, name in zip(res[0][1:], res[1][1:], ("x", "W", "a")):
        assert_close(a, b, np.abs(b) + np.abs(b).mean() * 20 + 1e-3, rtol=1e-4, what="grad " + name)


def test_gat_config3_full_size_forward_and_backward():
    """169,343 nodes, 1.17M power-law edges + self-loops, 8 heads x 16 at full size: every
    destination's attention sums to 1 per head; forward against the oracle's composition of
    the reference loops; forward and the three gradients (h, a_src, a_dst) against the fp64
    model of the layer at 1e-5 relative to the sums of absolute terms."""
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import cootocsc, gat_aggregate
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    ei, V = synthetic.make("gat_169k")
    ei, _ = oracle.add_remaining_self_loops(ei, None, 1.0, V)
    ei = ei.astype(np.int32)
    w = np.ones(ei.shape[1], np.float32)
    csc = cootocsc(to_gpu(ei), to_gpu(w), V)
    rng = np.random.default_rng(3)
    H, D = 8, 16
    h = rng.standard_normal((V, H, D)).astype(np.float32)
    a_src = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    a_dst = (rng.standard_normal((H, D)) / 4).astype(np.float32)
    g = rng.standard_normal((V, H, D)).astype(np.float32)
    raw = gat_forward_raw(to_gpu(h), csc, to_gpu(a_src), to_gpu(a_dst), 0.2, want_alpha=True)
    off = csc.column_offset.long()
    seg = torch.repeat_interleave(torch.arange(V, device=dev()), off[1:] - off[:-1])
    sums = torch.zeros((V, H), device=dev(), dtype=torch.float64).index_add_(0, seg, raw["alpha"].double())
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)
    row, coff, _ = oracle.cootocsc(ei, w, V)
    o_out, o_alpha = oracle.gat_forward_heads(h, (row, coff, None), a_src, a_dst, 0.2)
    slack = 1 + np.diff(coff).astype(np.float64) * 6e-3
    dst = np.repeat(np.arange(V), np.diff(coff))
    assert_close(raw["alpha"].cpu().numpy(), o_alpha, o_alpha * slack[dst][:, None], atol=1e-8, what="alpha vs oracle")
    assert_close(raw["out"].cpu().numpy(), o_out, alpha_weighted_abs(o_alpha, h, row, dst, V) * slack[:, None, None],
                 what="out vs oracle")
    # backward at full size
    ht, ast, adt = (to_gpu(t).requires_grad_(True) for t in (h, a_src, a_dst))
    out = gat_aggregate(ht, csc, ast, adt, 0.2)
    out.backward(to_gpu(g))
    torch.cuda.synchronize()
    h64, as64, ad64 = (torch.from_numpy(t.astype(np.float64)).requires_grad_(True) for t in (h, a_src, a_dst))
    ref, ref_alpha = torch_reference(h64, as64, ad64, torch.from_numpy(row.astype(np.int64)),
                                     torch.from_numpy(dst.astype(np.int64)), V)
    ref.backward(torch.from_numpy(g.astype(np.float64)))
    check_against_fp64(raw["alpha"], out, ht.grad, ast.grad, adt.grad, ref, ref_alpha, h64, as64, ad64, g, row, dst, V)


@pytest.mark.parametrize("fused", [True, False])
def test_gat_training_loop_follows_a_float64_model(fused):
    """Two GATConv layers (the model of examples/gat_example.py:95-106: relu(x W), attention,
    weighted sum; log-softmax + nll loss), 12 plain gradient steps: the loss of every step and the
    parameters at the end follow a float64 model started from the same parameters, through the
    fused kernels and through the unfused operator chain."""
    from jittorgeometric_amd.nn import GATConv, nll_loss
    from jittorgeometric_amd.ops import cootocsc
    from jittorgeometric_amd import synthetic
    V, F_in, C1, C2 = 1500, 48, 16, 5
    ei = synthetic.chung_lu(V, 12000, 2.3, max_degree=300, seed=21)
    loops = np.arange(V, dtype=np.int32)
    ei = np.concatenate([ei[:, ei[0] != ei[1]], np.stack([loops, loops])], axis=1).astype(np.int32)
    E = ei.shape[1]
    rng = np.random.default_rng(22)
    x = rng.standard_normal((V, F_in)).astype(np.float32)
    y = rng.integers(0, C2, V)
    csc = cootocsc(to_gpu(ei), torch.ones(E, device=dev()), V)
    row = csc.row_indices.cpu().numpy().astype(np.int64)
    dst = np.repeat(np.arange(V), np.diff(csc.column_offset.cpu().numpy())).astype(np.int64)
    src_t, dst_t = torch.from_numpy(row), torch.from_numpy(dst)
    torch.manual_seed(23)
    l1, l2 = GATConv(F_in, C1, fused=fused).to(dev()), GATConv(C1, C2, fused=fused).to(dev())
    params = list(l1.parameters()) + list(l2.parameters())
    ref_params = [p.detach().cpu().double().requires_grad_(True) for p in params]
    opt, ref_opt = torch.optim.SGD(params, lr=0.2), torch.optim.SGD(ref_params, lr=0.2)
    xt, yt = to_gpu(x), to_gpu(y)
    x64, y64 = torch.from_numpy(x.astype(np.float64)), torch.from_numpy(y)

    def ref_layer(h_in, W, a):
        C = W.shape[1]
        h = torch.relu(h_in @ W).reshape(V, 1, C)
        out, _ = torch_reference(h, a[:C, 0].reshape(1, C), a[C:, 0].reshape(1, C), src_t, dst_t, V)
        return out.reshape(V, C)

    losses, ref_losses = [], []
    for _ in range(12):
        opt.zero_grad(set_to_none=True)
        out = l2(l1(xt, csc), csc)
        loss = nll_loss(torch.log_softmax(out, dim=1), yt)
        loss.backward()
        opt.step()
        losses.append(loss.item())
        ref_opt.zero_grad(set_to_none=True)
        W1, a1, W2, a2 = ref_params
        ref = torch.nn.functional.nll_loss(torch.log_softmax(ref_layer(ref_layer(x64, W1, a1), W2, a2), dim=1), y64)
        ref.backward()
        ref_opt.step()
        ref_losses.append(ref.item())
    assert losses[-1] < losses[0], losses
    assert np.allclose(losses, ref_losses, rtol=1e-4, atol=0), (losses, ref_losses)
    for p, q in zip(params, ref_params):
        q = q.detach().numpy()
        assert_close(p.detach().cpu().numpy(), q, np.abs(q) + np.abs(q).mean(), rtol=1e-4, what="parameters after 12 steps")
