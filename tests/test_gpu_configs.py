"""The benchmark configurations at their full size, through the operators, against
the CPU oracle.

What the oracle can finish in seconds is compared directly: the conversions (bit
for bit) and, for the products, a sample of output rows that always holds the
rows with the most entries (the hubs) next to random ones, summed by the oracle's
own sequential loop over exactly those rows.  Every row of every product is also held to
float64 sums computed on the GPU with torch operators over the oracle's compressed arrays, and
the transpose identity <A x, g> = <x, A^T g> ties the forward product over the CSC arrays to
the backward product over the CSR arrays.  Layers are checked by
what the reference's call order fixes: a sample of rows of each layer's output
recomputed by the oracle from that layer's input, equal losses and gradients
through the two routes a layer offers (SpmmCsr / aggregateWithWeight), finiteness.

Tolerance: 1e-5 relative to the sum of the absolute terms of each output element
plus 1e-6 absolute, against the exact (float64) row sums.  The oracle's loop adds a
row's terms one after the other in fp32, as the reference does, and on rows of 10^5 -
10^6 entries that sum has itself drifted (0.5 % on a 3.8M-entry row of same-sign terms):
against it the allowance grows by the bound of sequential summation, (entries - 1) * 2^-24
of the sum of absolute terms, and the oracle is held to that same bound against float64."""
import functools

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, to_gpu

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ graphs ---
@functools.lru_cache(maxsize=1)          # one configuration resident at a time
def graph(name, norm):
    """(edge_index, weights, V, oracle CSC, oracle CSR, GPU CSC, GPU CSR) of a configuration
    after gcn_norm / sage_norm with self-loops, all from the same arrays."""
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    ei, V = synthetic.make(name)
    ei, w = (oracle.gcn_norm if norm == "gcn" else oracle.sage_norm)(ei, None, V)
    ei = np.ascontiguousarray(ei.astype(np.int32))
    ocsc = oracle.cootocsc(ei, w, V)
    ocsr = oracle.cootocsr(ei, w, V)
    ei_g, w_g = to_gpu(ei), to_gpu(w)
    csc, csr = cootocsc(ei_g, w_g, V), cootocsr(ei_g, w_g, V)
    return ei, w, V, ocsc, ocsr, csc, csr


def sample_rows(off, seed, n_random=3000, n_hubs=12):
    """The n_hubs rows with the most entries, some empty or single-entry rows, random rows."""
    deg = np.diff(off)
    rng = np.random.default_rng(seed)
    hubs = np.argsort(deg)[-n_hubs:]
    small = np.flatnonzero(deg <= 1)[:50]
    return np.unique(np.concatenate([hubs, small, rng.integers(0, deg.shape[0], n_random), [0, deg.shape[0] - 1]]))


def check_rows(got_rows, src, idx, off, wt, rows, what):
    """got_rows (the kernels' result on `rows`) against the exact row sums and against the
    oracle's sequential fp32 loop."""
    exact, terms = oracle.aggregate_rows_f64(src, idx, off, wt, rows)
    seq = oracle.aggregate_rows(src, idx, off, wt, rows)
    drift = (np.diff(off)[rows].astype(np.float64)[:, None]) * 2.0 ** -24      # sequential fp32 summation
    assert_close(got_rows, exact, terms, what=what + " vs float64")
    assert_close(seq, exact, terms * drift / 1e-5, atol=1e-30, what=what + ": oracle vs float64")
    assert_close(got_rows, seq, terms * (1 + drift / 1e-5), what=what + " vs oracle")


def dot64(a, b, rows=1 << 18):
    """sum(a * b) in float64 without a float64 copy of the whole arrays; also sum(|a| |b|)."""
    s = t = 0.0
    for i in range(0, a.shape[0], rows):
        x, y = a[i:i + rows].double(), b[i:i + rows].double()
        s += (x * y).sum().item()
        t += (x.abs() * y.abs()).sum().item()
    return s, t


def all_rows_f64(x, idx, off, wt, entries=1 << 20):
    """Every row of the product in float64 on the GPU, and the sums of the absolute terms: an
    arbiter that shares nothing with the kernels under test.  The compressed arrays are the
    oracle's; a slice of entries is multiplied out in float64, summed by a running sum along the
    entries, and a row's share of the slice is the difference of that running sum between the
    row's two ends (no atomics, so a row of millions of entries costs what any other does; the
    running sum's rounding, 1e-16 of at most a slice's total, is far below the 1e-6 allowed)."""
    V, F = off.shape[0] - 1, x.shape[1]
    d = dev()
    off_g = torch.from_numpy(off.astype(np.int64)).to(d)
    idx_g, w_g = torch.from_numpy(idx.astype(np.int64)).to(d), torch.from_numpy(wt).to(d).double()
    exact = torch.zeros((V, F), dtype=torch.float64, device=d)
    terms = torch.zeros((V, F), dtype=torch.float64, device=d)
    step = max(1, entries * 64 // max(F, 1))
    zero = torch.zeros((F, 1), dtype=torch.float64, device=d)
    for s in range(0, idx_g.shape[0], step):
        n = min(step, idx_g.shape[0] - s)
        r_lo = int(np.searchsorted(off, s, side="right")) - 1
        r_hi = int(np.searchsorted(off, s + n - 1, side="right")) - 1
        pos = (off_g[r_lo:r_hi + 2] - s).clamp_(0, n)
        # entries along the contiguous dimension: torch's running sum is two orders of magnitude
        # faster that way round
        t = (w_g[s:s + n, None] * x[idx_g[s:s + n]].double()).t().contiguous()
        for acc, val in ((exact, t), (terms, t.abs())):
            run = torch.cat([zero, val.cumsum(1)], dim=1)
            acc[r_lo:r_hi + 1] += (run[:, pos[1:]] - run[:, pos[:-1]]).t()
    return exact, terms


def check_all_rows(got, x, idx, off, wt, what):
    exact, terms = all_rows_f64(x, idx, off, wt)
    err = (got.double() - exact).abs_()
    bad = err > 1e-6 + 1e-5 * terms
    if bad.any():
        r, c = (int(v) for v in torch.nonzero(bad)[0])
        raise AssertionError("%s: %d of %d elements out of tolerance, first at row %d col %d: got %r want %r (terms %r)"
                             % (what, int(bad.sum()), bad.numel(), r, c, float(got[r, c]), float(exact[r, c]),
                                float(terms[r, c])))


def product_checks(name, F, seed):
    """Forward and backward product of one configuration at width F."""
    from jittorgeometric_amd.ops import aggregateWithWeight
    ei, w, V, ocsc, ocsr, csc, csr = graph(name, "gcn")
    gen = torch.Generator(device=dev()).manual_seed(seed)
    x = torch.randn((V, F), device=dev(), generator=gen).requires_grad_(True)
    g = torch.randn((V, F), device=dev(), generator=gen)
    out = aggregateWithWeight(x, csc, csr)
    out.backward(g)
    torch.cuda.synchronize()
    out, gx = out.detach(), x.grad
    assert torch.isfinite(out).all() and torch.isfinite(gx).all()
    lhs, lscale = dot64(out, g)
    rhs, _ = dot64(gx, x.detach())
    assert abs(lhs - rhs) <= 1e-6 * lscale, "transpose identity %s F=%d: %r vs %r" % (name, F, lhs, rhs)
    # every row against float64 sums, then a sample of rows against the oracle's own loop
    check_all_rows(out, x.detach(), *ocsc, what="%s forward F=%d, all rows" % (name, F))
    check_all_rows(gx, g, *ocsr, what="%s backward F=%d, all rows" % (name, F))
    x_h, g_h = x.detach().cpu().numpy(), g.cpu().numpy()
    for label, got, src, (idx, off, wt) in (("forward", out, x_h, ocsc), ("backward", gx, g_h, ocsr)):
        rows = sample_rows(off, seed)
        got_rows = got[torch.from_numpy(rows).to(dev())].cpu().numpy()
        check_rows(got_rows, src, idx, off, wt, rows, "%s %s F=%d" % (name, label, F))


# ------------------------------------------------------------- configuration 2
@pytest.mark.parametrize("F", [32, 64, 256])
def test_config2_products_at_the_other_widths(F):
    product_checks("powerlaw_1m", F, 200 + F)


# ------------------------------------------------------------- configuration 4
@pytest.mark.parametrize("F", [602, 256])
def test_config4_products_at_the_wide_widths(F):
    product_checks("dense_233k", F, 400 + F)


# ------------------------------------------------------------- configuration 5
def test_config5_conversions_bit_exact():
    ei, w, V, ocsc, ocsr, csc, csr = graph("powerlaw_2m4", "gcn")
    assert ei.shape[1] > 120_000_000 and V == 2_449_029
    for got, want in (((csr.column_indices, csr.row_offset, csr.edge_weight), ocsr),
                      ((csc.row_indices, csc.column_offset, csc.edge_weight), ocsc)):
        assert np.array_equal(got[1].cpu().numpy(), want[1])
        assert np.array_equal(got[0].cpu().numpy(), want[0])
        assert np.array_equal(got[2].cpu().numpy().view(np.int32), want[2].view(np.int32))


@pytest.mark.parametrize("F", [100, 256, 47])
def test_config5_products(F):
    product_checks("powerlaw_2m4", F, 500 + F)


def _labels_and_features(V, F_in, n_classes, seed):
    gen = torch.Generator(device=dev()).manual_seed(seed)
    x = torch.randn((V, F_in), device=dev(), generator=gen)
    y = torch.randint(0, n_classes, (V,), device=dev(), generator=gen)
    return x, y


def _layer_rows_check(name, out, lin_in, bias, off_idx_w, rows, what):
    """rows of a layer's aggregation recomputed by the oracle from the layer's own input."""
    idx, off, wt = off_idx_w
    src = lin_in.detach().cpu().numpy()
    got = out.detach()[torch.from_numpy(rows).to(dev())].cpu().numpy().astype(np.float64)
    if bias is not None:
        got = got - bias.detach().cpu().numpy().astype(np.float64)      # one more rounding, within the 1e-6
    check_rows(got, src, idx, off, wt, rows, what)


def test_config5_three_layer_gcn_step():
    """examples/gcn_example.py:48-59,96-115 with three layers 100 -> 256 -> 256 -> 47: one
    full-graph forward + backward through each of the two routes of GCNConv."""
    from jittorgeometric_amd.nn import GCNConv
    ei, w, V, ocsc, ocsr, csc, csr = graph("powerlaw_2m4", "gcn")
    x, y = _labels_and_features(V, 100, 47, 55)
    torch.manual_seed(5)
    dims = [100, 256, 256, 47]
    base = [GCNConv(dims[i], dims[i + 1], spmm=True).to(dev()) for i in range(3)]
    with torch.no_grad():
        for layer in base:
            layer.bias.normal_(0, 0.1)                   # the reference starts from zero biases; any value must work
    rows = sample_rows(ocsc[1], 56, n_random=1500)
    results = []
    for spmm in (True, False):
        layers = [GCNConv(dims[i], dims[i + 1], spmm=spmm).to(dev()) for i in range(3)]
        for a, b in zip(layers, base):
            a.load_state_dict(b.state_dict())
        h = x
        for i, layer in enumerate(layers):
            lin = h @ layer.weight                       # the layer's own dense product, for the oracle
            h_out = layer(h, csc, csr)
            if not results:
                _layer_rows_check("gcn", h_out, lin, layer.bias, ocsc, rows, "GCN layer %d rows" % (i + 1))
            h = torch.relu(h_out) if i < 2 else h_out
        if spmm:
            # the library's loss on these logits against torch's in float64: value and gradient
            from jittorgeometric_amd.nn import cross_entropy_loss
            mine = h.detach().clone().requires_grad_(True)
            cross_entropy_loss(mine, y).backward()
            ref_in = h.detach().double().requires_grad_(True)
            ref = torch.nn.functional.cross_entropy(ref_in, y)
            ref.backward()
            assert abs(cross_entropy_loss(mine, y).item() - ref.item()) <= 1e-5 * abs(ref.item())
            assert (mine.grad.double() - ref_in.grad).abs().max().item() <= 1e-5 / V
            del mine, ref_in, ref
            loss = torch.nn.functional.cross_entropy(h, y)
        else:
            loss = cross_entropy_loss(h, y)              # nn.cross_entropy_loss, examples/gcn_example.py:113
        loss.backward()
        torch.cuda.synchronize()
        grads = [p.grad.clone() for layer in layers for p in layer.parameters()]
        assert all(torch.isfinite(t).all() for t in grads) and torch.isfinite(loss)
        results.append((loss.item(), grads))
    (l0, g0), (l1, g1) = results
    assert abs(l0 - l1) <= 1e-5 * abs(l0), (l0, l1)
    for a, b in zip(g0, g1):
        assert_close(a.cpu().numpy(), b.cpu().numpy(), np.abs(b.cpu().numpy()) + b.abs().mean().item(), rtol=1e-4,
                     what="GCN gradients through the two routes")


def test_config5_three_layer_sage_mean_step():
    """examples/sage_example.py:60-61 (root_weight off, mean weights) with three layers; the
    weights are not symmetric, so the backward product must be the true transpose: the loss and
    the gradients through SpmmCsr (transposed arrays) and aggregateWithWeight (CSC / CSR) agree."""
    from jittorgeometric_amd.nn import SAGEConv
    ei, w, V, ocsc, ocsr, csc, csr = graph("powerlaw_2m4", "sage")
    x, y = _labels_and_features(V, 100, 47, 57)
    dims = [100, 256, 256, 47]
    rows = sample_rows(ocsc[1], 58, n_random=1500)
    torch.manual_seed(6)
    base = [SAGEConv(dims[i], dims[i + 1], root_weight=False, spmm=True).to(dev()) for i in range(3)]
    results = []
    for spmm in (True, False):
        layers = [SAGEConv(dims[i], dims[i + 1], root_weight=False, spmm=spmm).to(dev()) for i in range(3)]
        for a, b in zip(layers, base):
            a.load_state_dict(b.state_dict())
        h = x.clone().requires_grad_(True)
        h0 = h
        for i, layer in enumerate(layers):
            if not results:
                # aggregation happens at the layer's input width: rows of it against the oracle
                agg = layer.propagate_spmm(x=h, csr=csr)
                _layer_rows_check("sage", agg, h, None, ocsc, rows, "SAGE layer %d aggregation rows" % (i + 1))
            h_out = layer(h, None, None, csc, csr)
            h = torch.relu(h_out) if i < 2 else h_out
        loss = torch.nn.functional.nll_loss(torch.log_softmax(h, dim=1), y)
        loss.backward()
        torch.cuda.synchronize()
        grads = [h0.grad.clone()] + [p.grad.clone() for layer in layers for p in layer.parameters()]
        assert all(torch.isfinite(t).all() for t in grads) and torch.isfinite(loss)
        results.append((loss.item(), grads))
    (l0, g0), (l1, g1) = results
    assert abs(l0 - l1) <= 1e-5 * abs(l0), (l0, l1)
    for a, b in zip(g0, g1):
        assert_close(a.cpu().numpy(), b.cpu().numpy(), np.abs(b.cpu().numpy()) + b.abs().mean().item(), rtol=1e-4,
                     what="SAGE gradients through the two routes")


def test_release_cached_graph():
    """Frees the resident configuration so that later test files start from an empty GPU."""
    graph.cache_clear()
    torch.cuda.empty_cache()
