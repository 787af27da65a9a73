"""Two calls of the same entry point in flight at once on two streams of equal priority, each
with its own workspace and outputs: what the C ABI's header promises ("calls are re-entrant; two
calls may overlap on one GPU when they use different workspaces and outputs").  Each result is
compared bit for bit with the same call run alone.  The product follows
ops/cpp/aggregate_op.cc:42-58, the conversion ops/cpp/cootocsr_op.cc:35-53."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def lib():
    from jittorgeometric_amd import _lib
    return _lib, _lib.load()


def spmm_on(stream, off, idx, w, x, R):
    L, l = lib()
    C, F = x.shape
    E = idx.shape[0]
    with torch.cuda.stream(stream):
        out = torch.empty((R, F), dtype=torch.float32, device=dev())
        nbytes = L.query(l.jgamd_spmm_csx_workspace, R, E, F)
        ws = L.workspace(nbytes, dev())
        L.check(l.jgamd_spmm_csx(L.ptr(off), L.ptr(idx), L.ptr(w), L.ptr(x), L.ptr(out), R, C, E, F, L.ptr(ws), nbytes,
                                 stream.cuda_stream))
    return out, ws


def convert_on(stream, ei, w, V, key_row):
    L, l = lib()
    E = ei.shape[1]
    with torch.cuda.stream(stream):
        idx = torch.empty(E, dtype=torch.int32, device=dev())
        off = torch.empty(V + 1, dtype=torch.int32, device=dev())
        ow = torch.empty(E, dtype=torch.float32, device=dev())
        nbytes = L.query(l.jgamd_coo_to_csx_workspace, E, V, 0)
        ws = L.workspace(nbytes, dev())
        L.check(l.jgamd_coo_to_csx(L.ptr(ei), L.ptr(w), E, V, key_row, L.ptr(idx), L.ptr(off), L.ptr(ow), None, L.ptr(ws),
                                   nbytes, stream.cuda_stream))
    return (idx, off, ow), ws


def test_two_products_overlap_on_two_streams():
    rng = np.random.default_rng(3)
    V, E = 200000, 3000000
    ei, w = rand_graph(rng, V, E, 3, 0.2)
    row, off, wt = oracle.cootocsc(ei, w, V)
    col, roff, rw = oracle.cootocsr(ei, w, V)
    xa = to_gpu(rng.standard_normal((V, 128)).astype(np.float32))
    xb = to_gpu(rng.standard_normal((V, 96)).astype(np.float32))
    a = [to_gpu(t) for t in (off, row, wt)]
    b = [to_gpu(t) for t in (roff, col, rw)]
    main = torch.cuda.current_stream()
    alone_a, _ = spmm_on(main, a[0], a[1], a[2], xa, V)
    alone_b, _ = spmm_on(main, b[0], b[1], b[2], xb, V)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()          # default (equal) priority
    keep = []
    for _ in range(4):                                          # several rounds so that the launches interleave
        ra, wa = spmm_on(s1, a[0], a[1], a[2], xa, V)
        rb, wb = spmm_on(s2, b[0], b[1], b[2], xb, V)
        keep.append((ra, rb, wa, wb))
    torch.cuda.synchronize()
    for ra, rb, _, _ in keep:
        assert torch.equal(ra, alone_a) and torch.equal(rb, alone_b)
    want, terms = oracle.aggregate_f64(xa.cpu().numpy(), row, off, wt)
    assert_close(alone_a.cpu().numpy(), want, terms, what="product on its own stream")


def test_two_conversions_overlap_on_two_streams():
    rng = np.random.default_rng(4)
    V, E = 300000, 4000000
    ei, w = rand_graph(rng, V, E, 2, 0.2)
    ei_g, w_g = to_gpu(ei), to_gpu(w)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    keep = []
    for _ in range(3):
        csr, w1 = convert_on(s1, ei_g, w_g, V, 0)
        csc, w2 = convert_on(s2, ei_g, w_g, V, 1)
        keep.append((csr, csc, w1, w2))
    torch.cuda.synchronize()
    want_r, want_c = oracle.cootocsr(ei, w, V), oracle.cootocsc(ei, w, V)
    for csr, csc, _, _ in keep:
        for got, want in ((csr, want_r), (csc, want_c)):
            assert np.array_equal(got[0].cpu().numpy(), want[0])
            assert np.array_equal(got[1].cpu().numpy(), want[1])
            assert np.array_equal(got[2].cpu().numpy().view(np.int32), want[2].view(np.int32))


def test_spmmcsr_with_the_dense_operand_stored_transposed():
    """SpmmCsr(x, csr, trans_B=True) is op(A) x^T (ops/spmmcsr.py:31 hands the flag to cuSPARSE)."""
    from jittorgeometric_amd import CSR
    from jittorgeometric_amd.ops import SpmmCsr
    rng = np.random.default_rng(5)
    V, E, F = 300, 4000, 24
    ei, w = rand_graph(rng, V, E, 1)
    col, roff, rw = oracle.cootocsr(ei, w, V)
    csr = CSR(to_gpu(col), to_gpu(roff), to_gpu(rw))
    x = rng.standard_normal((F, V)).astype(np.float32)
    xt = to_gpu(x).requires_grad_(True)
    out = SpmmCsr(xt, csr, trans_A=True, trans_B=True)
    plain = SpmmCsr(to_gpu(np.ascontiguousarray(x.T)), csr, trans_A=True)
    assert out.shape == (V, F) and torch.equal(out, plain)
    g = rng.standard_normal((V, F)).astype(np.float32)
    out.backward(to_gpu(g))
    # d/dx of <g, A^T x^T> = (A g)^T: the product over the CSR arrays themselves, transposed
    want, terms = oracle.aggregate_f64(g, col, roff, rw)
    assert_close(xt.grad.cpu().numpy(), want.T, terms.T, what="gradient with trans_B")
