"""Writes tests/golden/oracle_vectors_v64.npz: a 64-node seeded power-law graph
with the CPU oracle's outputs for every operator of the path (conversion,
SpMM at F=7/8/33, edge softmax H=1/2 and its gradient, scatter operators, GAT
forward H=1 and H=2).  Run from the repository root:
    python tests/golden/make_oracle_vectors.py
The file pins the oracle against accidental change and gives the GPU tests a
fixture that does not depend on the oracle being rebuilt."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from jittorgeometric_amd import synthetic  # noqa: E402


def build():
    V = 64
    rng = np.random.default_rng(64)
    ei = synthetic.chung_lu(V, 600, 2.1, max_degree=40, seed=64)
    ei, w = oracle.gcn_norm(ei, None, V)
    ei = ei.astype(np.int32)
    out = {"edge_index": ei, "edge_weight": w, "v_num": np.int32(V)}
    col, roff, rw = oracle.cootocsr(ei, w, V)
    row, coff, cw = oracle.cootocsc(ei, w, V)
    out.update(csr_col=col, csr_off=roff, csr_w=rw, csc_row=row, csc_off=coff, csc_w=cw)
    for F in (7, 8, 33):
        x = rng.standard_normal((V, F)).astype(np.float32)
        out["x%d" % F] = x
        out["agg_fwd%d" % F] = oracle.aggregate(x, row, coff, cw)
        out["agg_bwd%d" % F] = oracle.aggregate(x, col, roff, rw)
        # sum of the absolute terms of every output element: what a difference in the order
        # of summation scales with (the tolerance of the GPU tests is relative to it)
        out["agg_fwd_terms%d" % F] = oracle.aggregate(np.abs(x), row, coff, np.abs(cw))
        out["agg_bwd_terms%d" % F] = oracle.aggregate(np.abs(x), col, roff, np.abs(rw))
    E = ei.shape[1]
    for H in (1, 2):
        z = (2 * rng.standard_normal((E, H))).astype(np.float32)
        g = rng.standard_normal((E, H)).astype(np.float32)
        y = oracle.edgesoftmax(z, coff).reshape(E, H)
        out["sm_x%d" % H], out["sm_g%d" % H], out["sm_y%d" % H] = z, g, y
        out["sm_dx%d" % H] = oracle.edgesoftmax_backward(g, y, coff).reshape(E, H)
    xv = rng.standard_normal((V, 5)).astype(np.float32)
    xe = rng.standard_normal((E, 5)).astype(np.float32)
    out.update(sc_x=xv, sc_xe=xe, sc_src=oracle.scattertoedge(xv, row, coff, 0),
               sc_dst=oracle.scattertoedge(xv, row, coff, 1), ev_src=oracle.edgetovertex(xe, row, coff, 0),
               ev_dst=oracle.edgetovertex(xe, row, coff, 1),
               ev_src_terms=oracle.edgetovertex(np.abs(xe), row, coff, 0),
               ev_dst_terms=oracle.edgetovertex(np.abs(xe), row, coff, 1))
    h = np.maximum(rng.standard_normal((V, 2, 6)), 0).astype(np.float32)
    a_src = (rng.standard_normal((2, 6)) / 2).astype(np.float32)
    a_dst = (rng.standard_normal((2, 6)) / 2).astype(np.float32)
    o2, al2 = oracle.gat_forward_heads(h, (row, coff, cw), a_src, a_dst, 0.2)
    o1, al1, _ = oracle.gat_forward(np.ascontiguousarray(h[:, 0, :]), (row, coff, cw),
                                    np.concatenate([a_src[0], a_dst[0]]), 0.2)
    out.update(gat_h=h, gat_a_src=a_src, gat_a_dst=a_dst, gat_out2=o2, gat_alpha2=al2, gat_out1=o1, gat_alpha1=al1)
    # sum over a destination's in-edges of alpha * |h[src]|, per head and feature
    terms = np.zeros_like(o2, dtype=np.float64)
    np.add.at(terms, np.repeat(np.arange(V), np.diff(coff)), al2[:, :, None].astype(np.float64) * np.abs(h[row]))
    out["gat_terms2"] = terms.astype(np.float32)
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_vectors_v64.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
