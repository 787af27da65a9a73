"""SpMM on a COO matrix.  Same call as jittor_geometric.ops.SpmmCoo
(ops/spmmcoo.py:21-44), whose arithmetic is cuSPARSE's COO product inside the
jittor wheel.  trans_A=True (the default) gives out[col] = sum of w * x[row]
over the edges (row, col), the quantity tests/test_mp_spmm.py:28-36 prints
beside aggregateWithWeight.  Here the edges are compressed by destination with
the stable conversion and the product runs as the row-gather kernel, so the
result does not depend on the order in which a scatter would have landed."""
import torch

from .. import _lib
from ._common import spmm
from .cootocsr import _convert


def _product(x, edge_index, edge_weight, by_row):
    V = x.shape[0]
    # by_row: out[row] = sum w * x[col]  (key = edge_index[0], gathered = edge_index[1])
    idx, off, w, _ = _convert(edge_index, edge_weight, V, 0 if by_row else 1)
    return spmm(off, idx, w, x, V)


class SpmmCooFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, edge_index, edge_weight, trans_A, trans_B):
        if trans_B:
            raise _lib.JgamdError("SpmmCoo: trans_B=True is not supported")
        ctx.edge_index, ctx.edge_weight, ctx.trans_A = edge_index, edge_weight, trans_A
        return _product(x, edge_index, edge_weight, by_row=not trans_A)

    @staticmethod
    def backward(ctx, grad_output):
        # the reference's grad runs the product without the transpose (ops/spmmcoo.py:38-40)
        g = _product(grad_output.contiguous(), ctx.edge_index, ctx.edge_weight, by_row=ctx.trans_A)
        return g, None, None, None, None


def SpmmCoo(x, edge_index, edge_weight, trans_A=True, trans_B=False):
    return SpmmCooFunc.apply(x, edge_index, edge_weight, trans_A, trans_B)
