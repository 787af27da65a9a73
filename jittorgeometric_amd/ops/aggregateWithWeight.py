"""Weighted aggregation over CSC (forward) / CSR (backward).  Same call as
jittor_geometric.ops.aggregateWithWeight (ops/aggregateWithWeight.py:19-54);
the loops of ops/cpp/aggregate_op.cc run as csrc/spmm.hip."""
import torch

from ._common import spmm


class AggregateFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csc, csr, edge_weight):
        ctx.csr = csr
        ctx.weight = edge_weight
        w = edge_weight if isinstance(edge_weight, torch.Tensor) else csc.edge_weight
        # the reference sizes the output like x (zeros_like, :28)
        return spmm(csc.column_offset, csc.row_indices, w, x, x.shape[0])

    @staticmethod
    def backward(ctx, grad_output):
        csr = ctx.csr
        w = ctx.weight if isinstance(ctx.weight, torch.Tensor) else csr.edge_weight
        g = spmm(csr.row_offset, csr.column_indices, w, grad_output.contiguous(), grad_output.shape[0])
        return g, None, None, None


def aggregateWithWeight(x, csc, csr, weight=None):
    """out[dst] = sum over edges (src -> dst) of w * x[src]; gradient
    grad_x[src] = sum w * grad_out[dst] through the CSR arrays."""
    return AggregateFunc.apply(x, csc, csr, weight)
