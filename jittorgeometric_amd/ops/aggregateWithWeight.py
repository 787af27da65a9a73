"""Weighted aggregation over CSC (forward) / CSR (backward).  Same call as
jittor_geometric.ops.aggregateWithWeight (ops/aggregateWithWeight.py:19-54);
the loops of ops/cpp/aggregate_op.cc run as csrc/spmm.hip."""
import torch

from ._common import csc_arrays, csr_arrays, spmm


class AggregateFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csc, csr, edge_weight):
        ctx.csr = csr
        ctx.weight = edge_weight
        off, idx, w = csc_arrays(csc)
        if isinstance(edge_weight, torch.Tensor):
            w = edge_weight.reshape(-1)
        # the reference sizes the output like x (zeros_like, :28)
        return spmm(off, idx, w, x, x.shape[0])

    @staticmethod
    def backward(ctx, grad_output):
        csr = ctx.csr
        off, idx, w = csr_arrays(csr)
        if isinstance(ctx.weight, torch.Tensor):
            w = ctx.weight.reshape(-1)
        g = spmm(off, idx, w, grad_output, grad_output.shape[0])
        return g, None, None, None


def aggregateWithWeight(x, csc, csr, weight=None):
    """out[dst] = sum over edges (src -> dst) of w * x[src]; gradient
    grad_x[src] = sum w * grad_out[dst] through the CSR arrays."""
    return AggregateFunc.apply(x, csc, csr, weight)
