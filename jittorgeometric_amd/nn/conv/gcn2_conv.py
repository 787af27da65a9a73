"""GCNII layer with the reference's constructor and call (nn/conv/gcn2_conv.py:47-73):

    support = (1 - beta) (1 - alpha) x   + beta x   W1
    initial = (1 - beta) alpha       x_0 + beta x_0 W2
    out     = A support + initial

Each of the two blends is one BLAS call (the scaled input is the product's
addend), and `+ initial` is applied where the product over the graph stores its
rows; the reference runs four scalings, two products, two additions, the
product over the graph and one more addition."""
import torch

from ..inits import glorot
from ...ops import SpmmCsr, aggregateWithWeight
from ...ops.propagate import propagate_axpby


class GCN2Conv(torch.nn.Module):
    def __init__(self, in_channels, out_channels, cached=False, add_self_loops=True, spmm=False, fused=True, **kwargs):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.cached = cached
        self.spmm = spmm
        self.fused = fused
        self.weight1 = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        self.weight2 = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight1)
        glorot(self.weight2)

    def forward(self, x, x_0, csc, csr, alpha, beta):
        if x.dim() == 2 and x_0.dim() == 2:
            support = torch.addmm(x, x, self.weight1, beta=(1 - beta) * (1 - alpha), alpha=beta)
            initial = torch.addmm(x_0, x_0, self.weight2, beta=(1 - beta) * alpha, alpha=beta)
        else:
            support = (1 - beta) * (1 - alpha) * x + beta * torch.matmul(x, self.weight1)
            initial = (1 - beta) * alpha * x_0 + beta * torch.matmul(x_0, self.weight2)
        if self.fused and support.is_cuda and support.dim() == 2 and support.dtype == torch.float32:
            # spmm=True only needs the CSR (gcn2_conv.py:70-71), otherwise both are used
            return propagate_axpby(support.contiguous(), initial.contiguous(),
                                   None if self.spmm and csr is not None else csc, csr, 1.0, 1.0)
        if self.spmm:
            return self.propagate_spmm(support, csr) + initial
        return self.propagate_msg(support, csc, csr) + initial

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}({}, {})".format(self.__class__.__name__, self.in_channels, self.out_channels)
