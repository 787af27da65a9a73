"""LightGCN propagation with the reference layer's constructor and call
(nn/conv/lightgcn_conv.py:16-44): one product over the graph, no weights."""
import torch

from ...ops import SpmmCsr, aggregateWithWeight


class LightGCNConv(torch.nn.Module):
    def __init__(self, spmm=True, **kwargs):
        super().__init__()
        self.spmm = spmm

    def reset_parameters(self):
        pass

    def forward(self, x, csc, csr):
        return self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}()".format(self.__class__.__name__)
