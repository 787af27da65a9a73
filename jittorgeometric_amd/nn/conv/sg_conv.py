"""Simplified graph convolution with the reference layer's constructor and
call (nn/conv/sg_conv.py:14-80): K products with the normalised adjacency,
then one linear layer."""
import torch

from ...ops import SpmmCsr, aggregateWithWeight
from ..dense import add_bias, xw
from ..inits import glorot, zeros


class SGConv(torch.nn.Module):
    def __init__(self, in_channels, out_channels, K=1, bias=True, spmm=True, **kwargs):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.K = K
        self.spmm = spmm
        # stored [in, out] like the other layers here; the reference's Linear keeps [out, in]
        self.weight = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        self.bias = torch.nn.Parameter(torch.empty(out_channels)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        zeros(self.bias)

    def forward(self, x, csc, csr):
        for _ in range(self.K):
            x = self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)
        out = xw(x, self.weight)
        if self.bias is not None:
            out = add_bias(out, self.bias)
        return out

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}({}, {}, K={})".format(self.__class__.__name__, self.in_channels, self.out_channels, self.K)
