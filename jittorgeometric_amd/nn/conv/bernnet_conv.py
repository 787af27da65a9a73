"""BernNet propagation with the reference layer's constructor and call
(nn/conv/bernnet_conv.py:44-80):

    out = sum_{i=0..K} C(K, i) / 2^K * relu(temp)[i] * A1^i A2^(K-i) x

with A1 the graph of (csc1, csr1) and A2 that of (csc2, csr2) (the Laplacian
L and 2I - L in the reference's model).  The reference evaluates every term
from the stored A2^k x, K (K + 1) / 2 + K products; here the sum is evaluated
by Horner's rule in A1,

    y = c_K t_K x;   y <- A1 y + c_j t_j A2^(K-j) x   for j = K-1 .. 0,

2 K products, each with the addition in the product's row store.  The result is
the same polynomial; its float32 rounding differs from the reference's order of
additions like that of any reordered sum."""
from math import comb

import torch

from ...ops import SpmmCsr, aggregateWithWeight
from ...ops.propagate import propagate_axpby


class BernNet(torch.nn.Module):
    def __init__(self, K, spmm=True, fused=True, **kwargs):
        super().__init__()
        self.K = K
        self.spmm = spmm
        self.fused = fused
        self.temp = torch.nn.Parameter(torch.ones(K + 1))

    def reset_parameters(self):
        with torch.no_grad():
            self.temp.fill_(1.0)

    def forward(self, x, csc1, csr1, csc2, csr2):
        K = self.K
        t = torch.relu(self.temp)
        c = [comb(K, i) / 2 ** K for i in range(K + 1)]
        if not (self.fused and x.is_cuda and x.dim() == 2 and x.dtype == torch.float32):
            one = lambda v, csc, csr: self.propagate_spmm(v, csr) if self.spmm else self.propagate_msg(v, csc, csr)
            tmp = [x]
            for _ in range(K):
                tmp.append(one(tmp[-1], csc2, csr2))
            out = c[0] * t[0] * tmp[K]
            for i in range(K):
                v = tmp[K - i - 1]
                for _ in range(i + 1):
                    v = one(v, csc1, csr1)
                out = out + c[i + 1] * t[i + 1] * v
            return out
        if self.spmm and csr1 is not None:
            csc1 = None
        if self.spmm and csr2 is not None:
            csc2 = None
        tmp = [x.contiguous()]
        for _ in range(K):
            tmp.append(propagate_axpby(tmp[-1], None, csc2, csr2))
        y = (c[K] * t[K]) * tmp[0]
        for j in range(K - 1, -1, -1):
            y = propagate_axpby(y, (c[j] * t[j]) * tmp[K - j], csc1, csr1, 1.0, 1.0)
        return y

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}(K={})".format(self.__class__.__name__, self.K)
