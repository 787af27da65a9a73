"""EvenNet propagation with the reference layer's call (nn/conv/even_conv.py:33-61):
out = temp[0] x, then K hops x <- A x of which hop k (counted from 0) is added
with temp[k+1] when k // 2 == 1.  As that test is written it names the third
and the fourth hop (k = 2, 3), not the even ones, and the result here is the
same: out = temp[0] x + temp[3] A^3 x + temp[4] A^4 x.  Hops after the last one
that is added cannot change the result and are not run.  temp = alpha (1 -
alpha)^k with the last one (1 - alpha)^K: constants (the reference's
reset_parameters replaces the parameter by a numpy array, even_conv.py:48-50).
The reference's constructor reads an undefined name (`Init`, even_conv.py:37)
and so cannot be called as it stands; that line has no counterpart here."""
import numpy as np
import torch

from ...ops import SpmmCsr, aggregateWithWeight
from ...ops.propagate import propagate_axpby


class EvenNet(torch.nn.Module):
    def __init__(self, K, alpha, spmm=True, fused=True, **kwargs):
        super().__init__()
        self.K = K
        self.alpha = alpha
        self.spmm = spmm
        self.fused = fused
        self.reset_parameters()

    def reset_parameters(self):
        self.temp = self.alpha * (1 - self.alpha) ** np.arange(self.K + 1)
        self.temp[-1] = (1 - self.alpha) ** self.K

    def forward(self, x, csc, csr):
        t = [float(v) for v in self.temp]
        added = [k for k in range(self.K) if k // 2 == 1]
        if not added:
            return x * t[0]
        if not (self.fused and x.is_cuda and x.dim() == 2 and x.dtype == torch.float32):
            out = x * t[0]
            for k in range(added[-1] + 1):
                x = self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)
                if k in added:
                    out = out + t[k + 1] * x
            return out
        # two plain hops, then out = t3 A x2 + t0 x in the third product's row store; the fourth,
        # if it counts, needs A^3 x itself as well
        csc = None if self.spmm and csr is not None else csc
        x0 = x.contiguous()
        x2 = propagate_axpby(propagate_axpby(x0, None, csc, csr), None, csc, csr)
        if len(added) == 1:
            return propagate_axpby(x2, x0, csc, csr, t[3], t[0])
        x3 = propagate_axpby(x2, None, csc, csr)
        out = torch.add(x0 * t[0], x3, alpha=t[3])
        return propagate_axpby(x3, out, csc, csr, t[4], 1.0)

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}(K={}, alpha={})".format(self.__class__.__name__, self.K, self.alpha)
