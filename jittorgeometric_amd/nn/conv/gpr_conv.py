"""Generalised PageRank propagation with the reference layer's constructor and
call (nn/conv/gpr_conv.py:18-101): Z = sum_k temp[k] * A^k x with learnable
temp, initialised as SGC / PPR / NPPR / Random / WS."""
import numpy as np
import torch

from ...ops import SpmmCsr, aggregateWithWeight


class GPRGNN(torch.nn.Module):
    def __init__(self, K, alpha, Init, spmm=True, Gamma=None, **kwargs):
        super().__init__()
        self.K = K
        assert Init in ["SGC", "PPR", "NPPR", "Random", "WS"]
        if Init == "SGC":
            temp = 0.0 * np.ones(K + 1)
            temp[-1] = 1.0
        elif Init == "PPR":
            temp = alpha * (1 - alpha) ** np.arange(K + 1)
            temp[-1] = (1 - alpha) ** K
        elif Init == "NPPR":
            temp = (alpha) ** np.arange(K + 1)
            temp = temp / np.sum(np.abs(temp))
        elif Init == "Random":
            bound = np.sqrt(3 / (K + 1))
            temp = np.random.uniform(-bound, bound, K + 1)
            temp = temp / np.sum(np.abs(temp))
        else:
            # the reference reads an undefined name here (gpr_conv.py:67); the weights are an argument instead
            if Gamma is None:
                raise ValueError("Init='WS' needs Gamma (K+1 weights)")
            temp = np.asarray(Gamma, dtype=np.float64)
        self.temp = torch.nn.Parameter(torch.tensor(temp, dtype=torch.float32))
        self.spmm = spmm

    def reset_parameters(self):
        pass

    def forward(self, x, csc, csr):
        out = x * self.temp[0]
        for k in range(self.K):
            x = self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)
            out = torch.addcmul(out, self.temp[k + 1], x)      # out + temp[k+1] * x in one pass
        return out

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}(K={})".format(self.__class__.__name__, self.K)
