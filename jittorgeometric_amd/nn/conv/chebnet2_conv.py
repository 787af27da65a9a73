"""ChebNetII propagation with the reference layer's constructor and call
(nn/conv/chebnet2_conv.py:55-93): K+1 learnable values at the Chebyshev nodes
x_j = cos((K - j + 0.5) pi / (K + 1)), clamped at zero, give the coefficients

    coe[i] = 2 / (K + 1) * sum_j relu(temp)[j] T_i(x_j)

and out = coe[0] / 2 T_0 x + sum_{i >= 1} coe[i] T_i(A) x by the recurrence
T_i = 2 A T_{i-1} - T_{i-2}.  The table T_i(x_j) is a constant of K, so the
coefficients are one small matrix product, and every step of the recurrence is
one kernel (the product over the graph with `2 * ... - T_{i-2}` in its row
store) where the reference runs a product, a scaling and a subtraction."""
import numpy as np
import torch

from ...ops import SpmmCsr, aggregateWithWeight
from ...ops.propagate import propagate_axpby


def node_table(K):
    """T[i, j] = T_i(x_j) for i, j = 0..K."""
    nodes = np.cos((K - np.arange(K + 1) + 0.5) * np.pi / (K + 1))
    T = np.ones((K + 1, K + 1))
    if K >= 1:
        T[1] = nodes
    for i in range(2, K + 1):
        T[i] = 2 * nodes * T[i - 1] - T[i - 2]
    return T


class ChebNetII(torch.nn.Module):
    def __init__(self, K, spmm=True, fused=True, **kwargs):
        super().__init__()
        if K < 1:
            # the reference's execute reads coe[1] (chebnet2_conv.py:82) and fails there
            raise ValueError("ChebNetII needs K >= 1")
        self.K = K
        self.spmm = spmm
        self.fused = fused
        self.temp = torch.nn.Parameter(torch.ones(K + 1))
        self.register_buffer("table", torch.tensor(node_table(K) * (2.0 / (K + 1)), dtype=torch.float32),
                             persistent=False)

    def reset_parameters(self):
        with torch.no_grad():
            self.temp.fill_(1.0)

    def coefficients(self):
        return self.table.to(self.temp.device) @ torch.relu(self.temp)

    def forward(self, x, csc, csr):
        coe = self.coefficients()
        fused = self.fused and x.is_cuda and x.dim() == 2 and x.dtype == torch.float32
        if fused:
            csc = None if self.spmm and csr is not None else csc
            x = x.contiguous()
            hop = lambda v, h, b, a: propagate_axpby(v, h, csc, csr, b, a)
        else:
            def hop(v, h, b, a):
                y = self.propagate_spmm(v, csr) if self.spmm else self.propagate_msg(v, csc, csr)
                return y if h is None else b * y + a * h
        t0 = x
        t1 = hop(t0, None, 1.0, 0.0)
        out = torch.addcmul(coe[0] / 2 * t0, coe[1], t1)
        for i in range(2, self.K + 1):
            t2 = hop(t1, t0, 2.0, -1.0)
            out = torch.addcmul(out, coe[i], t2)
            t0, t1 = t1, t2
        return out

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}(K={})".format(self.__class__.__name__, self.K)
