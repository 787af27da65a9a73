"""APPNP propagation with the reference layer's constructor and call
(nn/conv/appnp_conv.py:17-66): K times x <- (1 - alpha) * A x + alpha * h."""
import torch

from ...ops import SpmmCsr, aggregateWithWeight
from ...ops.propagate import appnp_propagate


class APPNP(torch.nn.Module):
    """fused=True (default) runs every hop as one kernel, product and blend
    together, forward and backward; fused=False is the reference's chain of
    operators (product, scale, add), kept for comparison."""

    def __init__(self, K, alpha, spmm=True, fused=True, **kwargs):
        super().__init__()
        self.K = K
        self.alpha = alpha
        self.spmm = spmm
        self.fused = fused

    def reset_parameters(self):
        pass

    def forward(self, x, csc, csr):
        if self.fused:
            # spmm=True only needs the CSR (appnp_conv.py:44-45), otherwise both are used
            return appnp_propagate(x, None if self.spmm and csr is not None else csc, csr, self.K, self.alpha)
        h = x
        for _ in range(self.K):
            x = self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)
            x = x * (1 - self.alpha)
            x = x + self.alpha * h
        return x

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}(K={}, alpha={})".format(self.__class__.__name__, self.K, self.alpha)
