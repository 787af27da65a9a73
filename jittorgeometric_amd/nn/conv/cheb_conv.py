"""Chebyshev spectral convolution with the constructor and call of the
reference's ChebConv (nn/conv/cheb_conv.py:69-163):

    out = sum_{k < K} T_k(L^) x  W_k (+ b),   L^ = 2 L / lambda_max - I

The reference sends `norm_e * x[src]` messages over the edge list at every
step (message passing through gathers and a scatter-add); the same sum is the
product over the compressed form of (edge_index, norm), so the scaled Laplacian
is converted once per call (kept while the same edge tensors come back) and
every step T_k = 2 L^ T_{k-1} - T_{k-2} is one kernel: the product with the
subtraction in its row store."""
import torch
from torch import nn

from ...ops import cootocsc
from ...ops._common import _stamp
from ...ops.propagate import propagate_axpby
from ...utils.get_laplacian import get_laplacian
from ..inits import glorot, zeros


class ChebConv(nn.Module):
    def __init__(self, in_channels, out_channels, K, normalization="sym", bias=True, **kwargs):
        super().__init__()
        assert K > 0
        assert normalization in [None, "sym", "rw"], "Invalid normalization"
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.normalization = normalization
        self.lins = nn.ModuleList([nn.Linear(in_channels, out_channels, bias=False) for _ in range(K)])
        self.bias = nn.Parameter(torch.zeros(out_channels)) if bias else None
        self._graph = None
        self.reset_parameters()

    def reset_parameters(self):
        for lin in self.lins:
            glorot(lin.weight)
        zeros(self.bias)
        self._graph = None

    def __norm__(self, edge_index, num_nodes, edge_weight, normalization, lambda_max=None, dtype=None, batch=None):
        edge_index, edge_weight = get_laplacian(edge_index, edge_weight, normalization, dtype, num_nodes)
        if lambda_max is None:
            lambda_max = 2.0 * edge_weight.max()
        elif not isinstance(lambda_max, torch.Tensor):
            lambda_max = torch.tensor([lambda_max], dtype=torch.float32, device=edge_weight.device)
        if batch is not None and lambda_max.numel() > 1:
            lambda_max = lambda_max[batch[edge_index[0].long()]]
        edge_weight = (2.0 * edge_weight) / lambda_max
        edge_weight = torch.where(edge_weight == float("inf"), torch.zeros_like(edge_weight), edge_weight)
        loop_mask = edge_index[0] == edge_index[1]
        return edge_index, torch.where(loop_mask, edge_weight - 1, edge_weight)

    def _compressed(self, x, edge_index, edge_weight, batch, lambda_max):
        """CSC arrays of the scaled Laplacian; rebuilt when any of the tensors it came from changes."""
        lam_key = _stamp(lambda_max) if isinstance(lambda_max, torch.Tensor) else lambda_max
        key = (_stamp(edge_index), _stamp(edge_weight), _stamp(batch), lam_key, x.size(0), self.normalization)
        if self._graph is not None and self._graph[0] == key:
            return self._graph[2]
        with torch.no_grad():
            ei, norm = self.__norm__(edge_index, x.size(0), edge_weight, self.normalization, lambda_max, batch=batch)
            csc = cootocsc(ei.contiguous(), norm.contiguous(), x.size(0))
        # the tensors are kept beside their stamps, so that no other tensor can take their id
        self._graph = (key, (edge_index, edge_weight, batch, lambda_max), csc)
        return csc

    def forward(self, x, edge_index, edge_weight=None, batch=None, lambda_max=None):
        if x.is_floating_point() and x.dtype != torch.float32:
            x = x.to(torch.float32)
        csc = self._compressed(x, edge_index, edge_weight, batch, lambda_max)
        x = x.contiguous()
        tx0 = tx1 = x
        out = self.lins[0](tx0)
        if len(self.lins) > 1:
            tx1 = propagate_axpby(x, None, csc, None)
            out = out + self.lins[1](tx1)
        for lin in self.lins[2:]:
            tx2 = propagate_axpby(tx1, tx0, csc, None, 2.0, -1.0)
            out = out + lin(tx2)
            tx0, tx1 = tx1, tx2
        return out if self.bias is None else out + self.bias

    execute = forward

    def __repr__(self):
        return "{}({}, {}, K={}, normalization={})".format(self.__class__.__name__, self.in_channels, self.out_channels,
                                                           len(self.lins), self.normalization)
