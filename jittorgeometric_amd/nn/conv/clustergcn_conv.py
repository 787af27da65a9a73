"""ClusterGCN layer with the constructor and call signature of the reference's
ClusterGCNConv (nn/conv/clustergcn_conv.py:42-158) on torch tensors:

    out = (A x) W_out + x W_root (+ b),   A from clustergcn_norm

Normalisation, both conversions, the product over the graph and the two dense
products with the bias row are the kernels of the GraphSAGE layer (the same
expression with other weights on the edges): one autograd node, both dense
products in one pass of the matrix-core kernel."""
import torch
from torch import nn

from ...ops import SpmmCsr, aggregateWithWeight, cootocsc, cootocsr
from ...ops import spmmcsr as _spmmcsr
from ...ops._common import both_orders
from ..dense import add_bias, xw
from ..inits import glorot, zeros
from .gcn_conv import _degree_norm, _normalised
from .sage_conv import SageLayerFunc


def clustergcn_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True,
                    diag_lambda=0.0, dtype=None):
    """w * d^-1[row] with the degree summed by column, and diag_lambda * d^-1[row] more on every
    self-loop (nn/conv/clustergcn_conv.py:14-39)."""
    edge_index, edge_weight, dinv, order = _degree_norm(edge_index, edge_weight, num_nodes, improved, add_self_loops, -1.0)
    if diag_lambda == 0.0:
        return _normalised(edge_index, edge_weight, dinv, None, dinv.shape[0], order)
    edge_index, weights = _normalised(edge_index, edge_weight, dinv, None, dinv.shape[0], None)
    row, col = edge_index[0], edge_index[1]
    return edge_index, torch.where(row == col, weights + diag_lambda * dinv[row.long()], weights)


class ClusterGCNConv(nn.Module):
    def __init__(self, in_channels, out_channels, diag_lambda=0.0, improved=False, cached=False,
                 add_self_loops=True, normalize=True, bias=True, spmm=True, **kwargs):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.diag_lambda = diag_lambda
        self.improved = improved
        self.cached = cached
        self.add_self_loops = add_self_loops
        self.normalize = normalize
        self._cached_edge_index = None
        self.weight_out = nn.Parameter(torch.empty(in_channels, out_channels))
        self.weight_root = nn.Parameter(torch.empty(in_channels, out_channels))
        self.bias = nn.Parameter(torch.empty(out_channels)) if bias else None
        self.spmm = spmm
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight_out)
        glorot(self.weight_root)
        zeros(self.bias)
        self._cached_edge_index = None

    def forward(self, x, edge_index, edge_weight=None):
        if x.is_floating_point() and x.dtype != torch.float32:
            x = x.to(torch.float32)
        cache = self._cached_edge_index
        if cache is None:
            if self.normalize:
                edge_index, edge_weight = clustergcn_norm(edge_index, edge_weight, x.size(0), self.improved,
                                                          self.add_self_loops, self.diag_lambda)
            elif edge_weight is None:
                # the reference converts only inside `if self.normalize` (clustergcn_conv.py:116-130) and
                # then reads csr / csc it never set; without normalisation the edges count as they are
                edge_weight = torch.ones(edge_index.shape[1], dtype=torch.float32, device=x.device)
            with torch.no_grad():
                csc = cootocsc(edge_index, edge_weight, x.size(0))
                csr = cootocsr(edge_index, edge_weight, x.size(0))
            if self.cached:
                self._cached_edge_index = (edge_index, edge_weight, csr, csc)
        else:
            edge_index, edge_weight, csr, csc = cache
        reference_grad = self.spmm and _spmmcsr.REFERENCE_GRAD
        if x.dim() == 2 and not reference_grad:
            fwd, bwd = both_orders(None if self.spmm else csc, csr)
            return SageLayerFunc.apply(x.contiguous(), self.weight_out, self.weight_root, self.bias, fwd, bwd, False)
        out = self.propagate_spmm(x, csr) if self.spmm else self.propagate_msg(x, csc, csr)
        out = xw(out, self.weight_out) + xw(x, self.weight_root)
        return out if self.bias is None else add_bias(out, self.bias)

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}({}, {})".format(self.__class__.__name__, self.in_channels, self.out_channels)
