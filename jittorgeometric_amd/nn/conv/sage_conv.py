"""GraphSAGE (mean) layer with the constructor and call signature of the
reference's SAGEConv (nn/conv/sage_conv.py:43-240) on torch tensors."""
import torch
from torch import nn

from ...ops import SpmmCsr, aggregateWithWeight, cootocsc, cootocsr
from ...ops import spmmcsr as _spmmcsr
from ...ops._common import both_orders, spmm, spmm_axpby
from ..dense import add_bias, column_sum, relu_backward_column_sum, rows_times, xt_g, xw
from ..inits import glorot, zeros
from .gcn_conv import _degree_norm, _normalised, _scale


def sage_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True, dtype=None):
    """Mean weights w * d^-1[col] (nn/conv/sage_conv.py:16-40)."""
    edge_index, edge_weight, dinv, order = _degree_norm(edge_index, edge_weight, num_nodes, improved, add_self_loops, -1.0)
    return _normalised(edge_index, edge_weight, None, dinv, dinv.shape[0], order)


class SageLayerFunc(torch.autograd.Function):
    """(A x) W1 + x W_root + b as one autograd node (sage_conv.py:172-190 builds it from five:
    product, two dense products, two additions).  Both dense products and the bias row are
    one pass of the matrix-core kernel (csrc/dense_rows.hip); in the backward pass the root term's input gradient is added in the transposed product's row
    store, so no pass over a [V,F] array only adds two arrays."""

    @staticmethod
    def forward(ctx, x, w1, w_root, bias, fwd, bwd, relu=False):
        agg = spmm(fwd[0], fwd[1], fwd[2], x, x.shape[0])
        out = rows_times(agg, w1, x if w_root is not None else None, w_root, bias, relu)
        ctx.bwd, ctx.relu = bwd, relu
        if relu:
            ctx.save_for_backward(x, agg, w1, w_root, out)      # the activation's mask is the output's sign
        else:
            ctx.save_for_backward(x, agg, w1, w_root)
        return out

    @staticmethod
    def backward(ctx, g):
        x, agg, w1, w_root = ctx.saved_tensors[:4]
        g = g.contiguous()
        need_x, need_w1, need_root, need_b = ctx.needs_input_grad[:4]
        gx = gw1 = groot = gb = None
        if ctx.relu:
            out = ctx.saved_tensors[4]
            if g.dtype == torch.float32:
                g, gb = relu_backward_column_sum(g, out)          # mask and bias gradient in one pass
            else:
                g = g * (out > 0)
                gb = g.sum(0)
            if not need_b:
                gb = None
        elif need_b:
            gb = column_sum(g) if g.dtype == torch.float32 else g.sum(0)
        if need_w1:
            gw1 = xt_g(agg, g)
        if need_root and w_root is not None:
            groot = xt_g(x, g)
        if need_x:
            off, idx, w = ctx.bwd
            if w1.shape[1] < w1.shape[0]:
                # A^T (g W1^T) = (A^T g) W1^T: the layer narrows, so the transposed product runs on g
                # itself, at the output width, and the two dense products of the input gradient are
                # one pass.  Same gradient, summed in another order; the forward pass is untouched.
                t = spmm(off, idx, w, g, g.shape[0])
                if w_root is not None:
                    gx = rows_times(t, w1.t(), g, w_root.t())
                else:
                    gx = rows_times(t, w1.t())
            else:
                g_agg = rows_times(g, w1.t())
                if w_root is not None:
                    gx = spmm_axpby(off, idx, w, g_agg, g.shape[0], 1.0, 1.0, rows_times(g, w_root.t()))
                else:
                    gx = spmm(off, idx, w, g_agg, g.shape[0])
        return gx, gw1, groot, gb, None, None, None


class SageTransformFirstFunc(torch.autograd.Function):
    """The same layer evaluated as A (x W1) + x W_root + b: the product over the graph runs at
    the output width.  Not an order the reference offers (sage_conv.py:172-190 always aggregates
    at the input width); cheaper when out_channels < in_channels (256 -> 47: a fifth of the
    gathered bytes).  Differs from SageLayerFunc in rounding only."""

    @staticmethod
    def forward(ctx, x, w1, w_root, bias, fwd, bwd):
        h1 = rows_times(x, w1, pad_rows=True)     # gathered next
        rest = None
        if w_root is not None:
            rest = rows_times(x, w_root, bias=bias)
        elif bias is not None:
            rest = bias
        if rest is None:
            out = spmm(fwd[0], fwd[1], fwd[2], h1, x.shape[0])
        else:
            out = spmm_axpby(fwd[0], fwd[1], fwd[2], h1, x.shape[0], 1.0, 1.0, rest)
        ctx.bwd = bwd
        ctx.save_for_backward(x, w1, w_root)
        return out

    @staticmethod
    def backward(ctx, g):
        x, w1, w_root = ctx.saved_tensors
        g = g.contiguous()
        need_x, need_w1, need_root, need_b = ctx.needs_input_grad[:4]
        gx = gw1 = groot = gb = None
        if need_b:
            gb = column_sum(g) if g.dtype == torch.float32 else g.sum(0)
        if need_root and w_root is not None:
            groot = xt_g(x, g)
        if need_x or need_w1:
            off, idx, w = ctx.bwd
            g_h1 = spmm(off, idx, w, g, g.shape[0])
            if need_w1:
                gw1 = xt_g(x, g_h1)
            if need_x:
                if w_root is not None:
                    gx = rows_times(g_h1, w1.t(), g, w_root.t())
                else:
                    gx = rows_times(g_h1, w1.t())
        return gx, gw1, groot, gb, None, None


class SAGEConv(nn.Module):
    """out = mean_aggregate(x) W1 (+ x W_root) (+ b); aggregation happens at
    the input width, before the dense product (sage_conv.py:172-190)."""

    def __init__(self, in_channels, out_channels, improved=False, cached=False, add_self_loops=True,
                 normalize=True, project=False, root_weight=True, bias=True, spmm=True, transform_first=False,
                 activation=None, **kwargs):
        super().__init__()
        if activation not in (None, "relu"):
            raise ValueError("activation must be None or 'relu', got %r" % (activation,))
        # not in the reference, off by default: relu(layer(x)) with the clamp in the dense kernel's store
        # and the mask applied in the pass that sums the bias gradient (examples/sage_example.py applies
        # the activation in a pass of its own after the layer)
        self.activation = activation
        self.transform_first = bool(transform_first)      # not in the reference: see SageTransformFirstFunc
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.improved = improved
        self.cached = cached
        self.add_self_loops = add_self_loops
        self.normalize = normalize
        self.project = project
        self._cached_edge_index = None
        if project:
            self.weight_proj = nn.Parameter(torch.empty(in_channels, in_channels))
            self.bias_proj = nn.Parameter(torch.empty(in_channels))
        else:
            self.weight_proj = None
            self.bias_proj = None
        self.weight1 = nn.Parameter(torch.empty(in_channels, out_channels))
        self.root_weight = nn.Parameter(torch.empty(in_channels, out_channels)) if root_weight else None
        self.bias = nn.Parameter(torch.empty(out_channels)) if bias else None
        self.spmm = spmm
        self.reset_parameters()

    def reset_parameters(self):
        if self.project:
            glorot(self.weight_proj)
            zeros(self.bias_proj)
        glorot(self.weight1)
        glorot(self.root_weight)
        zeros(self.bias)
        self._cached_edge_index = None

    def forward(self, x, edge_index=None, edge_weight=None, csc=None, csr=None):
        out, activated = self._layer(x, edge_index, edge_weight, csc, csr)
        return torch.relu(out) if self.activation == "relu" and not activated else out

    def _layer(self, x, edge_index, edge_weight, csc, csr):
        """(output, whether the activation has been applied already)."""
        if x.is_floating_point() and x.dtype != torch.float32:
            x = x.to(torch.float32)      # the kernels and the parameters are float32; other widths are narrowed
        if csc is None or csr is None:
            cache = self._cached_edge_index
            if cache is None:
                if self.normalize:
                    edge_index, edge_weight = sage_norm(edge_index, edge_weight, x.size(0), self.improved,
                                                        self.add_self_loops)
                with torch.no_grad():
                    csc = cootocsc(edge_index, edge_weight, x.size(0))
                    csr = cootocsr(edge_index, edge_weight, x.size(0))
                if self.cached:
                    self._cached_edge_index = (edge_index, edge_weight, csr, csc)
            else:
                edge_index, edge_weight, csr, csc = cache
        reference_grad = self.spmm and _spmmcsr.REFERENCE_GRAD      # that switch lives in SpmmCsr: unfused route
        if self.weight_proj is None and x.dim() == 2 and x.dtype == torch.float32 and not reference_grad:
            # spmm=True only needs the CSR arrays (:183-184); both routes give the same product
            fwd, bwd = both_orders(None if self.spmm and csr is not None else csc, csr)
            if self.transform_first:
                return SageTransformFirstFunc.apply(x.contiguous(), self.weight1, self.root_weight, self.bias, fwd,
                                                    bwd), False
            fused = self.activation == "relu"
            return SageLayerFunc.apply(x.contiguous(), self.weight1, self.root_weight, self.bias, fwd, bwd, fused), fused
        xs = (x, x)
        if self.weight_proj is not None:
            xs = (torch.relu(xs[0] @ self.weight_proj + self.bias_proj), xs[1])
        if self.spmm:
            out = self.propagate_spmm(x=xs[0], csr=csr)
        else:
            out = self.propagate_msg(x=xs[0], csc=csc, csr=csr)
        out = xw(out, self.weight1)
        if self.root_weight is not None:
            out = out + xw(xs[1], self.root_weight)
        if self.bias is not None:
            out = add_bias(out, self.bias)
        return out, False

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}({}, {})".format(self.__class__.__name__, self.in_channels, self.out_channels)
