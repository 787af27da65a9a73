"""GCN layer with the constructor and call signature of the reference's
GCNConv (nn/conv/gcn_conv.py:40-116) on torch tensors."""
import torch
from torch import nn

from ...ops import SpmmCsr, aggregateWithWeight, cootocsc
from ...ops import spmmcsr as _spmmcsr
from ...ops.propagate import aggregate_bias
from ...utils import add_remaining_self_loops
from ...utils.num_nodes import maybe_num_nodes
from ...ops._common import both_orders, spmm, spmm_axpby
from ..dense import add_bias, column_sum, relu_backward_column_sum, rows_times, xt_g, xw
from ..inits import glorot, zeros


def _degree_by_col(edge_index, edge_weight, num_nodes):
    """deg[v] = sum of the weights of the edges whose destination is v
    (jt.scatter(..., reduce='add') by col in gcn_conv.py:33-34): the column sum
    of the CSC arrays, i.e. conversion + gather-sum, in a fixed order and
    without the same-address atomics a hub destination causes."""
    return _degree_and_order(edge_index, edge_weight, num_nodes)[0]


def _degree_and_order(edge_index, edge_weight, num_nodes):
    """(deg, order): the degrees as above and, for a contiguous int32 edge list, what the sort by
    destination produced (row indices, offsets, weights in slot order), so that the conversion
    the caller runs next on the same edges with the normalised weights need not sort again."""
    from ...ops._common import spmm
    from ...ops.cootocsr import _convert
    if edge_index.shape[1] == 0:
        return torch.zeros((num_nodes,), dtype=torch.float32, device=edge_weight.device), None
    keep = edge_index.dtype == torch.int32 and edge_index.is_contiguous()
    idx, off, w, _ = _convert(edge_index, edge_weight, num_nodes, 1)
    deg = spmm(off, None, None, w.view(-1, 1), num_nodes).view(-1)
    return deg, ((idx, off, w) if keep else None)


def _scale(edge_index, edge_weight, by_row, by_col, num_nodes):
    """by_row[row] * w * by_col[col] (either factor may be None)."""
    from ... import _lib
    lib = _lib.load()
    dev = _lib.require_gpu(edge_index, edge_weight)
    ei = (edge_index if edge_index.dtype == torch.int32 else edge_index.to(torch.int32)).contiguous()
    w = edge_weight.contiguous()
    out = torch.empty_like(w)
    _lib.check(lib.jgamd_scale_edge_weights(_lib.ptr(ei), _lib.ptr(w), _lib.ptr(by_row), _lib.ptr(by_col), ei.shape[1],
                                            num_nodes, _lib.ptr(out), _lib.stream_ptr(dev)))
    return out


def _degree_norm(edge_index, edge_weight, num_nodes, improved, add_self_loops, power):
    """(edge_index, edge_weight, deg^power with inf -> 0) after the optional self-loop step."""
    from ... import _lib
    lib = _lib.load()
    dev = _lib.require_gpu(edge_index, edge_weight)
    fill_value = 2.0 if improved else 1.0
    num_nodes = int(maybe_num_nodes(edge_index, num_nodes))
    if edge_weight is None:
        edge_weight = torch.ones((edge_index.size(1),), dtype=torch.float32, device=dev)
    elif edge_weight.dtype != torch.float32:
        edge_weight = edge_weight.to(torch.float32)
    if add_self_loops:
        edge_index, edge_weight = add_remaining_self_loops(edge_index, edge_weight, fill_value, num_nodes)
    deg, order = _degree_and_order(edge_index, edge_weight, num_nodes)
    dinv = torch.empty_like(deg)
    _lib.check(lib.jgamd_degree_power(_lib.ptr(deg), num_nodes, float(power), _lib.ptr(dinv), _lib.stream_ptr(dev)))
    return edge_index, edge_weight, dinv, order


def _normalised(edge_index, edge_weight, by_row, by_col, num_nodes, order):
    """(edge_index, by_row[row] * w * by_col[col]); the sort by destination that the degree sum
    needed is handed on to the conversion that follows."""
    weights = _scale(edge_index, edge_weight, by_row, by_col, num_nodes)
    if order is not None:
        from ...ops.cootocsr import remember_order
        remember_order(edge_index, weights, num_nodes, 1, order[0], order[1], order[2], by_row, by_col)
    return edge_index, weights


def gcn_norm(edge_index, edge_weight=None, num_nodes=None, improved=False, add_self_loops=True, dtype=None):
    """Symmetric normalisation w = d^-1/2[row] * w * d^-1/2[col] with the
    degree summed by column (nn/conv/gcn_conv.py:18-37)."""
    edge_index, edge_weight, dis, order = _degree_norm(edge_index, edge_weight, num_nodes, improved, add_self_loops, -0.5)
    return _normalised(edge_index, edge_weight, dis, dis, dis.shape[0], order)


class GcnLayerFunc(torch.autograd.Function):
    """A_hat (x W) + b as one autograd node (gcn_conv.py:94-102 builds it from three: dense
    product, product over the graph, addition).  Forward: the dense kernel, then the product with
    the bias added in its row store.  Backward: g_W = x^T (A_hat^T g) and g_x = (A_hat^T g) W^T share
    one transposed product at the output width.  When x needs no gradient (the first layer of a
    model) and the layer widens, g_W = (A_hat x)^T g instead: the same sum in another order, with
    the product over the graph at the narrower input width."""

    @staticmethod
    def forward(ctx, x, weight, bias, fwd, bwd, relu=False):
        h = rows_times(x, weight, pad_rows=True)      # gathered next: rows of an odd width start on a line
        if bias is not None or relu:
            out = spmm_axpby(fwd[0], fwd[1], fwd[2], h, x.shape[0], 1.0, 1.0, bias, relu)
        else:
            out = spmm(fwd[0], fwd[1], fwd[2], h, x.shape[0])
        ctx.fwd, ctx.bwd, ctx.relu = fwd, bwd, relu
        if relu:
            ctx.save_for_backward(x, weight, out)       # the mask of the activation is the output's sign
        else:
            ctx.save_for_backward(x, weight)
        return out

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors[:2]
        g = g.contiguous()
        need_x, need_w, need_b = ctx.needs_input_grad[:3]
        gx = gw = gb = None
        if ctx.relu:
            # the gradient in front of the activation and the bias gradient in one pass over g
            out = ctx.saved_tensors[2]
            if g.dtype == torch.float32:
                g, gb = relu_backward_column_sum(g, out)
            else:
                g = g * (out > 0)
                gb = g.sum(0)
            if not need_b:
                gb = None
        elif need_b:
            gb = column_sum(g) if g.dtype == torch.float32 else g.sum(0)
        f_in, f_out = weight.shape
        if need_x or (need_w and f_out <= f_in):
            off, idx, w = ctx.bwd
            gh = spmm(off, idx, w, g, g.shape[0])
            if need_w:
                gw = xt_g(x, gh)
            if need_x:
                gx = rows_times(gh, weight.t())
        elif need_w:
            off, idx, w = ctx.fwd
            gw = xt_g(spmm(off, idx, w, x, x.shape[0]), g)
        return gx, gw, gb, None, None, None


class GCNConv(nn.Module):
    """out = A_hat (x W) + b.  `spmm=True` routes through SpmmCsr(x, csr), as
    the reference does on a GPU (gcn_conv.py:96-97); `spmm=False` through
    aggregateWithWeight(x, csc, csr) (gcn_conv.py:98-99).

    `aggregate_first=True` (not in the reference, off by default) evaluates the same
    expression as (A_hat x) W + b: the product over the graph then runs at the input
    width, which is the cheaper order when in_channels < out_channels (100 -> 256:
    half the gathered bytes); the dense product takes the bias in its own pass.  The
    two orders differ in rounding only.

    `activation="relu"` (not in the reference, off by default) returns relu(A_hat (x W) + b) with the
    clamp applied in the product's row store and, in the backward pass, the activation's mask
    applied in the pass that sums the bias gradient: what examples/gcn_example.py:84-90 writes as
    `x = nn.relu(self.conv1(x, csc, csr))`, without the two passes over [V,F] of a separate
    activation.  Same values as relu(layer(x))."""

    def __init__(self, in_channels, out_channels, bias=True, spmm=True, aggregate_first=False, activation=None,
                 **kwargs):
        super().__init__()
        if activation not in (None, "relu"):
            raise ValueError("activation must be None or 'relu', got %r" % (activation,))
        self.activation = activation
        self.aggregate_first = bool(aggregate_first)
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.weight = nn.Parameter(torch.empty(in_channels, out_channels))
        self.bias = nn.Parameter(torch.empty(out_channels)) if bias else None
        self.spmm = spmm
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        zeros(self.bias)

    def forward(self, x, csc, csr):
        if self.activation == "relu" and self._fused_route(x):
            fwd, bwd = both_orders(None if self.spmm and csr is not None else csc, csr)
            return GcnLayerFunc.apply(x.to(torch.float32).contiguous(), self.weight, self.bias, fwd, bwd, True)
        out = self._layer(x, csc, csr)
        return torch.relu(out) if self.activation == "relu" else out

    def _fused_route(self, x):
        """The layer runs as one autograd node (dense kernel, product with the bias in its row store)."""
        return (not self.aggregate_first and x.dim() == 2 and x.is_floating_point()
                and not (self.spmm and _spmmcsr.REFERENCE_GRAD))

    def _layer(self, x, csc, csr):
        if x.is_floating_point() and x.dtype != torch.float32:
            x = x.to(torch.float32)      # the kernels and the parameters are float32; other widths are narrowed
        if self.aggregate_first and x.dim() == 2:
            agg = self.propagate_spmm(x=x, csr=csr) if self.spmm else self.propagate_msg(x=x, csc=csc, csr=csr)
            return xw(agg, self.weight, self.bias)
        if x.dim() == 2 and x.dtype == torch.float32 and not (self.spmm and _spmmcsr.REFERENCE_GRAD):
            # spmm=True only needs the CSR (:96-97); both routes give the same product
            fwd, bwd = both_orders(None if self.spmm and csr is not None else csc, csr)
            return GcnLayerFunc.apply(x.contiguous(), self.weight, self.bias, fwd, bwd, False)
        x = xw(x, self.weight)
        if self.bias is not None and x.dim() == 2 and not (self.spmm and _spmmcsr.REFERENCE_GRAD):
            # product and bias in one kernel; spmm=True only needs the CSR (:96-97)
            return aggregate_bias(x, self.bias, None if self.spmm and csr is not None else csc, csr)
        if self.spmm:
            out = self.propagate_spmm(x=x, csr=csr)
        else:
            out = self.propagate_msg(x=x, csc=csc, csr=csr)
        if self.bias is not None:
            out = add_bias(out, self.bias)
        return out

    execute = forward

    def propagate_msg(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def propagate_spmm(self, x, csr):
        return SpmmCsr(x, csr)

    def __repr__(self):
        return "{}({}, {})".format(self.__class__.__name__, self.in_channels, self.out_channels)
