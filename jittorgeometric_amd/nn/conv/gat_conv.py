"""GAT layer with the constructor and call signature of the reference's
GATConv (nn/conv/gat_conv.py:18-93) on torch tensors.

`fused=True` (default) computes propagate() with the single-pass kernels of
csrc/gat.hip; `fused=False` runs the reference's own operator chain
(ScatterToEdge, EdgeSoftmax, ScatterToVertex), which is also what shapes
outside the fused kernels' range fall back to."""
import torch
from torch import nn

from ...ops import EdgeSoftmax, ScatterToEdge, ScatterToVertex, gat_aggregate
from ...ops.gat import fused_supported
from ..dense import xw
from ..inits import glorot
from .message_passiong_nts import MessagePassingNts


class GATConv(MessagePassingNts):
    """Single attention head, no bias, ReLU inside vertex_forward — as in the
    reference (gat_conv.py:46, :85-88).  `e_num` is accepted and unused there
    too (gat_conv.py:27)."""

    def __init__(self, in_channels, out_channels, e_num=None, improved=False, cached=False,
                 add_self_loops=True, normalize=True, bias=True, fused=True, **kwargs):
        super().__init__(**kwargs)
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.improved = improved
        self.cached = cached
        self.add_self_loops = add_self_loops
        self.normalize = normalize
        self.fused = fused
        self.weight = nn.Parameter(torch.empty(in_channels, out_channels))
        self.edge_weight = nn.Parameter(torch.empty(2 * out_channels, 1))
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        glorot(self.edge_weight)

    def forward(self, x, csc):
        out = self.vertex_forward(x)
        return self.propagate(x=out, csc=csc)

    execute = forward

    def propagate(self, x, csc):
        C = self.out_channels
        if self.fused and fused_supported(1, C):
            a_src = self.edge_weight[:C, 0].reshape(1, C)
            a_dst = self.edge_weight[C:, 0].reshape(1, C)
            return gat_aggregate(x.reshape(-1, 1, C), csc, a_src, a_dst, 0.2).reshape(-1, C)
        e_msg = self.scatter_to_edge(x, csc)
        out = self.edge_forward(e_msg, csc)
        return self.scatter_to_vertex(out, csc)

    def scatter_to_edge(self, x, csc):
        out1 = ScatterToEdge(x, csc, "src")
        out2 = ScatterToEdge(x, csc, "dst")
        return torch.cat([out1, out2], dim=1)

    def edge_forward(self, x, csc):
        out = x @ self.edge_weight
        m = torch.nn.functional.leaky_relu(out, 0.2)
        a = EdgeSoftmax(m, csc)
        half_dim = int(x.size(1) / 2)
        return x[:, 0:half_dim] * a

    def scatter_to_vertex(self, edge, csc):
        return ScatterToVertex(edge, csc, "src")

    def vertex_forward(self, x):
        return torch.relu(xw(x, self.weight))

    def __repr__(self):
        return "{}({}, {})".format(self.__class__.__name__, self.in_channels, self.out_channels)
