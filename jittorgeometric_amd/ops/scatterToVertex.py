"""Edge -> vertex sum over the CSC arrays.  Same call as
jittor_geometric.ops.ScatterToVertex (ops/scatterToVertex.py:23-50): whatever
`flow` says, the reference sums every edge into its destination
(edgetovertex flag 1, scatterToVertex.py:38), and so does this."""
import torch

from ._common import csc_arrays
from .scatterToEdge import edge_to_vertex, scatter_to_edge


class ScatterToVertexFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csc, flow):
        ctx.csc = csc
        v_num = csc_arrays(csc)[0].shape[0] - 1
        return edge_to_vertex(x, csc, 1, v_num)

    @staticmethod
    def backward(ctx, grad_output):
        return scatter_to_edge(grad_output, ctx.csc, 1), None, None


def ScatterToVertex(x, csc, flow):
    return ScatterToVertexFunc.apply(x, csc, flow)
