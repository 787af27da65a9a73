"""Base class with the hook names of the reference's MessagePassingNts
(nn/conv/message_passiong_nts.py:16-67): subclasses override the four stages
and call the operators of jittorgeometric_amd.ops."""
from torch import nn

from ...ops import aggregateWithWeight


class MessagePassingNts(nn.Module):
    def __init__(self, aggr="add", flow="source_to_target", node_dim=-2):
        super().__init__()

    def propagate(self, x):
        return

    def aggregate_with_weight(self, x, csc, csr):
        return aggregateWithWeight(x, csc, csr)

    def scatter_to_edge(self, x):
        return

    def edge_forward(self, x):
        return

    def scatter_to_vertex(self, x, csc):
        return

    def vertex_forward(self, x):
        return
