from .conv import GATConv, GCNConv, MessagePassingNts, SAGEConv, gcn_norm, sage_norm  # noqa: F401
