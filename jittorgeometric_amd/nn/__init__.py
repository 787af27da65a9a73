from .conv import APPNP, GATConv, GCNConv, MessagePassingNts, SAGEConv, SGConv, gcn_norm, sage_norm  # noqa: F401
