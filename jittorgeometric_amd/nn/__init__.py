from .conv import APPNP, GATConv, GCNConv, GPRGNN, MessagePassingNts, SAGEConv, SGConv, gcn_norm, sage_norm  # noqa: F401
