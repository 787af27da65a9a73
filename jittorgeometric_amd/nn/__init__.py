from .conv import GCNConv, SAGEConv, gcn_norm, sage_norm  # noqa: F401
