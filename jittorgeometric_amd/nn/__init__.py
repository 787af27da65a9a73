from .conv import (APPNP, BernNet, ChebConv, ChebNetII, ClusterGCNConv, EvenNet, GATConv, GCN2Conv, GCNConv, GPRGNN, LightGCNConv,  # noqa: F401
                   MessagePassingNts, SAGEConv, SGConv, clustergcn_norm, gcn_norm, sage_norm)
from .loss import cross_entropy_loss, nll_loss  # noqa: F401
