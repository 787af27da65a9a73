from .conv import APPNP, GATConv, GCNConv, GPRGNN, MessagePassingNts, SAGEConv, SGConv, gcn_norm, sage_norm  # noqa: F401
from .loss import cross_entropy_loss, nll_loss  # noqa: F401
