from .gcn_conv import GCNConv, gcn_norm  # noqa: F401
from .sage_conv import SAGEConv, sage_norm  # noqa: F401
