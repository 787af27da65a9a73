from .appnp_conv import APPNP  # noqa: F401
from .gat_conv import GATConv  # noqa: F401
from .gcn_conv import GCNConv, gcn_norm  # noqa: F401
from .gpr_conv import GPRGNN  # noqa: F401
from .message_passiong_nts import MessagePassingNts  # noqa: F401
from .sage_conv import SAGEConv, sage_norm  # noqa: F401
from .sg_conv import SGConv  # noqa: F401
