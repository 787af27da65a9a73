from .appnp_conv import APPNP  # noqa: F401
from .bernnet_conv import BernNet  # noqa: F401
from .cheb_conv import ChebConv  # noqa: F401
from .chebnet2_conv import ChebNetII  # noqa: F401
from .clustergcn_conv import ClusterGCNConv, clustergcn_norm  # noqa: F401
from .even_conv import EvenNet  # noqa: F401
from .gat_conv import GATConv  # noqa: F401
from .gcn2_conv import GCN2Conv  # noqa: F401
from .gcn_conv import GCNConv, gcn_norm  # noqa: F401
from .gpr_conv import GPRGNN  # noqa: F401
from .lightgcn_conv import LightGCNConv  # noqa: F401
from .message_passiong_nts import MessagePassingNts  # noqa: F401
from .sage_conv import SAGEConv, sage_norm  # noqa: F401
from .sg_conv import SGConv  # noqa: F401
