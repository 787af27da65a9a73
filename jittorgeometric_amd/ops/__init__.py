"""Operators with the names and argument order of jittor_geometric.ops
(ops/__init__.py:5-18), plus the fused GAT core and the fused propagation hops."""
from .aggregateWithWeight import aggregateWithWeight  # noqa: F401
from .cootocsc import cootocsc  # noqa: F401
from .cootocsr import cootocsr  # noqa: F401
from .csctocsr import csctocsr  # noqa: F401
from .edgesoftmax import EdgeSoftmax  # noqa: F401
from .gat import gat_aggregate  # noqa: F401
from .getweight import getweight  # noqa: F401
from .gpuinitco import gpuinitco  # noqa: F401
from .sampleprocessing import sampleprocessing  # noqa: F401
from .saparse_ops import from_nodes, to_nodes  # noqa: F401
from .scatterToEdge import ScatterToEdge  # noqa: F401
from .scatterToVertex import ScatterToVertex  # noqa: F401
from .propagate import aggregate_bias, appnp_propagate, propagate_axpby  # noqa: F401
from .spmmcoo import SpmmCoo  # noqa: F401
from .spmmcsr import SpmmCsr  # noqa: F401
from .toundirected import toUndirected  # noqa: F401
