"""COO -> CSC.  Same call as jittor_geometric.ops.cootocsc
(ops/cootocsc.py:29-36)."""
from .cootocsr import cootocsc  # noqa: F401
