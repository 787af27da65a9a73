"""Operators with the names and argument order of jittor_geometric.ops
(ops/__init__.py:5-13)."""
from .aggregateWithWeight import aggregateWithWeight  # noqa: F401
from .cootocsc import cootocsc  # noqa: F401
from .cootocsr import cootocsr  # noqa: F401
from .spmmcsr import SpmmCsr  # noqa: F401
