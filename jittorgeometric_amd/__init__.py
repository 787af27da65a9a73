"""MI355X-native sparse message-passing core with the call signatures of
jittor_geometric.ops / jittor_geometric.nn.conv (GCNConv, GATConv, SAGEConv).

Host side: PyTorch-ROCm tensors for device memory and streams.  Compute: the
hand-written gfx950 kernels of libjgamd.so, reached through ctypes with raw
device pointers.  There is no CPU implementation behind these operators:
calling them on CPU tensors, or without the built library, raises.
"""
from ._lib import JgamdError  # noqa: F401
from .data import CSC, CSR  # noqa: F401
from . import ops  # noqa: F401

__version__ = "0.1.0"
