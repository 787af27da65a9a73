"""Graph Laplacian as an edge list, with the call and the semantics of the
reference's utils/get_laplacian.py:9-81: self-loops removed, the degree summed
by row (the source endpoint), then

    None   L = D - A
    'sym'  L = I - D^-1/2 A D^-1/2
    'rw'   L = I - D^-1 A

with the N diagonal entries appended after the other edges.  The degree is the
library's fixed-order segment sum (conversion + gather-sum, no float atomics),
the scaling its per-edge kernel."""
import torch

from .loop import add_self_loops, remove_self_loops
from .num_nodes import maybe_num_nodes


def get_laplacian(edge_index, edge_weight=None, normalization=None, dtype=None, num_nodes=None):
    from .. import _lib
    from ..nn.conv.gcn_conv import _degree_by_col, _scale
    if normalization not in (None, "sym", "rw"):
        raise ValueError("Invalid normalization %r" % (normalization,))
    lib = _lib.load()
    dev = _lib.require_gpu(edge_index, edge_weight)
    edge_index, edge_weight = remove_self_loops(edge_index, edge_weight)
    if edge_weight is None:
        edge_weight = torch.ones((edge_index.size(1),), dtype=torch.float32, device=dev)
    elif edge_weight.dtype != torch.float32:
        edge_weight = edge_weight.to(torch.float32)
    N = int(maybe_num_nodes(edge_index, num_nodes))
    # summed by row: the same segment sum as the by-column degree of the flipped list
    deg = _degree_by_col(edge_index.flip(0).contiguous(), edge_weight, N)
    if normalization is None:
        edge_index, _ = add_self_loops(edge_index, num_nodes=N)
        return edge_index, torch.cat([-edge_weight, deg], dim=0)
    dinv = torch.empty_like(deg)
    power = -0.5 if normalization == "sym" else -1.0
    _lib.check(lib.jgamd_degree_power(_lib.ptr(deg), N, power, _lib.ptr(dinv), _lib.stream_ptr(dev)))   # inf -> 0
    if edge_index.shape[1]:
        scaled = _scale(edge_index, edge_weight, dinv, dinv if normalization == "sym" else None, N)
    else:
        scaled = edge_weight
    return add_self_loops(edge_index, -scaled, fill_value=1.0, num_nodes=N)
