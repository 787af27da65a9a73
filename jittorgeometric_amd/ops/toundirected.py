"""Both directions of every edge, sorted by (row, col), one copy of each pair.
Same call as jittor_geometric.ops.toUndirected (ops/toundirected.py:15-22); the
reference (ops/cpp/toundirected_op.cc:35-60) appends (r, c, a) and (c, r, a) per
edge, std::sorts by (row, col) and keeps the first of each run of equal pairs.
std::sort does not say which of several equal pairs comes first; here the sort
is stable, so the survivor is the earliest in append order (edge i forward,
then edge i reversed, then edge i+1 ...).  The sort is two passes of the stable
COO conversion: by col, then by row."""
import torch

from ._common import as_i32
from .cootocsr import _convert
from ..utils.num_nodes import maybe_num_nodes


def _expand(off, n):
    """Key of every slot of a compressed structure with offsets `off`."""
    counts = (off[1:] - off[:-1]).to(torch.int64)
    return torch.repeat_interleave(torch.arange(off.shape[0] - 1, dtype=torch.int32, device=off.device), counts,
                                   output_size=n)


def toUndirected(edge_index, edge_attr, num_nodes):
    edge_index = as_i32(edge_index, "edge_index")
    E = edge_index.shape[1]
    V = int(maybe_num_nodes(edge_index, num_nodes))
    dev = edge_index.device
    row, col = edge_index[0], edge_index[1]
    both = torch.stack([torch.stack([row, col], dim=1).reshape(-1), torch.stack([col, row], dim=1).reshape(-1)])
    n = 2 * E
    unit = torch.empty(n, dtype=torch.float32, device=dev)          # weights ride along unused
    rows1, off1, _, perm1 = _convert(both, unit, V, 1, with_perm=True)        # by col, stable
    cols1 = _expand(off1, n)
    cols2, off2, _, perm2 = _convert(torch.stack([rows1, cols1]), unit, V, 0, with_perm=True)   # then by row
    rows2 = _expand(off2, n)
    keep = torch.ones(n, dtype=torch.bool, device=dev)
    if n > 1:
        keep[1:] = (rows2[1:] != rows2[:-1]) | (cols2[1:] != cols2[:-1])
    source = perm1.to(torch.int64)[perm2.to(torch.int64)][keep]      # position in append order
    new_index = torch.stack([rows2[keep], cols2[keep]])
    attr = edge_attr.reshape(-1)[source // 2]
    # the reference gives the attributes the shape [1, length] (toundirected_op.cc:47-50)
    return new_index, attr.reshape(1, -1)
