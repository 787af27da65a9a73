"""Self-loop handling with the semantics of the reference's
utils/loop.py:98-136, run by the library's kernels (csrc/graph_norm.hip)."""
import torch

from .num_nodes import maybe_num_nodes


def add_remaining_self_loops(edge_index, edge_weight=None, fill_value=1.0, num_nodes=None):
    """Drops the existing self-loops and appends one loop per node AT THE END
    of the edge list; a dropped loop's weight is kept as that node's loop
    weight, every other loop gets fill_value.  GPU tensors only."""
    from .. import _lib
    lib = _lib.load()
    dev = _lib.require_gpu(edge_index, edge_weight)
    N = int(maybe_num_nodes(edge_index, num_nodes))
    if edge_index.dim() != 2 or edge_index.shape[0] != 2:
        raise _lib.JgamdError("edge_index must be [2, E], got %s" % (tuple(edge_index.shape),))
    ei = (edge_index if edge_index.dtype == torch.int32 else edge_index.to(torch.int32)).contiguous()
    w = None
    if edge_weight is not None:
        w = edge_weight.reshape(-1)
        w = (w if w.dtype == torch.float32 else w.to(torch.float32)).contiguous()
    E = ei.shape[1]
    buf = torch.empty(2 * (E + N), dtype=torch.int32, device=dev)
    out_w = torch.empty(E + N, dtype=torch.float32, device=dev)
    kept = torch.empty(1, dtype=torch.int32, device=dev)
    nbytes = _lib.query(lib.jgamd_add_remaining_self_loops_workspace, E, N)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_add_remaining_self_loops(_lib.ptr(ei), _lib.ptr(w), E, N, float(fill_value), _lib.ptr(buf),
                                                  _lib.ptr(out_w), _lib.ptr(kept), _lib.ptr(ws), nbytes,
                                                  _lib.stream_ptr(dev)))
    n_out = int(kept.item()) + N                      # the result's size is data-dependent, as in the reference
    out_index = buf[:2 * n_out].view(2, n_out)
    if edge_index.dtype != torch.int32:
        out_index = out_index.to(edge_index.dtype)
    return out_index, (out_w[:n_out] if edge_weight is not None else None)


def remove_self_loops(edge_index, edge_attr=None):
    """The edges with two different endpoints, in their order (utils/loop.py:22-38)."""
    mask = edge_index[0] != edge_index[1]
    edge_index = edge_index[:, mask]
    return edge_index, (None if edge_attr is None else edge_attr[mask])


def add_self_loops(edge_index, edge_weight=None, fill_value=1.0, num_nodes=None):
    """One loop (i, i) per node appended after the edges, with weight fill_value when the
    edges carry weights (utils/loop.py:64-95); existing loops stay."""
    N = int(maybe_num_nodes(edge_index, num_nodes))
    loop_index = torch.arange(N, dtype=edge_index.dtype, device=edge_index.device).unsqueeze(0).repeat(2, 1)
    if edge_weight is not None:
        if edge_weight.numel() != edge_index.size(1):
            raise ValueError("add_self_loops: %d weights for %d edges" % (edge_weight.numel(), edge_index.size(1)))
        loop_weight = torch.full((N,), fill_value, dtype=edge_weight.dtype, device=edge_weight.device)
        edge_weight = torch.cat([edge_weight, loop_weight], dim=0)
    return torch.cat([edge_index, loop_index], dim=1), edge_weight
