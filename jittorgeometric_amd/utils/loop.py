"""Self-loop handling with the semantics of the reference's
utils/loop.py:98-136.  GPU tensors go through the library's kernels
(csrc/graph_norm.hip); anything else through the same steps in torch."""
import torch

from .num_nodes import maybe_num_nodes


def _on_gpu(edge_index, edge_weight, N, fill_value):
    from .. import _lib
    lib = _lib.load()
    dev = edge_index.device
    ei = edge_index if edge_index.dtype == torch.int32 else edge_index.to(torch.int32)
    ei = ei.contiguous()
    w = None
    if edge_weight is not None:
        w = edge_weight.reshape(-1).contiguous()
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


def add_remaining_self_loops(edge_index, edge_weight=None, fill_value=1.0, num_nodes=None):
    """Drops the existing self-loops and appends one loop per node AT THE END
    of the edge list; a dropped loop's weight is kept as that node's loop
    weight, every other loop gets fill_value."""
    N = maybe_num_nodes(edge_index, num_nodes)
    if edge_index.is_cuda and (edge_weight is None or (edge_weight.is_cuda and edge_weight.dtype == torch.float32)):
        return _on_gpu(edge_index, edge_weight, int(N), fill_value)
    row, col = edge_index[0], edge_index[1]
    mask = row != col
    loop_index = torch.arange(0, N, dtype=row.dtype, device=row.device)
    loop_index = loop_index.unsqueeze(0).repeat(2, 1)
    out_index = torch.cat([edge_index[:, mask], loop_index], dim=1)
    if edge_weight is not None:
        inv_mask = ~mask
        loop_weight = torch.full((N,), fill_value, dtype=edge_weight.dtype, device=edge_weight.device)
        remaining = edge_weight[inv_mask]
        if remaining.numel() > 0:
            loop_weight[row[inv_mask].long()] = remaining
        edge_weight = torch.cat([edge_weight[mask], loop_weight], dim=0)
    return out_index, edge_weight
