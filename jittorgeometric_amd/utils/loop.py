"""Self-loop handling with the semantics of the reference's
utils/loop.py:98-136, on torch tensors (runs on whatever device holds them)."""
import torch

from .num_nodes import maybe_num_nodes


def add_remaining_self_loops(edge_index, edge_weight=None, fill_value=1.0, num_nodes=None):
    """Drops the existing self-loops and appends one loop per node AT THE END
    of the edge list; a dropped loop's weight is kept as that node's loop
    weight, every other loop gets fill_value."""
    N = maybe_num_nodes(edge_index, num_nodes)
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
