"""CSC -> CSR of a sampled layer.  Same call as jittor_geometric.ops.csctocsr
(ops/csctocsr.py:27-34); arithmetic of ops/cpp/csctocsr_op.cc:36-78: row k of the result
belongs to src[k], an entry whose row index is not listed in `src` is dropped, column
indices are dst ids, and a row keeps the column order of its entries.  Runs as the stable
conversion keyed on the position of each entry's source in `src`."""
import torch

from .. import _lib
from ._common import as_i32
from .cootocsr import _convert


def csctocsr(column_offset, row_indices, dst, src):
    dev = _lib.require_gpu(column_offset, row_indices, dst, src)
    off = as_i32(column_offset, "column_offset").to(torch.int64)
    dst = as_i32(dst, "dst")
    src = as_i32(src, "src").to(torch.int64)
    E = int(off[-1].item()) if off.numel() else 0
    row = as_i32(row_indices, "row_indices").to(torch.int64)[:E]
    n_src = src.shape[0]
    row_offset = torch.zeros(n_src + 1, dtype=torch.int32, device=dev)
    column_indices = torch.zeros(E, dtype=torch.int32, device=dev)
    if E == 0 or n_src == 0:
        return row_offset, column_indices
    # position of every id in `src` (ids are assumed distinct, as the sampled layers make them)
    top = int(max(int(src.max().item()), int(row.max().item()))) + 1
    where = torch.full((top,), -1, dtype=torch.int32, device=dev)
    where[src] = torch.arange(n_src, dtype=torch.int32, device=dev)
    key = where[row]                                           # -1: dropped by the conversion
    sizes = off[1:dst.shape[0] + 1] - off[:dst.shape[0]]
    col_id = torch.repeat_interleave(dst, sizes, output_size=E)
    unit = torch.empty(E, dtype=torch.float32, device=dev)
    idx, roff, _, _ = _convert(torch.stack([key, col_id]), unit, n_src, 0)
    kept = int(roff[-1].item())
    column_indices[:kept] = idx[:kept]
    return roff, column_indices
