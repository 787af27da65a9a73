"""Symmetric-normalisation weights of a layer's CSC arrays.  Same call as
jittor_geometric.ops.getweight (ops/getweight.py:29-37); arithmetic of
ops/cpp/getweight_op.cc:36-82: in-degree of dst[i] += size of column i, out-degree of
every row index += 1, weight = 1 / (sqrtf(out[src]) * sqrtf(in[dst]))."""
import torch

from .. import _lib
from ._common import as_i32


def getweight(vtx_size, csc_layer_dst, csc_layer_src, csc_layer_column_offset, csc_layer_row_indices):
    dev = _lib.require_gpu(csc_layer_dst, csc_layer_column_offset, csc_layer_row_indices)
    dst = as_i32(csc_layer_dst, "csc_layer_dst").to(torch.int64)
    off = as_i32(csc_layer_column_offset, "csc_layer_column_offset").to(torch.int64)
    n = dst.shape[0]
    E = int(off[-1].item()) if off.numel() else 0       # the reference sizes the result the same way (:32)
    row = as_i32(csc_layer_row_indices, "csc_layer_row_indices").to(torch.int64)[:E]
    sizes = off[1:n + 1] - off[:n]
    ins = torch.zeros(vtx_size, dtype=torch.int64, device=dev).index_add_(0, dst, sizes)
    outs = torch.bincount(row, minlength=vtx_size)
    col_of_entry = torch.repeat_interleave(dst, sizes, output_size=E)
    w = 1.0 / (outs[row].to(torch.float32).sqrt() * ins[col_of_entry].to(torch.float32).sqrt())
    return w
