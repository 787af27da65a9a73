"""Per-destination neighbour counts capped at the fanout.  Same call as
jittor_geometric.ops.gpuinitco (ops/gpuinitco.py:30-36); follows the GPU branch of
ops/cpp/gpuinitco_op.cc:37-50: out[i+1] = min(degree of dst[i], fanout), out[0] = 0 (the
caller turns the counts into offsets)."""
import torch

from .. import _lib
from ._common import as_i32


def gpuinitco(dst_size, fanout_i, csc_layer_dst, csc_global_column_offset):
    dev = _lib.require_gpu(csc_layer_dst, csc_global_column_offset)
    dst = as_i32(csc_layer_dst, "csc_layer_dst").to(torch.int64)[:dst_size]
    g = as_i32(csc_global_column_offset, "csc_global_column_offset")
    out = torch.zeros(dst_size + 1, dtype=torch.int32, device=dev)
    out[1:] = torch.clamp(g[dst + 1] - g[dst], max=int(fanout_i))
    return out
