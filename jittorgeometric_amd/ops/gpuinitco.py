"""Per-destination neighbour counts capped at the fanout.  Same call as
jittor_geometric.ops.gpuinitco (ops/gpuinitco.py:30-36); follows the GPU branch of
ops/cpp/gpuinitco_op.cc:37-50: out[i+1] = min(degree of dst[i], fanout), out[0] = 0 (the
caller turns the counts into offsets).  One kernel of csrc/sample.hip."""
import torch

from .. import _lib
from ._common import as_i32


def gpuinitco(dst_size, fanout_i, csc_layer_dst, csc_global_column_offset):
    lib = _lib.load()
    dev = _lib.require_gpu(csc_layer_dst, csc_global_column_offset)
    dst = as_i32(csc_layer_dst, "csc_layer_dst")
    g = as_i32(csc_global_column_offset, "csc_global_column_offset")
    dst_size = int(dst_size)
    if dst_size < 0 or dst_size > dst.shape[0]:
        raise _lib.JgamdError("gpuinitco: dst_size %d, %d destinations given" % (dst_size, dst.shape[0]))
    out = torch.empty(dst_size + 1, dtype=torch.int32, device=dev)
    _lib.check(lib.jgamd_layer_column_counts(_lib.ptr(dst), _lib.ptr(g), dst_size, max(g.shape[0] - 1, 0),
                                             int(fanout_i), _lib.ptr(out), _lib.stream_ptr(dev)))
    return out
