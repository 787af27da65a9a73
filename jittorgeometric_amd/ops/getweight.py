"""Symmetric-normalisation weights of a layer's CSC arrays.  Same call as
jittor_geometric.ops.getweight (ops/getweight.py:29-37); arithmetic of
ops/cpp/getweight_op.cc:36-82: in-degree of dst[i] += size of column i, out-degree of
every row index += 1, weight = 1 / (sqrtf(out[src]) * sqrtf(in[dst])).  The kernels are in
csrc/sample.hip; csc_layer_src is accepted and, as in the reference's loop, not read."""
import torch

from .. import _lib
from ._common import as_i32


def getweight(vtx_size, csc_layer_dst, csc_layer_src, csc_layer_column_offset, csc_layer_row_indices):
    lib = _lib.load()
    dev = _lib.require_gpu(csc_layer_dst, csc_layer_column_offset, csc_layer_row_indices)
    dst = as_i32(csc_layer_dst, "csc_layer_dst")
    off = as_i32(csc_layer_column_offset, "csc_layer_column_offset")
    row = as_i32(csc_layer_row_indices, "csc_layer_row_indices")
    n = dst.shape[0]
    if off.shape[0] < n + 1:
        raise _lib.JgamdError("getweight: %d offsets for %d destinations" % (off.shape[0], n))
    E = int(off[-1].item()) if off.numel() else 0       # the reference sizes the result the same way (:32)
    if E < 0 or E > row.shape[0]:
        raise _lib.JgamdError("getweight: last offset %d, %d row indices" % (E, row.shape[0]))
    w = torch.empty(E, dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_getweight_workspace, int(vtx_size))
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_getweight(_lib.ptr(dst), _lib.ptr(off), _lib.ptr(row), n, int(vtx_size), E, _lib.ptr(w),
                                   _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    return w
