"""COO -> CSR.  Same call as jittor_geometric.ops.cootocsr
(ops/cootocsr.py:28-35); the arithmetic of ops/cpp/cootocsr_op.cc:24-57 runs
as the stable two-level counting sort of csrc/convert.hip."""
import torch

from .. import _lib
from ..data import CSC, CSR
from ._common import as_f32, as_i32


def _convert(edge_index, edge_weight, v_num, key_row, with_perm=False):
    lib = _lib.load()
    dev = _lib.require_gpu(edge_index, edge_weight)
    if edge_index.dim() != 2 or edge_index.shape[0] != 2:
        raise _lib.JgamdError("edge_index must be [2, E], got %s" % (tuple(edge_index.shape),))
    edge_index = as_i32(edge_index, "edge_index")
    edge_weight = as_f32(edge_weight, "edge_weight").reshape(-1)
    E = edge_index.shape[1]
    if edge_weight.shape[0] != E:
        raise _lib.JgamdError("edge_weight has %d entries for %d edges" % (edge_weight.shape[0], E))
    v_num = int(v_num)
    # the reference hands zero-filled outputs to the op (ops/cootocsr.py:30-32); the library
    # writes every slot (slots past off[V], left over when keys were dropped, as zeros)
    idx = torch.empty(E, dtype=torch.int32, device=dev)
    off = torch.empty(v_num + 1, dtype=torch.int32, device=dev)
    w = torch.empty(E, dtype=torch.float32, device=dev)
    perm = torch.empty(E, dtype=torch.int32, device=dev) if with_perm else None
    nbytes = _lib.query(lib.jgamd_coo_to_csx_workspace, E, v_num, 1 if with_perm else 0)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_coo_to_csx(_lib.ptr(edge_index), _lib.ptr(edge_weight), E, v_num, key_row, _lib.ptr(idx),
                                    _lib.ptr(off), _lib.ptr(w), _lib.ptr(perm), _lib.ptr(ws), nbytes,
                                    _lib.stream_ptr(dev)))
    return idx, off, w, perm


def cootocsr(edge_index, edge_weight, v_num):
    """Returns CSR(column_indices, row_offset, edge_weight); rows keep the
    input order of their edges."""
    idx, off, w, _ = _convert(edge_index, edge_weight, v_num, 0)
    return CSR(idx, off, w)


def cootocsc(edge_index, edge_weight, v_num):
    """COO -> CSC (ops/cootocsc.py:29-36, ops/cpp/cootocsc_op.cc:23-53)."""
    idx, off, w, _ = _convert(edge_index, edge_weight, v_num, 1)
    return CSC(idx, off, w)
