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


def remember_order(edge_index, edge_weight, v_num, key_row, idx, off, w_sorted, by_idx, by_seg):
    """Keeps the outcome of a conversion of `edge_index` on the weight tensor that a later
    conversion of the same edge list will bring.  The normalisations (gcn_norm, sage_norm) sort
    the edge list by destination to sum the degrees and return, for the same edges, the weights
    by_row[row] * w * by_col[col]; the caller then converts that result again
    (examples/gcn_example.py:48-59).  The second sort would find the same slots: its index and
    offset arrays are the first one's, and its weights are the first one's scaled slot by slot
    (jgamd_scale_csx_weights: the same three factors in the same order, so the same bits)."""
    edge_weight._jgamd_order = (edge_index, edge_index._version, edge_weight._version, int(v_num), key_row, idx, off,
                                w_sorted, by_idx, by_seg)


def _remembered(edge_index, edge_weight, v_num, key_row):
    """(idx, off, w) from an order kept by remember_order for exactly these tensors, or None.  The
    arrays are handed out once (two holders must not share memory)."""
    kept = getattr(edge_weight, "_jgamd_order", None)
    if kept is None:
        return None
    ei, ei_version, w_version, V, key, idx, off, w_sorted, by_idx, by_seg = kept
    if (ei is not edge_index or ei._version != ei_version or edge_weight._version != w_version or V != int(v_num)
            or key != key_row or edge_weight.dim() != 1 or edge_weight.dtype != torch.float32
            or edge_weight.shape[0] != idx.shape[0]):
        return None
    edge_weight._jgamd_order = None
    lib = _lib.load()
    dev = edge_weight.device
    E = idx.shape[0]
    if E == 0:
        return idx, off, w_sorted
    w = torch.empty(E, dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_scale_csx_weights_workspace, E)
    ws = _lib.workspace(nbytes, dev)
    n_factor = (by_idx if by_idx is not None else by_seg).shape[0]
    _lib.check(lib.jgamd_scale_csx_weights(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w_sorted), _lib.ptr(by_idx),
                                           _lib.ptr(by_seg), V, E, n_factor, _lib.ptr(w), _lib.ptr(ws), nbytes,
                                           _lib.stream_ptr(dev)))
    return idx, off, w


def cootocsr(edge_index, edge_weight, v_num):
    """Returns CSR(column_indices, row_offset, edge_weight); rows keep the
    input order of their edges."""
    kept = _remembered(edge_index, edge_weight, v_num, 0)
    if kept is not None:
        return CSR(*kept)
    idx, off, w, _ = _convert(edge_index, edge_weight, v_num, 0)
    return CSR(idx, off, w)


def cootocsc(edge_index, edge_weight, v_num):
    """COO -> CSC (ops/cootocsc.py:29-36, ops/cpp/cootocsc_op.cc:23-53)."""
    kept = _remembered(edge_index, edge_weight, v_num, 1)
    if kept is not None:
        return CSC(*kept)
    idx, off, w, _ = _convert(edge_index, edge_weight, v_num, 1)
    return CSC(idx, off, w)
