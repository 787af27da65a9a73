"""Neighbour lists of a set of nodes, concatenated in the order the nodes are given (a node
listed twice contributes twice).  Same calls as jittor_geometric.ops.from_nodes / to_nodes
(ops/saparse_ops.py:9-71), whose Python loops slice one node at a time; here the library
counts and scans the lengths and one launch of the neighbour-copy kernel (csrc/sample.hip,
fanout -1) writes all lists."""
import torch

from .. import _lib
from ._common import as_i32


def _gather_lists(off, idx, nodes):
    lib = _lib.load()
    dev = _lib.require_gpu(off, idx, nodes)
    off = as_i32(off, "offsets")
    idx = as_i32(idx, "indices")
    nodes = as_i32(nodes, "nodes").reshape(-1)
    n = nodes.shape[0]
    loff = torch.empty(n + 1, dtype=torch.int32, device=dev)
    nbytes = _lib.query(lib.jgamd_layer_column_offsets_workspace, n)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_layer_column_offsets(_lib.ptr(nodes), _lib.ptr(off), n, max(off.shape[0] - 1, 0),
                                              2 ** 31 - 1, _lib.ptr(loff), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    total = int(loff[-1].item())
    if total < 0:
        raise _lib.JgamdError("from_nodes / to_nodes: more than 2^31-1 neighbours in total")
    out = torch.empty(total, dtype=torch.int32, device=dev)
    _lib.check(lib.jgamd_sample_neighbors(_lib.ptr(nodes), _lib.ptr(loff), _lib.ptr(off), _lib.ptr(idx), n,
                                          off.shape[0] - 1, -1, total, 0, _lib.ptr(out), _lib.stream_ptr(dev)))
    return out


def from_nodes(csc, nodes):
    if csc is None:
        raise ValueError("CSC structure must be provided.")
    return _gather_lists(csc.column_offset, csc.row_indices, nodes)


def to_nodes(csr, nodes):
    if csr is None:
        raise ValueError("CSR structure must be provided.")
    return _gather_lists(csr.row_offset, csr.column_indices, nodes)
