"""Vertex -> edge copy over the CSC arrays.  Same call as
jittor_geometric.ops.ScatterToEdge (ops/scatterToEdge.py:22-51):
flow "src" gives out[e] = x[row_indices[e]], anything else out[e] = x[dst(e)].
The gradient is the matching edge -> vertex sum (ops/scatterToEdge.py:42-46),
run as a gather (csrc/spmm.hip) so that it is reproducible."""
import torch

from .. import _lib
from ._common import as_f32, csc_arrays, spmm, transposed


def edge_to_vertex(x, csc, flag, v_num):
    """ops/cpp/edgetovertex_op.cc:36-55.  flag 1: out[v] = sum of x[e] over the
    column of v.  flag 0: out[u] = sum of x[e] over the edges whose source is u
    (through the transposed offsets and the slot permutation)."""
    off, idx, w = csc_arrays(csc)
    if flag == 1:
        return spmm(off, None, None, x, v_num)
    V = off.shape[0] - 1
    off_t, _, _, perm = transposed(csc, off, idx, w, V, V)
    return spmm(off_t, perm, None, x, v_num)


def scatter_to_edge(x, csc, flag):
    lib = _lib.load()
    dev = _lib.require_gpu(x, csc.row_indices, csc.column_offset)
    x = as_f32(x, "x")
    off, idx, _ = csc_arrays(csc)
    if x.dim() != 2:
        raise _lib.JgamdError("ScatterToEdge: x must be [V, F], got %s" % (tuple(x.shape),))
    V, F = x.shape
    E = idx.shape[0]
    out = torch.empty((E, F), dtype=torch.float32, device=dev)
    _lib.check(lib.jgamd_scatter_to_edge(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(x),
                                         _lib.ptr(out), off.shape[0] - 1, E, F, flag,
                                         _lib.stream_ptr(dev)))
    return out


class ScatterToEdgeFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csc, flow):
        ctx.csc = csc
        ctx.flag = 0 if flow == "src" else 1
        ctx.v_num = x.shape[0]
        return scatter_to_edge(x, csc, ctx.flag)

    @staticmethod
    def backward(ctx, grad_output):
        return edge_to_vertex(grad_output, ctx.csc, ctx.flag, ctx.v_num), None, None


def ScatterToEdge(x, csc, flow):
    return ScatterToEdgeFunc.apply(x, csc, flow)
