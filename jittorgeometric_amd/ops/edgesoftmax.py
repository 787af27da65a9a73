"""Softmax over the in-edges of every destination.  Same call as
jittor_geometric.ops.EdgeSoftmax (ops/edgesoftmax.py:62-80); the loops of
ops/cpp/edgesoftmax_op.cc:36-66 and edgesoftmaxbackward_op.cc:27-54 run as
csrc/edge_ops.hip.  x is [E] or [E,1] as in the reference, or [E,H] for H
independent heads."""
import torch

from .. import _lib
from ._common import PLAN_TILES, as_f32, csc_arrays, csx_plan


def _heads(x):
    return 1 if x.dim() == 1 else int(x.shape[1])


class EdgeSoftmaxFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csc):
        lib = _lib.load()
        dev = _lib.require_gpu(x, csc.column_offset)
        x = as_f32(x, "x")
        off = csc_arrays(csc)[0]
        V, E, H = off.shape[0] - 1, x.shape[0], _heads(x)
        if x.dim() > 2:
            raise _lib.JgamdError("EdgeSoftmax: x must be [E] or [E,H], got %s" % (tuple(x.shape),))
        y = torch.empty(x.shape, dtype=torch.float32, device=dev)
        nbytes = _lib.query(lib.jgamd_edge_softmax_workspace, V, E)
        ws = _lib.workspace(nbytes, dev)
        tiles = csx_plan(off, V, E, PLAN_TILES)[0] if H in (1, 2, 4, 8) and V > 0 and E > 0 else None
        if tiles is not None:
            _lib.check(lib.jgamd_edge_softmax_fwd_planned(_lib.ptr(tiles), _lib.ptr(off), _lib.ptr(x), _lib.ptr(y), V, E,
                                                          H, _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
        else:
            _lib.check(lib.jgamd_edge_softmax_fwd(_lib.ptr(off), _lib.ptr(x), _lib.ptr(y), V, E, H, _lib.ptr(ws),
                                                  nbytes, _lib.stream_ptr(dev)))
        ctx.save_for_backward(y)
        ctx.csc = csc
        return y

    @staticmethod
    def backward(ctx, grad_output):
        lib = _lib.load()
        (y,) = ctx.saved_tensors
        off = csc_arrays(ctx.csc)[0]
        g = as_f32(grad_output, "grad")
        dev = _lib.require_gpu(g, y)
        V, E, H = off.shape[0] - 1, y.shape[0], _heads(y)
        dx = torch.empty(y.shape, dtype=torch.float32, device=dev)
        nbytes = _lib.query(lib.jgamd_edge_softmax_workspace, V, E)
        ws = _lib.workspace(nbytes, dev)
        tiles = csx_plan(off, V, E, PLAN_TILES)[0] if H in (1, 2, 4, 8) and V > 0 and E > 0 else None
        if tiles is not None:
            _lib.check(lib.jgamd_edge_softmax_bwd_planned(_lib.ptr(tiles), _lib.ptr(off), _lib.ptr(y), _lib.ptr(g),
                                                          _lib.ptr(dx), V, E, H, _lib.ptr(ws), nbytes,
                                                          _lib.stream_ptr(dev)))
        else:
            _lib.check(lib.jgamd_edge_softmax_bwd(_lib.ptr(off), _lib.ptr(y), _lib.ptr(g), _lib.ptr(dx), V, E, H,
                                                  _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
        return dx, None


def EdgeSoftmax(x, csc):
    return EdgeSoftmaxFunc.apply(x, csc)
