"""Dense feature transform x @ W of the conv layers (gcn_conv.py:95 in the
reference).  The products run in torch's hipBLASLt (MFMA); only the weight
gradient is arranged differently: x^T @ g has a tiny [Fin,Fout] output and a
reduction over every node, for which the library picks a kernel without
split-K (1.8 ms at V=1M, Fin=Fout=128).  It is computed here as a batched
product over slabs of nodes followed by a sum over the slabs."""
import torch

_SLABS = 256          # partial products; V/_SLABS rows of x each
_MIN_ROWS = 1 << 16   # below this the plain product is used


def xt_g(x, g):
    """x^T @ g for x [V,Fin], g [V,Fout]: partial products over slabs of nodes, then their sum."""
    V = x.shape[0]
    rows = V // _SLABS
    if V < _MIN_ROWS or rows == 0 or not (x.is_contiguous() and g.is_contiguous()):
        return x.t() @ g
    main = rows * _SLABS
    xs = x[:main].view(_SLABS, rows, x.shape[1])
    gs = g[:main].view(_SLABS, rows, g.shape[1])
    gw = torch.bmm(xs.transpose(1, 2), gs).sum(0)
    if main < V:
        gw = gw + x[main:].t() @ g[main:]
    return gw


class _XW(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        return x @ weight

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        gx = gw = None
        if ctx.needs_input_grad[0]:
            gx = g @ weight.t()
        if ctx.needs_input_grad[1]:
            gw = xt_g(x, g)
        return gx, gw


def xw(x, weight):
    """x @ weight with a split weight gradient; x [V,Fin], weight [Fin,Fout]."""
    if x.dim() != 2 or not x.is_contiguous():
        return x @ weight
    return _XW.apply(x, weight)


def column_sum(x):
    """sum over rows of a contiguous [R,F] float32 GPU tensor (csrc/dense_ops.hip)."""
    from .. import _lib
    lib = _lib.load()
    dev = _lib.require_gpu(x)
    R, F = x.shape
    out = torch.empty(F, dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_column_sum_workspace, R, F)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_column_sum(_lib.ptr(x), _lib.ptr(out), R, F, _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    return out


class _AddBias(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bias):
        return x + bias

    @staticmethod
    def backward(ctx, g):
        gb = None
        if ctx.needs_input_grad[1]:
            if g.dim() == 2 and g.dtype == torch.float32:
                gb = column_sum(g.contiguous())
            else:
                gb = g.sum(0)
        return g, gb


def add_bias(x, bias):
    """x + bias (broadcast over rows) whose bias gradient is the library's column sum."""
    return _AddBias.apply(x, bias)
