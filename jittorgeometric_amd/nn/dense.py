"""Dense feature transform x @ W of the conv layers (gcn_conv.py:95 in the
reference).  Products of the node features with a weight matrix (forward, and
the input gradient g @ W^T) run in the library's matrix-core kernel
(csrc/dense_rows.hip), which also takes a second operand pair and a bias row
in the same pass; shapes it does not cover go to torch's BLAS.  The weight
gradient x^T @ g has a tiny [Fin,Fout] output and a reduction over every node,
for which the BLAS library picks a kernel without split-K (1.8 ms at V=1M,
Fin=Fout=128): it is computed as a batched product over slabs of nodes
followed by a sum over the slabs."""
import torch

_SLABS = 256          # partial products; V/_SLABS rows of x each
_MIN_ROWS = 1 << 16   # below this the plain product is used


def _plain(t):
    return t.dtype == torch.float32 and t.is_cuda and t.dim() == 2 and t.is_contiguous() and t.data_ptr() % 16 == 0


def padded_width(n):
    """Floats between the rows of a [V,n] result that a product over the graph gathers next.
    A gathered row costs the 128-byte lines it touches.  Dense rows of 4n bytes start at every
    multiple of gcd(4n, 128) inside a line, and for some widths a good share of them straddles
    one line more than a row that starts on a line would (47 floats = 188 bytes: three lines
    instead of two for 14 of the 32 possible starts, 2.44 on average; 40, 80 or 100 floats never
    do).  Such widths, above one line, are padded to whole lines: 47 -> 64 runs the product at
    8.3 instead of 7.0 TB/s on the 2.45M-node graph although the array grows by a third;
    everything else stays dense."""
    import math
    row = 4 * n
    if n <= 32 or row % 128 == 0:
        return n
    g = math.gcd(row, 128)
    starts = range(0, 128, g)
    dense = sum((o + row + 127) // 128 for o in starts) / len(starts)
    return (n + 31) // 32 * 32 if dense - (row + 127) // 128 >= 0.2 else n


def rows_times(x1, w1, x2=None, w2=None, bias=None, relu=False, pad_rows=False):
    """x1 @ w1 (+ x2 @ w2) (+ bias), clamped at zero with relu, in one pass over the rows: the
    library's matrix-core kernel (csrc/dense_rows.hip) for the shapes it covers, torch's BLAS
    products otherwise.  pad_rows: where the BLAS route is taken, the result may be a [V,N] view
    of rows padded_width(N) floats apart (the product is written with that leading dimension,
    no extra pass)."""
    from .. import _lib
    two = x2 is not None
    K1, N = w1.shape
    K2 = w2.shape[0] if two else 0
    ok = x1.is_cuda and _plain(x1) and w1.dtype == torch.float32 and x1.shape[1] == K1 and x1.shape[0] >= 1 << 12
    if two:
        ok = ok and _plain(x2) and w2.dtype == torch.float32 and x2.shape == (x1.shape[0], K2) and w2.shape[1] == N
    if bias is not None:
        ok = ok and bias.dtype == torch.float32 and bias.numel() == N
    if ok:
        lib = _lib.load()
        ok = bool(lib.jgamd_dense_rows_supported(K1, K2, N))
    if not ok:
        wide = padded_width(N) if pad_rows and x1.dim() == 2 and x1.is_cuda and x1.dtype == torch.float32 else N
        if wide != N and not two:
            out = torch.empty((x1.shape[0], wide), dtype=torch.float32, device=x1.device)[:, :N]
            if bias is not None:
                torch.addmm(bias, x1, w1, out=out)
            else:
                torch.mm(x1, w1, out=out)
            return out.relu_() if relu else out
        out = torch.addmm(bias, x1, w1) if bias is not None else x1 @ w1
        out = out.addmm_(x2, w2) if two else out
        return out.relu_() if relu else out
    dev = _lib.require_gpu(x1, w1, x2, w2, bias)
    w1 = w1.contiguous()
    w2 = w2.contiguous() if two else None
    bias = bias.contiguous() if bias is not None else None
    if bias is not None and bias.data_ptr() % 16:
        bias = bias.clone()
    out = torch.empty((x1.shape[0], N), dtype=torch.float32, device=dev)
    _lib.check(lib.jgamd_dense_rows(_lib.ptr(x1), _lib.ptr(w1), K1, _lib.ptr(x2), _lib.ptr(w2), K2, _lib.ptr(bias),
                                    _lib.ptr(out), x1.shape[0], N, 1 if relu else 0, _lib.stream_ptr(dev)))
    return out


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
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        return rows_times(x, weight, bias=bias)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        gx = gw = gb = None
        g = g.contiguous()
        if ctx.needs_input_grad[0]:
            gx = rows_times(g, weight.t())      # copied row-major only where the library's kernel runs
        if ctx.needs_input_grad[1]:
            gw = xt_g(x, g)
        if ctx.needs_input_grad[2]:
            gb = column_sum(g) if g.dtype == torch.float32 and g.dim() == 2 else g.sum(0)
        return gx, gw, gb


def xw(x, weight, bias=None):
    """x @ weight (+ bias) with a split weight gradient; x [V,Fin], weight [Fin,Fout]."""
    if x.dim() != 2 or not x.is_contiguous():
        out = x @ weight
        return out if bias is None else out + bias
    return _XW.apply(x, weight, bias)


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


def relu_backward_column_sum(g, y):
    """(g where y > 0 else 0, its sum over rows) for the upstream gradient g and a ReLU's output y,
    both contiguous [R,F] float32 GPU tensors, in one pass (csrc/dense_ops.hip)."""
    from .. import _lib
    lib = _lib.load()
    dev = _lib.require_gpu(g, y)
    R, F = g.shape
    masked = torch.empty_like(g)
    out = torch.empty(F, dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_column_sum_workspace, R, F)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_relu_backward_column_sum(_lib.ptr(g), _lib.ptr(y), _lib.ptr(masked), _lib.ptr(out), R, F,
                                                  _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    return masked, out


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
