"""Fused GAT core: logits, edge softmax and weighted aggregation in one
kernel pass (csrc/gat.hip).  No single counterpart in the reference: it
replaces the chain ScatterToEdge x2 -> concat -> matmul -> leaky_relu ->
EdgeSoftmax -> multiply -> ScatterToVertex of GATConv.propagate
(nn/conv/gat_conv.py:61-83) and the gradient chain Jittor derives from it."""
import torch

from .. import _lib
from ._common import PLAN_GAT, as_f32, csc_arrays, csx_plan, transposed


def fused_supported(H, D, backward=True):
    """Shapes the fused kernels take; others go through the operator chain."""
    F = H * D
    vec = 4 if D % 4 == 0 else 2 if D % 2 == 0 else 1
    while vec > 1 and F <= 64 * (vec // 2):
        vec //= 2
    if F > 2048 or -(-F // (64 * vec)) > 8:
        return False
    if backward and H > 1:
        lph = D // vec
        return 1 <= lph <= 64 and (lph & (lph - 1)) == 0
    return True


def gat_forward_raw(h, csc, a_src, a_dst, slope=0.2, want_alpha=False, for_backward=False, want_scores=None):
    """h [V,H,D], a_src/a_dst [H,D] -> dict(out, el, er, smax, ssum, alpha, pos, spos); pos / spos
    (the positive-logit share of out and of the attention, which the backward kernels read) are
    only computed with for_backward, and el / er only when something reads them (want_scores;
    by default with want_alpha or for_backward): without them the kernel takes the scores itself."""
    lib = _lib.load()
    dev = _lib.require_gpu(h, csc.row_indices, csc.column_offset, a_src, a_dst)
    h, a_src, a_dst = as_f32(h, "h"), as_f32(a_src, "a_src"), as_f32(a_dst, "a_dst")
    off, idx, _ = csc_arrays(csc)
    if h.dim() != 3 or tuple(a_src.shape) != tuple(h.shape[1:]) or tuple(a_dst.shape) != tuple(h.shape[1:]):
        raise _lib.JgamdError("gat: h must be [V,H,D] and a_src/a_dst [H,D], got %s, %s, %s"
                              % (tuple(h.shape), tuple(a_src.shape), tuple(a_dst.shape)))
    V, H, D = h.shape
    if off.shape[0] != V + 1:
        raise _lib.JgamdError("gat: %d column offsets for %d nodes" % (off.shape[0], V))
    E = idx.shape[0]
    mk = lambda *s: torch.empty(s, dtype=torch.float32, device=dev)
    if want_scores is None:
        want_scores = want_alpha or for_backward
    if (want_alpha or for_backward) and not want_scores:
        raise _lib.JgamdError("gat: alpha and the backward arrays need el / er")
    out, smax, ssum = mk(V, H, D), mk(V, H), mk(V, H)
    el, er = (mk(V, H), mk(V, H)) if want_scores else (None, None)
    alpha = mk(E, H) if want_alpha else None
    pos, spos = (mk(V, H, D), mk(V, H)) if for_backward else (None, None)
    nbytes = _lib.query(lib.jgamd_gat_fwd_workspace, V, E, H, D)
    ws = _lib.workspace(nbytes, dev)
    plan, n_fix, n_grp = csx_plan(off, V, E, PLAN_GAT) if V > 0 else (None, -1, -1)
    _lib.check(lib.jgamd_gat_fwd(_lib.ptr(plan), n_fix, n_grp, _lib.ptr(off), _lib.ptr(idx), _lib.ptr(h),
                                 _lib.ptr(a_src), _lib.ptr(a_dst), float(slope), _lib.ptr(el), _lib.ptr(er),
                                 _lib.ptr(smax), _lib.ptr(ssum), _lib.ptr(pos), _lib.ptr(spos), _lib.ptr(alpha),
                                 _lib.ptr(out), V, E, H, D, _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    return dict(out=out, el=el, er=er, smax=smax, ssum=ssum, alpha=alpha, pos=pos, spos=spos)


class GatFusedFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h, a_src, a_dst, csc, slope):
        # what backward reads must be what forward read: dense fp32 copies, not the caller's views
        h, a_src, a_dst = as_f32(h, "h"), as_f32(a_src, "a_src"), as_f32(a_dst, "a_dst")
        needs_grad = any(ctx.needs_input_grad[:3])
        r = gat_forward_raw(h, csc, a_src, a_dst, slope, for_backward=needs_grad)
        if needs_grad:
            ctx.save_for_backward(h, a_src, a_dst, r["el"], r["er"], r["smax"], r["ssum"], r["out"], r["pos"],
                                  r["spos"])
        ctx.csc = csc
        ctx.slope = slope
        return r["out"]

    @staticmethod
    def backward(ctx, g_out):
        lib = _lib.load()
        h, a_src, a_dst, el, er, smax, ssum, out, pos, spos = ctx.saved_tensors
        csc = ctx.csc
        g_out = as_f32(g_out, "g_out")
        dev = _lib.require_gpu(g_out, h)
        V, H, D = h.shape
        off, idx, w = csc_arrays(csc)
        E = idx.shape[0]
        off_t, idx_t, _, _ = transposed(csc, off, idx, w, V, V)
        g_h = torch.empty((V, H, D), dtype=torch.float32, device=dev)
        g_as = torch.empty((H, D), dtype=torch.float32, device=dev)
        g_ad = torch.empty((H, D), dtype=torch.float32, device=dev)
        nbytes = _lib.query(lib.jgamd_gat_bwd_workspace, V, E, H, D)
        ws = _lib.workspace(nbytes, dev)
        plan, n_fix, n_grp = csx_plan(off_t, V, E, PLAN_GAT) if V > 0 else (None, -1, -1)
        _lib.check(lib.jgamd_gat_bwd(_lib.ptr(plan), n_fix, n_grp, _lib.ptr(off_t), _lib.ptr(idx_t), _lib.ptr(h),
                                     _lib.ptr(a_src), _lib.ptr(a_dst), float(ctx.slope), _lib.ptr(el), _lib.ptr(er),
                                     _lib.ptr(smax), _lib.ptr(ssum), _lib.ptr(spos), _lib.ptr(out), _lib.ptr(pos),
                                     _lib.ptr(g_out), _lib.ptr(g_h), _lib.ptr(g_as), _lib.ptr(g_ad), V, E, H, D,
                                     _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
        return g_h, g_as, g_ad, None, None


def gat_aggregate(h, csc, a_src, a_dst, slope=0.2):
    """out[v,k,:] = sum over in-edges e of v of softmax_e(leaky_relu(a_src[k].h[src(e),k] +
    a_dst[k].h[v,k])) * h[src(e),k,:]; differentiable in h, a_src, a_dst."""
    return GatFusedFunc.apply(h, a_src, a_dst, csc, slope)
