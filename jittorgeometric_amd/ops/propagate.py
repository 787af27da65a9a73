"""Hops of the reference's polynomial propagation layers with the element-wise
tail folded into the product: one kernel per hop computes
beta * (A x) + alpha * h, where the reference runs the product and then
x * (1 - alpha) and x + alpha * h as separate passes
(nn/conv/appnp_conv.py:42-51)."""
import torch

from ._common import both_orders, spmm_axpby


class HopFunc(torch.autograd.Function):
    """out = beta * A x + alpha * h; gradients beta * A^T g and alpha * g."""

    @staticmethod
    def forward(ctx, x, h, fwd, bwd, beta, alpha):
        ctx.bwd, ctx.beta, ctx.alpha = bwd, beta, alpha
        ctx.has_h = h is not None
        return spmm_axpby(fwd[0], fwd[1], fwd[2], x, x.shape[0], beta, alpha, h)

    @staticmethod
    def backward(ctx, g):
        g = g.contiguous()
        off, idx, w = ctx.bwd
        gx = spmm_axpby(off, idx, w, g, g.shape[0], ctx.beta, 0.0, None) if ctx.needs_input_grad[0] else None
        gh = ctx.alpha * g if (ctx.has_h and ctx.needs_input_grad[1]) else None
        return gx, gh, None, None, None, None


def propagate_axpby(x, h, csc, csr, beta=1.0, alpha=0.0):
    """beta * aggregateWithWeight(x, csc, csr) + alpha * h in one pass over the graph."""
    fwd, bwd = both_orders(csc, csr)
    return HopFunc.apply(x, h, fwd, bwd, float(beta), float(alpha))


class AggregateBiasFunc(torch.autograd.Function):
    """A x + bias with the bias added in the product's row store
    (nn/conv/gcn_conv.py:102-110 adds it in a pass of its own)."""

    @staticmethod
    def forward(ctx, x, bias, fwd, bwd):
        ctx.bwd = bwd
        return spmm_axpby(fwd[0], fwd[1], fwd[2], x, x.shape[0], 1.0, 1.0, bias)

    @staticmethod
    def backward(ctx, g):
        from ..nn.dense import column_sum
        g = g.contiguous()
        off, idx, w = ctx.bwd
        gx = spmm_axpby(off, idx, w, g, g.shape[0], 1.0, 0.0, None) if ctx.needs_input_grad[0] else None
        gb = column_sum(g) if ctx.needs_input_grad[1] else None
        return gx, gb, None, None


def aggregate_bias(x, bias, csc, csr):
    """aggregateWithWeight(x, csc, csr) + bias in one pass; either of csc / csr may be None."""
    fwd, bwd = both_orders(csc, csr)
    return AggregateBiasFunc.apply(x.contiguous(), bias, fwd, bwd)


class AppnpFunc(torch.autograd.Function):
    """K hops x <- (1 - alpha) A x + alpha h with x_0 = h.  With M = (1 - alpha) A^T the
    gradient is M^K g + alpha * (M^(K-1) + ... + M + I) g, evaluated by the same hop:
    v <- M v + alpha g, K times from v = g."""

    @staticmethod
    def forward(ctx, h, fwd, bwd, K, alpha):
        ctx.bwd, ctx.K, ctx.alpha = bwd, K, alpha
        x = h
        for _ in range(K):
            x = spmm_axpby(fwd[0], fwd[1], fwd[2], x, x.shape[0], 1.0 - alpha, alpha, h)
        return x if K > 0 else h.clone()

    @staticmethod
    def backward(ctx, g):
        g = g.contiguous()
        off, idx, w = ctx.bwd
        v = g
        for _ in range(ctx.K):
            v = spmm_axpby(off, idx, w, v, v.shape[0], 1.0 - ctx.alpha, ctx.alpha, g)
        return v, None, None, None, None


def appnp_propagate(x, csc, csr, K, alpha):
    fwd, bwd = both_orders(csc, csr)
    return AppnpFunc.apply(x.contiguous(), fwd, bwd, int(K), float(alpha))
