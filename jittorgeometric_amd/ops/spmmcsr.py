"""SpMM on a CSR matrix.  Same call as jittor_geometric.ops.SpmmCsr
(ops/spmmcsr.py:21-44), whose arithmetic is cuSPARSE inside the jittor wheel.
trans_A=True (the default) multiplies by the transpose of the CSR matrix:
out[c] = sum over entries (r, c) of w * x[r]."""
import torch

from .. import _lib
from ._common import csr_arrays, spmm, transposed

# False: backward is the exact transpose of forward (the true gradient).
# True: backward re-applies the forward product, as the reference does
# (ops/spmmcsr.py:35-39); the two agree whenever the matrix is symmetric,
# e.g. for gcn_norm weights on an undirected graph.
REFERENCE_GRAD = False


def _product(x, csr, trans_A):
    off, col, w = csr_arrays(csr)
    v_num = off.shape[0] - 1
    if trans_A:
        # the transposed product is run as a gather over the transposed arrays,
        # built once per CSR object (stable, so the result is reproducible)
        off_t, idx_t, w_t, _ = transposed(csr, off, col, w, v_num, v_num)
        return spmm(off_t, idx_t, w_t, x, v_num)
    return spmm(off, col, w, x, v_num)


class SpmmCsrFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, csr, trans_A):
        ctx.csr = csr
        ctx.trans_A = trans_A
        return _product(x, csr, trans_A)

    @staticmethod
    def backward(ctx, grad_output):
        trans = ctx.trans_A if REFERENCE_GRAD else not ctx.trans_A
        return _product(grad_output, ctx.csr, trans), None, None


def SpmmCsr(x, csr, trans_A=True, trans_B=False):
    """op(A) x, or op(A) x^T with trans_B=True (x is then [F, V], the dense operand stored
    transposed, as the flag tells cuSPARSE: ops/spmmcsr.py:31 hands it on unread).  No caller
    in the reference sets trans_B and its output allocation (v_num rows, size(x, 1) columns,
    ops/spmmcsr.py:24-28) only fits a square x; what cuSPARSE does with the flag is the
    documented op(B) = B^T, "parity unpinned" like the rest of that third-party product."""
    if trans_B:
        if x.dim() != 2:
            raise _lib.JgamdError("SpmmCsr: x must be two-dimensional, got %s" % (tuple(x.shape),))
        x = x.t().contiguous()          # differentiable: the gradient comes back transposed
    return SpmmCsrFunc.apply(x, csr, trans_A)
