"""Mean cross-entropy over the rows of a logits matrix: the loss of the reference's
training steps (nn.cross_entropy_loss(pred, label) in examples/gcn_example.py:113,
nn.log_softmax + nn.nll_loss in examples/sage_example.py:69,83; both functions live in
the jittor package).  Forward and gradient are one library kernel each
(csrc/loss.hip): with millions of rows and a few dozen classes a generic framework
loss spends most of its time in single-block reductions."""
import torch

from .. import _lib


class _CrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, output, target, log_probs):
        lib = _lib.load()
        dev = _lib.require_gpu(output, target)
        if output.dim() != 2:
            raise _lib.JgamdError("cross_entropy_loss: output must be [rows, classes], got %s" % (tuple(output.shape),))
        if target.dim() != 1 or target.shape[0] != output.shape[0]:
            raise _lib.JgamdError("cross_entropy_loss: %d labels for %d rows" % (target.numel(), output.shape[0]))
        if target.dtype not in (torch.int32, torch.int64):
            target = target.to(torch.int64)
        x = output if output.dtype == torch.float32 else output.to(torch.float32)
        x = x.contiguous()
        target = target.contiguous()
        V, C = x.shape
        loss = torch.empty((), dtype=torch.float32, device=dev)
        count = torch.empty((), dtype=torch.int32, device=dev)
        lse = torch.empty(V, dtype=torch.float32, device=dev)
        nbytes = _lib.query(lib.jgamd_cross_entropy_workspace, V, C)
        ws = _lib.workspace(nbytes, dev)
        i64 = 1 if target.dtype == torch.int64 else 0
        _lib.check(lib.jgamd_cross_entropy_fwd(_lib.ptr(x), _lib.ptr(target), i64, int(bool(log_probs)), V, C,
                                               _lib.ptr(loss), _lib.ptr(count),
                                               _lib.ptr(lse), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
        ctx.save_for_backward(x, target, lse, count)
        ctx.i64 = i64
        ctx.in_dtype = output.dtype
        return loss

    @staticmethod
    def backward(ctx, g):
        if not ctx.needs_input_grad[0]:
            return None, None, None
        x, target, lse, count = ctx.saved_tensors
        lib = _lib.load()
        dev = x.device
        g = g.to(torch.float32).contiguous()
        grad = torch.empty_like(x)
        V, C = x.shape
        _lib.check(lib.jgamd_cross_entropy_bwd(_lib.ptr(x), _lib.ptr(target), ctx.i64, _lib.ptr(lse), _lib.ptr(count),
                                               _lib.ptr(g), V, C, _lib.ptr(grad), _lib.stream_ptr(dev)))
        return (grad if ctx.in_dtype == torch.float32 else grad.to(ctx.in_dtype)), None, None


def cross_entropy_loss(output, target):
    """mean_i (logsumexp(output[i,:]) - output[i, target[i]]) over the rows whose label lies in
    [0, classes); the other rows are left out and get a zero gradient."""
    return _CrossEntropy.apply(output, target, False)


def nll_loss(log_probs, target):
    """mean_i -log_probs[i, target[i]] for rows of log-probabilities (the second half of
    log_softmax + nll_loss, examples/sage_example.py:69,83); the gradient is -1 / rows at the
    labels and zero elsewhere.  Same kernels, with the softmax term switched off."""
    return _CrossEntropy.apply(log_probs, target, True)
