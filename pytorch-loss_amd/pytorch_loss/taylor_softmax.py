"""Taylor softmax on the HIP kernels.

Same surface as the reference's V3 classes (pytorch_loss/taylor_softmax.py:16-198):
``TaylorSoftmaxFunc.apply(feat, dim, n, use_log)``, ``taylor_softmax_v3``, the modules
``TaylorSoftmaxV3`` / ``LogTaylorSoftmaxV3`` (usage as ``nn.Softmax`` / ``nn.LogSoftmax``) and
``TaylorCrossEntropyLossV3(n, ignore_index, reduction)`` (usage as ``nn.CrossEntropyLoss``).
exp(x) is replaced by its Taylor polynomial of even order ``n``.

The reference's cross entropy is the log module followed by ``F.nll_loss``; here it is one kernel
per direction that never writes the (N, C, *) log-probabilities (same values: the loss of a pixel
is ``-log_taylor_softmax(logits)[label]``, ignored pixels give 0, 'mean' divides by the number of
non-ignored pixels).
"""
import torch
import torch.nn as nn

from . import _native


def _even_order(n):
    """What the reference asserts wherever the order is used (taylor_softmax.py:38, 50, 85)."""
    assert n % 2 == 0 and n > 0, "the order of the Taylor polynomial must be even and positive"
    return n


def _even(n):
    """What the constructors of the reference's log module and cross entropy assert (taylor_softmax.py:131, 181):
    an even order; n = 0 (or a negative even one) passes there and fails in the first forward, as it does here."""
    assert n % 2 == 0, "the order of the Taylor polynomial must be even"
    return n


class TaylorSoftmaxFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, feat, dim=1, n=2, use_log=False):
        ctx.call = (feat, dim, n, use_log)
        return _native.taylor_softmax_forward(*ctx.call)

    @staticmethod
    def backward(ctx, grad_output):
        return (_native.taylor_softmax_backward(grad_output, *ctx.call),) + (None,) * 3


def taylor_softmax_v3(inten, dim=1, n=4, use_log=False):
    return TaylorSoftmaxFunc.apply(inten, dim, _even_order(n), use_log)


class _TaylorAlongDim(nn.Module):
    use_log = False

    def __init__(self, dim=1, n=2):
        super().__init__()
        self.dim, self.n = dim, _even_order(n)

    def forward(self, x):
        return taylor_softmax_v3(x, self.dim, self.n, self.use_log)


class TaylorSoftmaxV3(_TaylorAlongDim):
    """Usage as ``nn.Softmax(dim)``."""


class LogTaylorSoftmaxV3(_TaylorAlongDim):
    """Usage as ``nn.LogSoftmax(dim)``."""
    use_log = True

    def __init__(self, dim=1, n=2):
        nn.Module.__init__(self)
        self.dim, self.n = dim, _even(n)


class TaylorCrossEntropyFunctionV3(torch.autograd.Function):
    """-log_taylor_softmax(logits)[label] per pixel, or its 'sum' / 'mean' over the non-ignored
    pixels produced inside the kernel; backward folds the upstream gradient (and the 1/n_valid of a
    mean) into the gradient kernel."""

    @staticmethod
    def forward(ctx, logits, labels, n, ignore_index, reduction):
        ctx.args = args = _native.taylor_args(logits, labels)
        sums = None
        if reduction in ("mean", "sum") and ctx.needs_input_grad[0]:
            # long rows: the forward leaves each row's sum for an elementwise backward
            loss, n_valid, sums = _native.taylor_ce_forward_reduced_sums(logits, labels, n, ignore_index,
                                                                         reduction == "mean", args=args)
        else:
            loss, n_valid = _native.taylor_ce_forward(logits, labels, n, ignore_index, reduction, args=args)
        ctx.vars = (n, ignore_index, n_valid if reduction == "mean" else None, sums)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        n, ignore_index, n_valid, sums = ctx.vars
        if sums is not None:
            grad = _native.taylor_ce_backward_scaled_sums(sums, n, ignore_index, grad_output, n_valid, ctx.args)
        else:
            grad = _native.taylor_ce_backward(None, None, n, ignore_index, grad_output, n_valid, args=ctx.args)
        return grad, None, None, None, None


class TaylorCrossEntropyLossV3(nn.Module):

    def __init__(self, n=2, ignore_index=-1, reduction='mean'):
        super().__init__()
        self.n, self.ignore_index, self.reduction = _even(n), ignore_index, reduction

    def forward(self, logits, labels):
        return TaylorCrossEntropyFunctionV3.apply(logits, labels, _even_order(self.n), self.ignore_index, self.reduction)
