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


class TaylorSoftmaxFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, feat, dim=1, n=2, use_log=False):
        ctx.vars = feat, dim, n, use_log
        return _native.taylor_softmax_forward(feat, dim, n, use_log)

    @staticmethod
    def backward(ctx, grad_output):
        feat, dim, n, use_log = ctx.vars
        return _native.taylor_softmax_backward(grad_output, feat, dim, n, use_log), None, None, None


def taylor_softmax_v3(inten, dim=1, n=4, use_log=False):
    assert n % 2 == 0 and n > 0
    return TaylorSoftmaxFunc.apply(inten, dim, n, use_log)


class TaylorSoftmaxV3(nn.Module):

    def __init__(self, dim=1, n=2):
        super().__init__()
        assert n % 2 == 0 and n > 0
        self.dim = dim
        self.n = n

    def forward(self, x):
        return taylor_softmax_v3(x, self.dim, self.n, use_log=False)


class LogTaylorSoftmaxV3(nn.Module):

    def __init__(self, dim=1, n=2):
        super().__init__()
        assert n % 2 == 0
        self.dim = dim
        self.n = n

    def forward(self, x):
        return taylor_softmax_v3(x, self.dim, self.n, use_log=True)


class TaylorCrossEntropyFunctionV3(torch.autograd.Function):
    """-log_taylor_softmax(logits)[label] per pixel, or its 'sum' / 'mean' over the non-ignored
    pixels produced inside the kernel; backward folds the upstream gradient (and the 1/n_valid of a
    mean) into the gradient kernel."""

    @staticmethod
    def forward(ctx, logits, labels, n, ignore_index, reduction):
        ctx.args = args = _native.taylor_args(logits, labels)
        loss, n_valid = _native.taylor_ce_forward(logits, labels, n, ignore_index, reduction, args=args)
        ctx.vars = (n, ignore_index, n_valid if reduction == "mean" else None)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        n, ignore_index, n_valid = ctx.vars
        grad = _native.taylor_ce_backward(None, None, n, ignore_index, grad_output, n_valid, args=ctx.args)
        return grad, None, None, None, None


class TaylorCrossEntropyLossV3(nn.Module):

    def __init__(self, n=2, ignore_index=-1, reduction='mean'):
        super().__init__()
        assert n % 2 == 0
        self.n = n
        self.reduction = reduction
        self.ignore_index = ignore_index

    def forward(self, logits, labels):
        return TaylorCrossEntropyFunctionV3.apply(logits, labels, self.n, self.ignore_index, self.reduction)
