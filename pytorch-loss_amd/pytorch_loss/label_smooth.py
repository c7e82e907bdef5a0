"""Label-smoothed softmax cross entropy on the HIP kernels.

Same surface as the reference's V3 pair (pytorch_loss/label_smooth.py:126-171):
``LSRCrossEntropyFunctionV3.apply(logits, labels, lb_smooth, lb_ignore)`` returns the
per-pixel losses, ``LabelSmoothSoftmaxCEV3(lb_smooth, reduction, ignore_index)`` reduces
them.  Target weight is ``1 - lb_smooth``, every other class gets ``lb_smooth / C``.
"""
import torch
import torch.nn as nn

from . import _native


class LSRCrossEntropyFunctionV3(torch.autograd.Function):
    """forward -> losses of shape ``labels.shape`` (0 at ignored pixels);
    backward -> d/dlogits, with the upstream gradient folded into the same kernel."""

    @staticmethod
    def forward(ctx, logits, labels, lb_smooth, lb_ignore):
        ctx.variables = (logits, labels, lb_ignore, lb_smooth)
        ctx.args = args = _native.lsr_args(logits, labels)
        return _native.lsr_forward(logits, labels, lb_ignore, lb_smooth, args=args)

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, lb_ignore, lb_smooth = ctx.variables
        grad = _native.lsr_backward(logits, labels, lb_ignore, lb_smooth, grad_output, args=ctx.args)
        return grad, None, None, None


class _LSRReducedFunction(torch.autograd.Function):
    """'sum' / 'mean' of the per-pixel losses produced inside the forward kernel (per-block
    partials, then a fixed-order finishing kernel), so the module needs no ATen pass over the
    pixels for `losses.sum()` and `(labels != ignore).sum()`; backward folds the scalar
    upstream gradient and the 1/n_valid of a mean into the gradient kernel. On fp32 logits whose channel
    planes have an odd length (513 x 513, 769 x 769 crops) the forward also keeps every pixel's log-sum-exp
    (4 bytes per pixel, only when a gradient will be asked for) and the backward forms the gradient from it
    plane by plane instead of recomputing the softmax (see plh_lsr_backward_scaled_lse)."""

    @staticmethod
    def forward(ctx, logits, labels, lb_smooth, lb_ignore, mean):
        ctx.args = args = _native.lsr_args(logits, labels)
        lse = None
        if ctx.needs_input_grad[0]:
            loss, n_valid, lse = _native.lsr_forward_reduced_lse(logits, labels, lb_ignore, lb_smooth, mean, args=args)
        else:
            loss, n_valid = _native.lsr_forward_reduced(logits, labels, lb_ignore, lb_smooth, mean, args=args)
        ctx.variables = (logits, labels, lb_ignore, lb_smooth, n_valid if mean else None, lse)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, lb_ignore, lb_smooth, n_valid, lse = ctx.variables
        if lse is not None:
            grad = _native.lsr_backward_scaled_lse(lse, lb_ignore, lb_smooth, grad_output, n_valid, ctx.args)
        else:
            grad = _native.lsr_backward_scaled(logits, labels, lb_ignore, lb_smooth, grad_output, n_valid, args=ctx.args)
        return grad, None, None, None, None


class _LSRFusedReducedFunction(torch.autograd.Function):
    """fb=True with 'sum' / 'mean': loss and gradient from ONE pass over the logits, as the large-margin module's
    fb=True (large_margin_softmax._LargeMarginFusedReducedFunction). The kept gradient is the one under an upstream
    gradient of 1, already divided by the number of valid pixels for 'mean'; backward multiplies it in place by the
    upstream scalar, a pass over it only when that scalar is not 1."""

    @staticmethod
    def forward(ctx, logits, labels, lb_smooth, lb_ignore, mean):
        loss, grads, tag = _native.lsr_forward_backward_reduced(logits, labels, lb_ignore, lb_smooth, mean)
        ctx.variables = (grads, tag)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        grads, tag = _native.take_kept(ctx)
        return _native.scale_unless_one(grads, tag, grad_output), None, None, None, None


class LabelSmoothSoftmaxCEV3(nn.Module):
    """Usage as nn.CrossEntropyLoss: logits (N, C, *) float, labels (N, *) int64.

    reduction: 'mean' divides the summed loss by the number of non-ignored pixels,
    'sum' sums, anything else returns the per-pixel tensor.

    fb (not in the reference, whose LSR module has no forward+backward Function; the keyword of its
    LargeMarginSoftmaxV3): True computes the gradient in the forward pass of a 'mean' / 'sum' loss and keeps it for
    backward - one pass over the logits per step instead of two, as long as the loss reaches backward() with an
    upstream gradient of 1; a weighted or scaled loss costs a further pass over the kept gradient. fp16 logits and
    reduction 'none' are not affected.
    """

    def __init__(self, lb_smooth=0.1, reduction="mean", ignore_index=-100, fb=False):
        super().__init__()
        self.lb_smooth = lb_smooth
        self.reduction = reduction
        self.lb_ignore = ignore_index
        self.fb = fb

    def forward(self, logits, labels):
        if (self.fb and self.reduction in ("sum", "mean") and logits.numel() > 0 and logits.dtype != torch.float16
                and logits.requires_grad and torch.is_grad_enabled()):
            return _LSRFusedReducedFunction.apply(logits, labels, self.lb_smooth, self.lb_ignore,
                                                  self.reduction == "mean")
        if self.reduction in ("sum", "mean") and logits.numel() > 0:
            return _LSRReducedFunction.apply(logits, labels, self.lb_smooth, self.lb_ignore,
                                             self.reduction == "mean")
        losses = LSRCrossEntropyFunctionV3.apply(logits, labels, self.lb_smooth, self.lb_ignore)
        if self.reduction == "sum":
            return losses.sum()
        if self.reduction == "mean":
            n_valid = (labels != self.lb_ignore).sum()
            return losses.sum() / n_valid
        return losses
