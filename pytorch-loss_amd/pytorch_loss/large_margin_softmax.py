"""Large-margin softmax cross entropy (Kobayashi, BMVC 2019) on the HIP kernels.

Same surface as the reference's V3 classes (pytorch_loss/large_margin_softmax.py:149-201
and the repository root copy large_margin_softmax.py:146-229, which adds the fused
``LargeMarginSoftmaxFuncV3FB`` and the module's ``fb`` switch).
"""
import torch
import torch.nn as nn

from . import _native


class LargeMarginSoftmaxFuncV3(torch.autograd.Function):
    """forward -> per-pixel losses; backward recomputes from the inputs."""

    @staticmethod
    def forward(ctx, logits, labels, lam=0.3, ignore_index=255):
        ctx.variables = (logits, labels, lam, ignore_index)
        ctx.args = args = _native.lmargin_args(logits, labels)
        return _native.lmargin_forward(logits, labels, lam, ignore_index, args=args)

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, lam, ignore_index = ctx.variables
        grads = _native.lmargin_backward(logits, labels, lam, ignore_index, grad_output, args=ctx.args)
        return grads, None, None, None


class LargeMarginSoftmaxFuncV3FB(torch.autograd.Function):
    """forward -> (per-pixel losses, valid_cnt int64[1]); the gradient is produced by the same
    kernel and kept for backward."""

    @staticmethod
    def forward(ctx, logits, labels, lam=0.3, ignore_index=255):
        losses, grads, valid_cnt = _native.lmargin_forward_backward(logits, labels, lam, ignore_index)
        ctx.variables = grads
        ctx.mark_non_differentiable(valid_cnt)
        return losses, valid_cnt

    @staticmethod
    def backward(ctx, grad_output, grad_cnt):
        grads = _native.take_kept(ctx)
        grads.mul_(grad_output.unsqueeze(1))
        return grads, None, None, None


class _LargeMarginReducedFunction(torch.autograd.Function):
    """'sum' / 'mean' produced inside the forward kernel; see label_smooth._LSRReducedFunction."""

    @staticmethod
    def forward(ctx, logits, labels, lam, ignore_index, mean):
        ctx.args = args = _native.lmargin_args(logits, labels)
        stats = None
        if ctx.needs_input_grad[0]:
            # long rows: the forward also keeps eight floats per row, and the backward works elementwise from them
            loss, n_valid, stats = _native.lmargin_forward_reduced_stats(logits, labels, lam, ignore_index, mean, args=args)
        else:
            loss, n_valid = _native.lmargin_forward_reduced(logits, labels, lam, ignore_index, mean, args=args)
        ctx.variables = (logits, labels, lam, ignore_index, n_valid if mean else None, stats)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, lam, ignore_index, n_valid, stats = ctx.variables
        if stats is not None:
            grads = _native.lmargin_backward_scaled_stats(stats, lam, ignore_index, grad_output, n_valid, ctx.args)
        else:
            grads = _native.lmargin_backward_scaled(logits, labels, lam, ignore_index, grad_output, n_valid, args=ctx.args)
        return grads, None, None, None, None


class _LargeMarginFusedReducedFunction(torch.autograd.Function):
    """fb=True with 'sum' / 'mean': loss and gradient from ONE pass over the logits. The kept gradient is the one under
    an upstream gradient of 1 (what loss.backward() sends), already divided by the number of valid pixels for 'mean';
    backward multiplies it in place by the upstream scalar, which costs a pass over it only when that scalar is not 1
    (a weighted or scaled loss) - the reference's FB Function multiplies by a per-pixel tensor every time
    (large_margin_softmax.py:189 of the repository root)."""

    @staticmethod
    def forward(ctx, logits, labels, lam, ignore_index, mean):
        loss, grads, tag = _native.lmargin_forward_backward_reduced(logits, labels, lam, ignore_index, mean)
        ctx.variables = (grads, tag)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        grads, tag = _native.take_kept(ctx)
        return _native.scale_unless_one(grads, tag, grad_output), None, None, None, None


class LargeMarginSoftmaxV3(nn.Module):
    """Usage as nn.CrossEntropyLoss: logits (N, C, *) float, labels (N, *) int64.

    fb=True selects the fused forward+backward (one kernel, keeps a gradient-sized tensor between
    forward and backward): with 'mean' / 'sum' the reduction and the division are part of that one
    pass, so a step reads the logits once and writes the gradient once; with 'none' it is the
    reference's FB Function, whose backward multiplies the kept gradient by the per-pixel upstream
    tensor. The default recomputes in backward and keeps nothing but the inputs.
    """

    def __init__(self, lam=0.3, reduction="mean", ignore_index=255, fb=False):
        super().__init__()
        self.reduction = reduction
        self.ignore_index = ignore_index
        self.lam = lam
        self.fb = fb

    def forward(self, logits, labels):
        # fp16 logits keep the two passes: a gradient kept in fp16 at 1/n_valid of its size is subnormal before a loss
        # scale could lift it, where the backward kernel multiplies in fp32 and rounds once
        # (and a forward that no backward will follow computes no gradient)
        fused = self.fb and logits.dtype != torch.float16 and logits.requires_grad and torch.is_grad_enabled()
        if self.reduction in ("sum", "mean") and logits.numel() > 0:
            func = _LargeMarginFusedReducedFunction if fused else _LargeMarginReducedFunction
            return func.apply(logits, labels, self.lam, self.ignore_index, self.reduction == "mean")
        valid_cnt = None
        if self.fb:
            losses, valid_cnt = LargeMarginSoftmaxFuncV3FB.apply(logits, labels, self.lam, self.ignore_index)
        else:
            losses = LargeMarginSoftmaxFuncV3.apply(logits, labels, self.lam, self.ignore_index)
        if self.reduction == "mean":
            n_valid = valid_cnt if valid_cnt is not None else (labels != self.ignore_index).sum()
            return losses.sum() / n_valid
        if self.reduction == "sum":
            return losses.sum()
        return losses
