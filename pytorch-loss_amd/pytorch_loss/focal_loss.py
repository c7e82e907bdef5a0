"""Sigmoid focal loss on the HIP kernels.

Same surface as the reference's V3 classes (focal_loss.py:129-200 of the repository
root copy; pytorch_loss/focal_loss.py:129-178 for the packaged one):
``FocalSigmoidLossFuncV3.apply(logits, labels, alpha, gamma)`` (separate forward and
backward kernels), ``FocalSigmoidLossFuncV3FB`` (one fused kernel that also stores the
gradient) and the module ``FocalLossV3(alpha, gamma, reduction)``.  Labels are float
tensors with the logits' shape; soft labels are allowed.
"""
import torch
import torch.nn as nn

from . import _native


class FocalSigmoidLossFuncV3(torch.autograd.Function):
    """Recomputes everything from (logits, labels) in backward: nothing but the inputs is kept."""

    @staticmethod
    def forward(ctx, logits, labels, alpha, gamma):
        ctx.variables = (logits, labels, alpha, gamma)
        ctx.args = args = _native.focal_args(logits, labels)
        return _native.focal_forward(logits, labels, gamma, alpha, args=args)

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, alpha, gamma = ctx.variables
        grads = _native.focal_backward(logits, labels, gamma, alpha, grad_output, args=ctx.args)
        return grads, None, None, None


class FocalSigmoidLossFuncV3FB(torch.autograd.Function):
    """Forward computes loss and gradient in one pass and keeps the gradient for backward."""

    @staticmethod
    def forward(ctx, logits, labels, alpha, gamma):
        loss, grads = _native.focal_forward_backward(logits, labels, gamma, alpha)
        ctx.variables = grads
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        grads = _native.take_kept(ctx)
        grads.mul_(grad_output)
        return grads, None, None, None


class _FocalReducedFunction(torch.autograd.Function):
    """'sum' / 'mean' over all elements produced inside the forward kernel (per-block partials,
    fixed-order finish); backward folds the scalar upstream gradient and 1/numel into its kernel."""

    @staticmethod
    def forward(ctx, logits, labels, alpha, gamma, mean):
        ctx.variables = (logits, labels, alpha, gamma, mean)
        ctx.args = args = _native.focal_args(logits, labels)
        return _native.focal_forward_reduced(logits, labels, gamma, alpha, mean, args=args)

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, alpha, gamma, mean = ctx.variables
        scale = 1.0 / logits.numel() if mean else 1.0
        grads = _native.focal_backward_scaled(logits, labels, gamma, alpha, grad_output, scale, args=ctx.args)
        return grads, None, None, None, None


class _FocalFusedReducedFunction(torch.autograd.Function):
    """fb=True with 'sum' / 'mean': loss and gradient from ONE pass over logits and labels (12 bytes per fp32 element
    instead of the 20 of a forward and a backward). The kept gradient is the one under an upstream gradient of 1 (what
    loss.backward() sends), already divided by the element count for 'mean'; backward multiplies it in place by the
    upstream scalar, which costs a pass over it only when that scalar is not 1 - the reference's FB Function
    multiplies every time (focal_loss.py:170 of the repository root)."""

    @staticmethod
    def forward(ctx, logits, labels, alpha, gamma, mean):
        loss, grads, tag = _native.focal_forward_backward_reduced(logits, labels, gamma, alpha, mean)
        ctx.variables = (grads, tag)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        grads, tag = _native.take_kept(ctx)
        return _native.scale_unless_one(grads, tag, grad_output), None, None, None, None


class FocalLossV3(nn.Module):
    """Usage as nn.BCEWithLogitsLoss. reduction 'mean' averages over every element.

    fb=True computes the gradient in the forward pass, as the FocalLossV3 of the reference's repository root does
    (focal_loss.py:196), and keeps it for backward: one pass over the inputs per step instead of two. The default keeps
    nothing but the inputs (the packaged copy, pytorch_loss/focal_loss.py:173)."""

    def __init__(self, alpha=0.25, gamma=2, reduction="mean", fb=False):
        super().__init__()
        self.alpha = alpha
        self.gamma = gamma
        self.reduction = reduction
        self.fb = fb

    def forward(self, logits, label):
        # fp16 logits keep the two passes: a gradient kept in fp16 at 1/numel of its size is subnormal before a loss
        # scale could lift it, where the backward kernel multiplies in fp32 and rounds once
        # (and a forward that no backward will follow computes no gradient)
        fused = self.fb and logits.dtype != torch.float16 and logits.requires_grad and torch.is_grad_enabled()
        if fused and self.reduction in ("mean", "sum") and logits.numel() > 0:
            return _FocalFusedReducedFunction.apply(logits, label, self.alpha, self.gamma, self.reduction == "mean")
        if not fused and self.reduction in ("mean", "sum") and logits.numel() > 0:
            return _FocalReducedFunction.apply(logits, label, self.alpha, self.gamma, self.reduction == "mean")
        # per-element losses: the two-kernel Function moves the same bytes as the fused one once the upstream multiply
        # is folded into the backward kernel, and keeps no gradient-sized tensor alive
        func = FocalSigmoidLossFuncV3FB if self.fb else FocalSigmoidLossFuncV3
        loss = func.apply(logits, label, self.alpha, self.gamma)
        if self.reduction == "mean":
            return loss.mean()
        if self.reduction == "sum":
            return loss.sum()
        return loss
