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
        grads = ctx.variables
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


class FocalLossV3(nn.Module):
    """Usage as nn.BCEWithLogitsLoss. reduction 'mean' averages over every element."""

    def __init__(self, alpha=0.25, gamma=2, reduction="mean"):
        super().__init__()
        self.alpha = alpha
        self.gamma = gamma
        self.reduction = reduction

    def forward(self, logits, label):
        if self.reduction in ("mean", "sum") and logits.numel() > 0:
            return _FocalReducedFunction.apply(logits, label, self.alpha, self.gamma, self.reduction == "mean")
        # the two-kernel Function moves the same bytes as the fused one once the upstream
        # multiply is folded into the backward kernel, and keeps no gradient-sized tensor alive
        loss = FocalSigmoidLossFuncV3.apply(logits, label, self.alpha, self.gamma)
        if self.reduction == "mean":
            return loss.mean()
        if self.reduction == "sum":
            return loss.sum()
        return loss
