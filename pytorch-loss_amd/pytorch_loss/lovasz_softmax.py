"""Lovasz-softmax on the HIP kernels.

Same surface as the reference's V3 pair (pytorch_loss/lovasz_softmax.py:75-116):
``LovaszSoftmaxFunctionV3.apply(logits, labels, ignore_index)`` returns one loss per
class (every class, present in the batch or not), the module reduces over classes.
"""
import torch
import torch.nn as nn

from . import _native


class LovaszSoftmaxFunctionV3(torch.autograd.Function):
    """Keeps the Jaccard differences (C x pixels, fp32) between forward and backward."""

    @staticmethod
    def forward(ctx, logits, labels, ignore_index):
        ctx.args = args = _native.lovasz_args(logits, labels)
        losses, jacc = _native.lovasz_forward(logits, labels, ignore_index, args=args)
        ctx.vars = (logits, labels, jacc, ignore_index)
        return losses

    @staticmethod
    def backward(ctx, grad_output):
        logits, labels, jacc, ignore_index = ctx.vars
        grad = _native.lovasz_backward(grad_output, logits, labels, jacc, ignore_index, args=ctx.args)
        return grad, None, None


class LovaszSoftmaxV3(nn.Module):
    """Usage as nn.CrossEntropyLoss. reduction 'mean'/'sum' act on the C per-class losses."""

    def __init__(self, reduction="mean", ignore_index=-100):
        super().__init__()
        self.reduction = reduction
        self.lb_ignore = ignore_index

    def forward(self, logits, label):
        losses = LovaszSoftmaxFunctionV3.apply(logits, label, self.lb_ignore)
        if self.reduction == "sum":
            return losses.sum()
        if self.reduction == "mean":
            return losses.mean()
        return losses
