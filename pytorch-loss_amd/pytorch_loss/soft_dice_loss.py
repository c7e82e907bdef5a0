"""Soft dice loss for binary segmentation on the HIP kernels.

Same surface as the reference's V3 pair (pytorch_loss/soft_dice_loss.py:112-164):
``SoftDiceLossV3(p, smooth)(logits, labels)`` flattens both tensors into one row and returns a
``(1,)`` loss; ``SoftDiceLossV3Func.apply(logits, labels, p, smooth)`` takes ``(N, L)`` tensors
and returns one loss per row.  Labels are floats of the logits' shape.
"""
import torch
import torch.nn as nn

from . import _native


class SoftDiceLossV3Func(torch.autograd.Function):
    """forward -> (N,) losses; keeps the inputs and each row's (numer, denor), so backward is one
    elementwise kernel."""

    @staticmethod
    def forward(ctx, logits, labels, p, smooth):
        assert logits.size() == labels.size() and logits.dim() == 2
        loss, stats, args = _native.soft_dice_forward(logits, labels, p, smooth)
        ctx.vars = args, stats, p
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        args, stats, p = ctx.vars
        return _native.soft_dice_backward(grad_output, stats, p, args), None, None, None


class SoftDiceLossV3(nn.Module):

    def __init__(self, p=1, smooth=1.):
        super().__init__()
        self.p = p
        self.smooth = smooth

    def forward(self, logits, labels):
        logits = logits.view(1, -1)
        labels = labels.view(1, -1)
        return SoftDiceLossV3Func.apply(logits, labels, self.p, self.smooth)
