"""Online hard example mining losses on the HIP kernels.

Same surface as the reference's pytorch_loss/ohem_loss.py:13-45: both modules first relabel the
easy pixels as ignored (``score_ohem_label``: beyond the ``n_min`` lowest-scoring pixels, every
pixel whose softmax probability at its label exceeds ``score_thresh`` gets ``ignore_index``),
then take the mean loss over what is left.  ``OhemCELoss`` uses plain cross entropy (the reference calls
``nn.CrossEntropyLoss(ignore_index, reduction='mean')``, ohem_loss.py:20): the relabelling pass over
the logits already has every pixel's cross entropy at hand, so the forward is that one pass (it keeps the
selection as one byte per pixel instead of writing new labels), and the backward is the label-smoothed kernel
with a smoothing factor of 0 on the original labels and that mask;
``OhemLargeMarginLoss`` uses ``LargeMarginSoftmaxV3`` (ohem_loss.py:33-45), whose forward kernel
holds every pixel's softmax and so leaves the scores as well: again one pass over the logits.
"""
import torch
import torch.nn as nn

from . import _native
from .large_margin_softmax import LargeMarginSoftmaxV3


def score_ohem_label(logits, labels, ignore_index, score_thresh, n_min):
    """Stand-in for ``ohem_cpp.score_ohem_label`` (csrc/ohem_label_kernel.cu:266-276): new labels,
    detached from any graph; logits may be fp32, fp16 or bf16 (scores are formed in fp32)."""
    return _native.ohem_score_label(logits.detach(), labels, ignore_index, score_thresh, n_min)


class _OhemLossFunction(torch.autograd.Function):
    """Mean loss over the pixels that keep their label: cross entropy, or the large-margin loss when
    `lam` is not None. No gradient flows through the relabelling (the reference runs it under
    no_grad, ohem_loss.py:25)."""

    @staticmethod
    def forward(ctx, logits, labels, ignore_index, score_thresh, n_min, lam):
        loss, n_valid, args, kept = _native.ohem_ce_forward(logits, labels, ignore_index, score_thresh, n_min, lam)
        ctx.vars = args, kept, n_valid, ignore_index, lam
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        args, kept, n_valid, ignore_index, lam = ctx.vars
        grad = _native.ohem_backward(args, kept, ignore_index, grad_output, n_valid, lam)
        return grad, None, None, None, None, None


class _OhemLoss(nn.Module):
    lam = None       # None: cross entropy

    def __init__(self, score_thresh, n_min=None, ignore_index=255):
        super().__init__()
        self.score_thresh = score_thresh
        self.ignore_lb = ignore_index
        self.n_min = n_min

    def forward(self, logits, labels):
        n_min = labels.numel() // 16 if self.n_min is None else self.n_min
        return _OhemLossFunction.apply(logits, labels, self.ignore_lb, self.score_thresh, n_min, self.lam)


class OhemCELoss(_OhemLoss):

    def __init__(self, score_thresh, n_min=None, ignore_index=255):
        super().__init__(score_thresh, n_min, ignore_index)
        self.criteria = nn.CrossEntropyLoss(ignore_index=ignore_index, reduction="mean")    # ohem_loss.py:20; not called


class OhemLargeMarginLoss(_OhemLoss):

    def __init__(self, score_thresh, n_min=None, ignore_index=255):
        super().__init__(score_thresh, n_min, ignore_index)
        # kept for its parameters, as the reference keeps it (ohem_loss.py:40); `lam` is read per call
        self.criteria = LargeMarginSoftmaxV3(ignore_index=ignore_index, reduction="mean")

    @property
    def lam(self):
        return self.criteria.lam
