"""One-hot / label-smoothed target encoding on the HIP kernel.

Same surface as the reference's pytorch_loss/one_hot.py:7-74: ``convert_to_one_hot`` (plain one
hot), ``convert_to_one_hot_cu`` (with label smoothing: ``1 - smooth`` at the label,
``smooth / minleng`` elsewhere) and the module ``OnehotEncoder``.  Ignored pixels become all-zero
columns.  Labels must be int64 on the GPU; a label that is neither ignored nor inside
``[0, minleng)`` raises, as in the reference.
"""
import torch
import torch.nn as nn

from . import _native


@torch.no_grad()
def convert_to_one_hot(x, minleng, ignore_idx=-1):
    """(N, ...) int64 -> (N, minleng, ...) float32 (one_hot.py:7-37; there a scatter_ on zeros)."""
    return _native.onehot(x, minleng, 0.0, ignore_idx)


@torch.no_grad()
def convert_to_one_hot_cu(x, minleng, smooth=0., ignore_idx=-1):
    """(N, ...) int64 -> (N, minleng, ...) float32 with label smoothing (one_hot.py:40-53)."""
    return _native.onehot(x, minleng, smooth, ignore_idx)


class OnehotEncoder(nn.Module):
    """one_hot.py:57-74.  ``check=False`` skips the read-back of the range flags (and with it the
    only host synchronisation of the call) for labels already known to be valid."""

    def __init__(self, n_classes, lb_smooth=0., ignore_idx=-1, check=True):
        super().__init__()
        self.n_classes = n_classes
        self.lb_smooth = lb_smooth
        self.ignore_idx = ignore_idx
        self.check = check

    @torch.no_grad()
    def forward(self, label):
        return _native.onehot(label, self.n_classes, self.lb_smooth, self.ignore_idx, self.check).detach()
