"""Layer norm over the channel dimension of NCHW tensors on the HIP kernels.

Same surface as the reference's V3 pair (pytorch_loss/layer_norm.py:111-167):
``LayerNormV3(n_chan, affine=True, eps=1e-6)(x)`` normalises a ``(N, C, H, W)`` tensor over C and
applies a per-channel weight and bias with ordinary torch ops; ``LayerNormV3Func.apply(x, eps)``
takes ``(N, C, M)``.

The Function's backward returns what the reference's kernel returns (csrc/layer_norm.cu:212-216),
which is not the derivative of the forward; it is kept because the point of this module is to give
the reference's results.  fp16 inputs are read natively (the arithmetic is fp32 inside the kernels,
so the reference's cast to fp32 against overflow, pytorch_loss/layer_norm.py:131, is not needed).
"""
import torch
import torch.nn as nn

from . import _native


class LayerNormV3Func(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, eps):
        y, xc, tag = _native.layer_norm_forward(x, eps)
        ctx.saved = (xc, tag, eps, x.dtype)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        return _native.layer_norm_backward(grad_output, *ctx.saved), None


class LayerNormV3(nn.Module):

    def __init__(self, n_chan, affine=True, eps=1e-6):
        super().__init__()
        self.n_chan = n_chan
        self.affine = affine
        self.eps = eps
        per_channel = (1, n_chan, 1)
        self.weight = nn.Parameter(torch.ones(per_channel)) if affine else None
        self.bias = nn.Parameter(torch.zeros(per_channel)) if affine else None

    def forward(self, x):
        n, c, h, w = x.shape                     # NCHW only, like the reference
        y = LayerNormV3Func.apply(x.view(n, c, h * w), self.eps).to(x.dtype)
        if self.affine:
            y = self.weight * y + self.bias
        return y.view(n, c, h, w)
