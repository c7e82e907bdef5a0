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
        out, xc, tag = _native.layer_norm_forward(x, eps)
        ctx.vars = xc, tag, eps, x.dtype
        return out

    @staticmethod
    def backward(ctx, grad_output):
        xc, tag, eps, dtype = ctx.vars
        return _native.layer_norm_backward(grad_output, xc, tag, eps, dtype), None


class LayerNormV3(nn.Module):

    def __init__(self, n_chan, affine=True, eps=1e-6):
        super().__init__()
        self.n_chan, self.affine = n_chan, affine
        self.weight, self.bias = None, None
        self.eps = eps
        if affine:
            self.weight = nn.Parameter(torch.ones(1, n_chan, 1))
            self.bias = nn.Parameter(torch.zeros(1, n_chan, 1))

    def forward(self, x):
        N, C, H, W = x.size()
        x = x.view(N, C, -1)
        dt = x.dtype
        x = LayerNormV3Func.apply(x, self.eps).to(dt)
        if self.affine:
            x = self.weight * x + self.bias
        return x.view(N, C, H, W)
