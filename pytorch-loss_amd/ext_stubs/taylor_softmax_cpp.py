"""Stands in for the extension built from csrc/taylor_softmax.cu (PYBIND11_MODULE at :419-422)."""
import torch

from ._abi import I32, I64, P, bind, check, gpu_only, native, stream

_fwd = bind("plh_taylor_softmax_forward", [P, I32, P, I64, I64, I64, I64, I32, P])
_bwd = bind("plh_taylor_softmax_backward", [P, P, I32, P, I64, I64, I64, I64, I32, P])


def _around(t, dim):
    dim = dim % t.dim()
    n = 1
    for s in t.shape[:dim]:
        n *= s
    return n, t.shape[dim], t.numel() // max(1, n * t.shape[dim])


def taylor_softmax_forward(feat, dim, n, use_log):
    """csrc/taylor_softmax.cu:395-404 -> f(x) / sum_dim f(x), or its logarithm, f the Taylor series of exp of order n."""
    gpu_only("taylor softmax function", feat)
    x, tag = native(feat)
    out = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, out.data_ptr(), *_around(x, dim), n, 1 if use_log else 0, stream()))
    return out.to(feat.dtype)


def taylor_softmax_backward(grad, feat, dim, n, use_log):
    """csrc/taylor_softmax.cu:406-417 -> gradient with respect to feat."""
    gpu_only("taylor softmax function", feat, grad)
    x, tag = native(feat)
    g = grad.to(x.dtype).expand(x.shape).contiguous()
    out = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_bwd(g.data_ptr(), x.data_ptr(), tag, out.data_ptr(), *_around(x, dim), n, 1 if use_log else 0,
                       stream()))
    return out.to(feat.dtype)
