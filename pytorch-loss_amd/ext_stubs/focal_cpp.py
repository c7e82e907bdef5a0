"""Stands in for the extension built from csrc/focal_kernel.cu (PYBIND11_MODULE at :337-341).
Argument order (gamma, alpha) as on the reference's C++ side (:301-304)."""
import torch

from ._abi import F32, I32, I64, P, TAG, bind, check, gpu_only, stream

_fwd = bind("plh_focal_forward", [P, I32, P, P, I64, F32, F32, P])
_bwd = bind("plh_focal_backward", [P, I32, P, P, I64, P, I64, F32, F32, P])
_fb = bind("plh_focal_forward_backward", [P, I32, P, P, P, I64, F32, F32, P])


def _pair(logits, labels):
    """Logits and labels in one element type the kernels read (csrc/focal_kernel.cu:173 asserts equal types)."""
    gpu_only("focal loss", logits, labels)
    if logits.shape != labels.shape:
        raise RuntimeError("labels and logits must have the same shape")
    if logits.dtype == labels.dtype and logits.dtype in TAG:
        return logits.contiguous(), labels.contiguous(), TAG[logits.dtype]
    return logits.float().contiguous(), labels.float().contiguous(), 0


def focalloss_forward(logits, labels, gamma, alpha):
    x, y, tag = _pair(logits, labels)
    losses = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, y.data_ptr(), losses.data_ptr(), x.numel(), gamma, alpha, stream()))
    return losses.to(logits.dtype)


def focalloss_backward(logits, labels, gamma, alpha):
    x, y, tag = _pair(logits, labels)
    grad = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_bwd(x.data_ptr(), tag, y.data_ptr(), None, 0, grad.data_ptr(), x.numel(), gamma, alpha, stream()))
    return grad.to(logits.dtype)


def focalloss_forward_backward(logits, labels, gamma, alpha):
    """-> (losses, dloss/dlogits), csrc/focal_kernel.cu:323-335."""
    x, y, tag = _pair(logits, labels)
    losses = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    grad = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fb(x.data_ptr(), tag, y.data_ptr(), losses.data_ptr(), grad.data_ptr(), x.numel(), gamma, alpha,
                      stream()))
    return losses.to(logits.dtype), grad.to(logits.dtype)
