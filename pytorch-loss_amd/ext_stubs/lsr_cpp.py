"""Stands in for the extension built from csrc/lsr_kernel.cu (PYBIND11_MODULE at :319-322)."""
import torch

from ._abi import F32, I32, I64, P, bind, check, dims, gpu_only, native, stream
from ._abi import labels as int64_labels

_fwd = bind("plh_lsr_forward", [P, I32, P, P, I64, I64, I64, I64, F32, P])
_bwd = bind("plh_lsr_backward", [P, I32, P, P, I64, P, I64, I64, I64, I64, F32, P])


def lsr_forward(logits, labels, ignore_index, smooth):
    """csrc/lsr_kernel.cu:296-305 -> per-pixel losses, shape of `labels`, dtype of `logits`."""
    gpu_only("LSR loss", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    losses = torch.empty(lb.shape, dtype=torch.float32, device=x.device)     # losses are fp32 at the ABI
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, lb.data_ptr(), losses.data_ptr(), *dims(x), ignore_index, smooth, stream()))
    return losses.to(logits.dtype)


def lsr_backward(logits, labels, ignore_index, smooth):
    """csrc/lsr_kernel.cu:307-317 -> dloss/dlogits; pytorch_loss/label_smooth.py:144 then multiplies by
    the upstream gradient (a NULL grad_output asks the library for the reference's raw gradient)."""
    gpu_only("LSR loss", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    grad = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_bwd(x.data_ptr(), tag, lb.data_ptr(), None, 0, grad.data_ptr(), *dims(x), ignore_index, smooth,
                       stream()))
    return grad.to(logits.dtype)
