"""Stands in for the extension built from csrc/large_margin_kernel.cu (PYBIND11_MODULE at :834-838).
Python-side argument order (lam, ignore_index), as the reference's interface functions take it (:796-831)."""
import torch

from ._abi import F32, I32, I64, P, bind, check, dims, gpu_only, native, stream
from ._abi import labels as int64_labels

_fwd = bind("plh_lmargin_forward", [P, I32, P, P, I64, I64, I64, I64, F32, P])
_bwd = bind("plh_lmargin_backward", [P, I32, P, P, I64, P, I64, I64, I64, I64, F32, P])
_fb = bind("plh_lmargin_forward_backward", [P, I32, P, P, P, P, I64, I64, I64, I64, F32, P])


def l_margin_forward(logits, labels, lam, ignore_index):
    gpu_only("large margin loss", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    losses = torch.empty(lb.shape, dtype=torch.float32, device=x.device)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, lb.data_ptr(), losses.data_ptr(), *dims(x), ignore_index, lam, stream()))
    return losses.to(logits.dtype)


def l_margin_backward(logits, labels, lam, ignore_index):
    gpu_only("large margin loss", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    grad = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_bwd(x.data_ptr(), tag, lb.data_ptr(), None, 0, grad.data_ptr(), *dims(x), ignore_index, lam, stream()))
    return grad.to(logits.dtype)


def l_margin_forward_backward(logits, labels, lam, ignore_index):
    """-> (losses, dloss/dlogits, valid_cnt int64[1]), csrc/large_margin_kernel.cu:820-831."""
    gpu_only("large margin loss", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    losses = torch.empty(lb.shape, dtype=torch.float32, device=x.device)
    grad = torch.empty_like(x)
    cnt = torch.zeros(1, dtype=torch.int64, device=x.device)
    if x.numel():
        with torch.cuda.device_of(x):
            check(_fb(x.data_ptr(), tag, lb.data_ptr(), losses.data_ptr(), grad.data_ptr(), cnt.data_ptr(), *dims(x),
                      ignore_index, lam, stream()))
    return losses.to(logits.dtype), grad.to(logits.dtype), cnt
