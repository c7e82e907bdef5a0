"""Stands in for the extension built from csrc/one_hot_kernel.cu (PYBIND11_MODULE at :351-353)."""
import torch

from ._abi import F32, I64, P, bind, check, gpu_only, stream

_onehot = bind("plh_onehot", [P, P, P, I64, I64, I64, I64, F32, P])


def label_one_hot(labels, ignore_index, smooth, min_len):
    """csrc/one_hot_kernel.cu:339-349 -> fp32 (N, min_len, *): 1 - smooth at the label, smooth / min_len elsewhere,
    0 in every channel of an ignored pixel; labels outside [0, min_len) raise like the TORCH_CHECKs at :301-302."""
    gpu_only("onehot method", labels)
    if labels.dtype != torch.int64:
        raise RuntimeError("date type should be kLong")
    lb = labels.contiguous()
    n_size = lb.shape[0]
    out = torch.empty((n_size, min_len) + tuple(lb.shape[1:]), dtype=torch.float32, device=lb.device)
    flags = torch.empty((2,), dtype=torch.int32, device=lb.device)
    with torch.cuda.device_of(lb):
        check(_onehot(lb.data_ptr(), out.data_ptr(), flags.data_ptr(), n_size, min_len, lb.numel() // max(1, n_size),
                      ignore_index, smooth, stream()))
    too_big, negative = flags.tolist()          # the reference reads its max / min back the same way (:154-155)
    if too_big:
        raise RuntimeError("label should be less than min_len")
    if negative:
        raise RuntimeError("label should be more than 0")
    return out
