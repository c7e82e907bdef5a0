"""What the stand-in modules share: the loaded library, element-type tags, shape flattening
and the mapping of return codes to RuntimeError (the reference raises through AT_ERROR / AT_ASSERTM)."""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("PLH_LIBRARY", os.path.join(_HERE, "..", "pytorch_loss", "libpytorch_loss_hip.so"))

P, I32, I64, F32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
TAG = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}      # PLH_DTYPE_F32 / _F16 / _BF16

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python pytorch-loss_amd/build.py`" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.plh_error_string.restype = ctypes.c_char_p
        _lib.plh_error_string.argtypes = [ctypes.c_int]
    return _lib


def bind(name, argtypes, restype=ctypes.c_int):
    fn = getattr(lib(), name)
    fn.argtypes, fn.restype = argtypes, restype
    return fn


def check(rc):
    if rc:
        raise RuntimeError(lib().plh_error_string(rc).decode())


def dims(t):
    """(n_size, dimsize, m_size) as the reference flattens them (csrc/lsr_kernel.cu:199-202)."""
    n, c = t.shape[0], t.shape[1]
    return n, c, t.numel() // max(1, n * c)


def native(t):
    """fp32 / fp16 / bf16 tensors are read as they are, anything else through an fp32 copy."""
    t = t if t.dtype in TAG else t.float()
    return t.contiguous(), TAG[t.dtype]


def stream():
    return torch.cuda.current_stream().cuda_stream


def gpu_only(what, *tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("this %s only supports gpu mode" % what)


def labels(t, logits):
    """The int64 labels of `logits` as the C ABI reads them: the reference takes them through
    `labels.contiguous().data_ptr<int64_t>()` (e.g. csrc/lsr_kernel.cu:224), which raises for any other dtype;
    a label tensor that is not (N, *) of the logits' (N, C, *) would be read out of bounds, so it raises too."""
    if t.dtype != torch.int64:
        raise RuntimeError("expected scalar type Long for the labels but found %s" % t.dtype)
    n, _, m = dims(logits)
    if t.numel() != n * m:
        raise RuntimeError("labels of shape %s do not go with logits of shape %s" % (tuple(t.shape), tuple(logits.shape)))
    return t.contiguous()
