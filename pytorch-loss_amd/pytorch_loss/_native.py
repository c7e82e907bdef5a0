"""ctypes binding of libpytorch_loss_hip.so and the tensor marshalling around it.

The shared library speaks plain pointers and sizes (include/pytorch_loss_hip.h).
This module owns everything the reference's C++ host wrappers did with ATen:
device checks, `.contiguous()`, output and workspace allocation (through torch's
caching allocator, so the library itself never allocates), device guard and
current-stream lookup, and turning non-zero return codes into RuntimeError.

There is no fallback: if the library is missing or a tensor is not on a GPU the
call raises, like the reference's AT_ERROR("... only supports gpu mode")
(csrc/lsr_kernel.cu:300-302).
"""
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpytorch_loss_hip.so")
ABI_VERSION = 5

_lib = None

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_i32 = ctypes.c_int32

_SIGNATURES = {
    "plh_abi_version": (ctypes.c_int, []),
    "plh_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "plh_reduce_workspace_bytes": (_i64, [_i64]),
    "plh_lsr_forward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lsr_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lsr_forward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lsr_forward_reduced_static": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lsr_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_focal_forward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _f32, _f32, _p]),
    "plh_focal_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _p, _i64, _f32, _f32, _p]),
    "plh_focal_forward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _i32, _p, _i64, _i64, _f32, _f32, _p]),
    "plh_focal_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _i64, _f32, _f32, _p]),
    "plh_focal_forward_backward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _i64, _f32, _f32, _p]),
    "plh_lsr_forward_backward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_focal_forward_backward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _i32, _p, _i64, _i64, _f32, _f32, _p]),
    "plh_lmargin_forward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_forward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_forward_backward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_forward_backward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_scale_unless_one": (ctypes.c_int, [_p, _i32, _i64, _p, _p]),
    "plh_lmargin_saves_stats": (ctypes.c_int, [_i32, _i64, _i64, _i64]),
    "plh_lmargin_forward_reduced_stats": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward_scaled_stats": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lovasz_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "plh_lovasz_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_lsr_saves_lse": (ctypes.c_int, [_i32, _i64, _i64, _i64]),
    "plh_lsr_forward_reduced_lse": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lsr_backward_scaled_lse": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lovasz_lookback_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "plh_lovasz_forward_lookback": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_lovasz_backward": (ctypes.c_int, [_p, _p, _i32, _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "plh_ohem_workspace_bytes": (_i64, [_i64]),
    "plh_ohem_scores": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "plh_ohem_select_labels": (ctypes.c_int, [_p, _p, _p, _p, _i64, _i64, _i64, _f32, _i64, _p]),
    "plh_ohem_score_label": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _p]),
    "plh_ohem_ce_workspace_bytes": (_i64, [_i64]),
    "plh_ohem_ce_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32, _i64,
                                           _p]),
    "plh_ohem_lmargin_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32,
                                                _f32, _i64, _p]),
    "plh_ohem_ce_forward_kept": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32,
                                                _i64, _p]),
    "plh_ohem_lmargin_forward_kept": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64,
                                                     _f32, _f32, _i64, _p]),
    "plh_lsr_backward_kept": (ctypes.c_int, [_p, _i32, _p, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward_kept": (ctypes.c_int, [_p, _i32, _p, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_taylor_softmax_forward": (ctypes.c_int, [_p, _i32, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "plh_taylor_softmax_backward": (ctypes.c_int, [_p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "plh_taylor_ce_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_taylor_ce_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _f32, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_taylor_ce_saves_sums": (ctypes.c_int, [_i32, _i64, _i64, _i64]),
    "plh_taylor_ce_forward_reduced_sums": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_taylor_ce_backward_scaled_sums": (ctypes.c_int, [_p, _i32, _p, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_soft_dice_workspace_bytes": (_i64, [_i64, _i64]),
    "plh_soft_dice_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _f32, _f32, _p]),
    "plh_soft_dice_backward": (ctypes.c_int, [_p, _p, _i32, _p, _p, _p, _i64, _i64, _f32, _p]),
    "plh_layer_norm_forward": (ctypes.c_int, [_p, _i32, _p, _i64, _i64, _i64, _f32, _p]),
    "plh_layer_norm_backward": (ctypes.c_int, [_p, _p, _i32, _p, _i64, _i64, _i64, _f32, _p]),
    "plh_onehot": (ctypes.c_int, [_p, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_stream_copy": (ctypes.c_int, [_p, _p, _i64, _p]),
}


def load():
    """Load the HIP library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "pytorch_loss: %s is missing; build it with `python pytorch-loss_amd/build.py` "
                "(there is no CPU or pure-PyTorch fallback)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise RuntimeError("pytorch_loss: %s does not export %s; rebuild it" % (LIB_PATH, name))
            fn.restype = res
            fn.argtypes = args
        got = lib.plh_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError("pytorch_loss: library ABI %d, binding expects %d" % (got, ABI_VERSION))
        _lib = lib
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError("pytorch_loss HIP library: %s (code %d)" % (load().plh_error_string(rc).decode(), rc))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device=None):
    """The current HIP stream of `device` (default: the current device) as a pointer argument."""
    if _raw_stream is not None:
        return _p(_raw_stream(torch.cuda.current_device() if device is None or device.index is None
                              else device.index))
    if device is None:
        return _p(torch.cuda.current_stream().cuda_stream)
    return _p(torch.cuda.current_stream(device).cuda_stream)


def _ptr(t):
    return _p(t.data_ptr()) if t is not None else _p(0)


def _call(x, entry, *args):
    """Run library function `entry` with `x`'s device current (the library launches on whatever
    device is current) and on that device's current stream, appended as the last argument."""
    fn = getattr(load(), entry)
    dev = x.device
    if dev.index is None or dev.index == torch.cuda.current_device():
        rc = fn(*args, _stream(dev))
    else:
        with torch.cuda.device(dev):
            rc = fn(*args, _stream(dev))
    if rc != 0:
        _check(rc)


def _require_gpu(what, *tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("this %s only supports gpu mode" % what)
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError("%s: all tensors must be on the same device" % what)


def _f32c(t):
    """fp32 contiguous view/copy."""
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


_DTYPE_TAGS = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _logits(t):
    """-> (contiguous tensor in a dtype the kernels read natively, dtype tag). fp32, fp16 and bf16
    are read as they are (arithmetic is fp32 in every case); anything else is cast to fp32 first."""
    if t.dtype not in _DTYPE_TAGS:
        t = t.float()
    return t.contiguous(), _DTYPE_TAGS[t.dtype]


def _loss_dtype(dtype):
    """dtype of the returned losses for logits of `dtype`: the same, except under autocast, where
    the reference's custom_fwd(cast_inputs=float32) makes the whole op fp32."""
    return torch.float32 if torch.is_autocast_enabled("cuda") else dtype


def _labels_i64(labels, logits, what):
    if labels.dtype != torch.int64:
        if labels.is_floating_point() or labels.dtype == torch.bool:
            raise RuntimeError("%s: labels must be an integer tensor (int64)" % what)
        labels = labels.long()
    if tuple(labels.shape) != tuple(logits.shape[:1]) + tuple(logits.shape[2:]):
        raise RuntimeError("%s: labels of shape %s do not match logits of shape %s (expect (N, *) vs (N, C, *))"
                           % (what, tuple(labels.shape), tuple(logits.shape)))
    return labels.contiguous()


def _dims(logits, what):
    if logits.dim() < 2:
        raise RuntimeError("%s: logits must have at least 2 dims (N, C, ...)" % what)
    n_size, dimsize = int(logits.shape[0]), int(logits.shape[1])
    m_size = 1
    for d in logits.shape[2:]:
        m_size *= int(d)
    return n_size, dimsize, m_size


def _upstream(grad_output, like_shape):
    """-> (tensor kept alive or None, stride). Expanded scalars are passed as one value."""
    if grad_output is None:
        return None, 0
    if tuple(grad_output.shape) != tuple(like_shape):
        grad_output = grad_output.expand(like_shape)
    if grad_output.numel() > 0 and all(s == 0 for s, n in zip(grad_output.stride(), grad_output.shape) if n > 1):
        # produced by sum()/mean() backward: a single value broadcast over the loss tensor
        one = grad_output.as_strided((1,), (1,))
        if one.dtype != torch.float32:
            one = one.float()
        return one, 0
    return _f32c(grad_output), 1


def _back_to(t, dtype):
    return t if dtype == torch.float32 else t.to(dtype)


# ------------------------------------------------------------------ LSR ----
# LSR and large-margin share their marshalling: `entry` names the library function, `param` is the
# smoothing factor or the margin weight.

class SegArgs:
    """Checked and marshalled (logits, labels) of a channel-dim loss: computed once in forward and
    handed to backward, which works on the same tensors."""
    __slots__ = ("x", "tag", "lb", "n", "c", "m", "dtype")


def seg_args(logits, labels, what, entry):
    _require_gpu(what, logits, labels)
    a = SegArgs()
    a.n, a.c, a.m = _dims(logits, entry)
    a.x, a.tag = _logits(logits)
    a.lb = _labels_i64(labels, logits, entry)
    a.dtype = logits.dtype
    return a


def _pixel_forward(entry, a, ignore_index, param):
    losses = torch.empty(a.lb.shape, dtype=torch.float32, device=a.x.device)
    if a.x.numel() == 0:
        return _back_to(losses.zero_(), _loss_dtype(a.dtype))
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(losses), a.n, a.c, a.m, int(ignore_index), float(param))
    return _back_to(losses, _loss_dtype(a.dtype))


def _pixel_backward(entry, a, ignore_index, param, grad_output):
    """dloss/dlogits, already multiplied by ``grad_output`` (None = unit upstream gradient)."""
    grad = torch.empty_like(a.x)
    if a.x.numel() == 0:
        return _back_to(grad, a.dtype)
    go, stride = _upstream(grad_output, a.lb.shape)
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(go), stride, _ptr(grad), a.n, a.c, a.m,
          int(ignore_index), float(param))
    return _back_to(grad, a.dtype)


# Reduction workspaces (per-block partial sums of a fused 'mean' / 'sum') are kept per (device, stream, thread):
# a forward writes its partials and its finishing kernel reads them on the same stream, so the next call on that
# stream may use the same bytes, and a step costs one dictionary look-up where it cost an allocation and a call
# into the library. Calls under stream capture allocate as before (their memory belongs to the graph's pool).
_WS_BYTES = {}
_WS_CACHE = {}


def _reduce_workspace(units, device):
    units = int(units)
    nbytes = _WS_BYTES.get(units)
    if nbytes is None:
        nbytes = int(load().plh_reduce_workspace_bytes(units))
        if nbytes < 0:
            _check(nbytes)
        if len(_WS_BYTES) < 4096:
            _WS_BYTES[units] = nbytes
    index = device.index if device.index is not None else torch.cuda.current_device()
    if _raw_stream is None or torch.cuda.is_current_stream_capturing():
        return torch.empty((nbytes,), dtype=torch.uint8, device=device), nbytes
    key = (index, _raw_stream(index), threading.get_ident())
    ws = _WS_CACHE.get(key)
    if ws is None or ws.numel() < nbytes:
        if len(_WS_CACHE) >= 64:
            _WS_CACHE.clear()
        ws = _WS_CACHE[key] = torch.empty((nbytes,), dtype=torch.uint8, device=device)
    return ws, nbytes


def _scalar_f32(t):
    """A 0-dim upstream gradient as one fp32 value in device memory."""
    if t.dtype == torch.float32 and t.numel() == 1:
        return t
    t = t.reshape(-1)[:1]
    return t if t.dtype == torch.float32 else t.float()


def _pixel_forward_reduced(entry, a, ignore_index, param, mean):
    """-> (loss 0-dim, n_valid 0-dim int64)."""
    loss = torch.empty((), dtype=torch.float32, device=a.x.device)
    n_valid = torch.empty((), dtype=torch.int64, device=a.x.device)
    ws, ws_bytes = _reduce_workspace(a.n * a.m, a.x.device)
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), None, _ptr(loss), _ptr(n_valid), 1 if mean else 0,
          _ptr(ws), ws_bytes, a.n, a.c, a.m, int(ignore_index), float(param))
    return _back_to(loss, _loss_dtype(a.dtype)), n_valid


def _pixel_backward_scaled(entry, a, ignore_index, param, grad_scalar, divide_by):
    grad = torch.empty_like(a.x)
    if a.x.numel() == 0:
        return _back_to(grad, a.dtype)
    go = _scalar_f32(grad_scalar)
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(go), 1.0, _ptr(divide_by), _ptr(grad), a.n, a.c, a.m,
          int(ignore_index), float(param))
    return _back_to(grad, a.dtype)


def lsr_args(logits, labels):
    return seg_args(logits, labels, "LSR loss", "lsr")


def lsr_forward(logits, labels, ignore_index, smooth, args=None):
    return _pixel_forward("plh_lsr_forward", args or lsr_args(logits, labels), ignore_index, smooth)


def lsr_backward(logits, labels, ignore_index, smooth, grad_output=None, args=None):
    return _pixel_backward("plh_lsr_backward", args or lsr_args(logits, labels), ignore_index, smooth, grad_output)


def lsr_forward_reduced(logits, labels, ignore_index, smooth, mean, args=None):
    return _pixel_forward_reduced("plh_lsr_forward_reduced", args or lsr_args(logits, labels), ignore_index, smooth,
                                  mean)


def lsr_backward_scaled(logits, labels, ignore_index, smooth, grad_scalar, divide_by=None, args=None):
    return _pixel_backward_scaled("plh_lsr_backward_scaled", args or lsr_args(logits, labels), ignore_index, smooth,
                                  grad_scalar, divide_by)


def lsr_forward_reduced_lse(logits, labels, ignore_index, smooth, mean, args=None):
    """lsr_forward_reduced that also keeps every pixel's log-sum-exp where the library's backward can use it (fp32
    logits on channel planes of odd length, see plh_lsr_saves_lse). -> (loss, n_valid, lse or None)."""
    a = args or lsr_args(logits, labels)
    if a.x.numel() == 0 or not load().plh_lsr_saves_lse(a.tag, a.n, a.c, a.m):
        return _pixel_forward_reduced("plh_lsr_forward_reduced", a, ignore_index, smooth, mean) + (None,)
    dev = a.x.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    n_valid = torch.empty((), dtype=torch.int64, device=dev)
    lse = torch.empty((a.n * a.m,), dtype=torch.float32, device=dev)
    ws, ws_bytes = _reduce_workspace(a.n * a.m, dev)
    _call(a.x, "plh_lsr_forward_reduced_lse", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(lse), _ptr(loss), _ptr(n_valid),
          1 if mean else 0, _ptr(ws), ws_bytes, a.n, a.c, a.m, int(ignore_index), float(smooth))
    return _back_to(loss, _loss_dtype(a.dtype)), n_valid, lse


def lsr_backward_scaled_lse(lse, ignore_index, smooth, grad_scalar, divide_by, args, kept=None):
    """The gradient from the forward's log-sum-exp (lsr_forward_reduced_lse); `kept`: optional byte mask."""
    a = args
    grad = torch.empty_like(a.x)
    go = _scalar_f32(grad_scalar)
    _call(a.x, "plh_lsr_backward_scaled_lse", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(lse), _ptr(kept) if kept is not None else None,
          _ptr(go), 1.0, _ptr(divide_by), _ptr(grad), a.n, a.c, a.m, int(ignore_index), float(smooth))
    return _back_to(grad, a.dtype)


# -------------------------------------------------------------- lmargin ----

def lmargin_args(logits, labels):
    return seg_args(logits, labels, "large margin loss", "l_margin")


def lmargin_forward(logits, labels, lam, ignore_index, args=None):
    return _pixel_forward("plh_lmargin_forward", args or lmargin_args(logits, labels), ignore_index, lam)


def lmargin_backward(logits, labels, lam, ignore_index, grad_output=None, args=None):
    return _pixel_backward("plh_lmargin_backward", args or lmargin_args(logits, labels), ignore_index, lam,
                           grad_output)


def lmargin_forward_reduced(logits, labels, lam, ignore_index, mean, args=None):
    return _pixel_forward_reduced("plh_lmargin_forward_reduced", args or lmargin_args(logits, labels), ignore_index,
                                  lam, mean)


def lmargin_backward_scaled(logits, labels, lam, ignore_index, grad_scalar, divide_by=None, args=None):
    return _pixel_backward_scaled("plh_lmargin_backward_scaled", args or lmargin_args(logits, labels), ignore_index,
                                  lam, grad_scalar, divide_by)


def lmargin_forward_reduced_stats(logits, labels, lam, ignore_index, mean, args=None):
    """lmargin_forward_reduced that also keeps every row's statistics where the library's backward can use them (long
    rows, see plh_lmargin_saves_stats). -> (loss, n_valid, stats or None)."""
    a = args or lmargin_args(logits, labels)
    if a.x.numel() == 0 or not load().plh_lmargin_saves_stats(a.tag, a.n, a.c, a.m):
        return _pixel_forward_reduced("plh_lmargin_forward_reduced", a, ignore_index, lam, mean) + (None,)
    dev = a.x.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    n_valid = torch.empty((), dtype=torch.int64, device=dev)
    stats = torch.empty((a.n * a.m, 8), dtype=torch.float32, device=dev)
    ws, ws_bytes = _reduce_workspace(a.n * a.m, dev)
    _call(a.x, "plh_lmargin_forward_reduced_stats", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(stats), _ptr(loss), _ptr(n_valid),
          1 if mean else 0, _ptr(ws), ws_bytes, a.n, a.c, a.m, int(ignore_index), float(lam))
    return _back_to(loss, _loss_dtype(a.dtype)), n_valid, stats


def lmargin_backward_scaled_stats(stats, lam, ignore_index, grad_scalar, divide_by, args, kept=None):
    """The gradient from the forward's row statistics (lmargin_forward_reduced_stats); `kept`: optional byte mask."""
    a = args
    grad = torch.empty_like(a.x)
    go = _scalar_f32(grad_scalar)
    _call(a.x, "plh_lmargin_backward_scaled_stats", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(stats),
          _ptr(kept) if kept is not None else None, _ptr(go), 1.0, _ptr(divide_by), _ptr(grad), a.n, a.c, a.m,
          int(ignore_index), float(lam))
    return _back_to(grad, a.dtype)


def lmargin_forward_backward(logits, labels, lam, ignore_index):
    """-> (losses, grad under unit upstream gradient, valid_cnt int64[1])"""
    a = lmargin_args(logits, labels)
    losses = torch.empty(a.lb.shape, dtype=torch.float32, device=a.x.device)
    grad = torch.empty_like(a.x)
    cnt = torch.zeros(1, dtype=torch.int64, device=a.x.device)
    if a.x.numel():
        _call(a.x, "plh_lmargin_forward_backward", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(losses), _ptr(grad), _ptr(cnt),
              a.n, a.c, a.m, int(ignore_index), float(lam))
    else:
        losses.zero_()
    return _back_to(losses, _loss_dtype(a.dtype)), _back_to(grad, a.dtype), cnt


def lsr_forward_backward_reduced(logits, labels, ignore_index, smooth, mean):
    return _pixel_forward_backward_reduced("plh_lsr_forward_backward_reduced", lsr_args(logits, labels), ignore_index,
                                           smooth, mean)


def lmargin_forward_backward_reduced(logits, labels, lam, ignore_index, mean):
    return _pixel_forward_backward_reduced("plh_lmargin_forward_backward_reduced", lmargin_args(logits, labels),
                                           ignore_index, lam, mean)


def _pixel_forward_backward_reduced(entry, a, ignore_index, param, mean):
    """One pass over the logits: -> (loss: the sum or the mean, gradient under an upstream gradient of 1, the
    gradient's dtype tag or None)."""
    dev = a.x.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    n_valid = torch.empty((), dtype=torch.int64, device=dev)
    grad = torch.empty_like(a.x)
    ws, ws_bytes = _reduce_workspace(a.n * a.m, dev)
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(loss), _ptr(n_valid), _ptr(grad),
          1 if mean else 0, _ptr(ws), ws_bytes, a.n, a.c, a.m, int(ignore_index), float(param))
    return _back_to(loss, _loss_dtype(a.dtype)), _back_to(grad, a.dtype), (a.tag if a.x.dtype == a.dtype else None)


def take_kept(ctx):
    """The gradient that a forward+backward Function kept in ctx.variables, handed over to the one backward that may use
    it: while the context still referred to the tensor, autograd would copy it into logits.grad (a pass over it) instead
    of taking it, and a second backward would multiply it a second time."""
    kept = ctx.variables
    if kept is None:
        raise RuntimeError("pytorch_loss: the gradient kept by this forward+backward (fb) loss went to an earlier "
                           "backward(); run the forward again, or use fb=False to call backward() twice")
    ctx.variables = None
    return kept


def scale_unless_one(data, tag, grad_scalar):
    """data *= grad_scalar in place (a 0-dim tensor), without touching data when it is exactly 1; tag: the library's
    dtype tag of `data`, or None for a tensor the library does not hold (then torch multiplies)."""
    if tag is None or not data.is_contiguous() or data.data_ptr() % 16 != 0:
        return data.mul_(grad_scalar)
    if data.numel():
        _call(data, "plh_scale_unless_one", _ptr(data), tag, data.numel(), _ptr(_scalar_f32(grad_scalar)))
    return data


# ---------------------------------------------------------------- focal ----

class FocalArgs:
    """Logits and labels in one dtype the kernels read; mixed or exotic dtypes become fp32 copies."""
    __slots__ = ("x", "y", "tag", "dtype")


def focal_args(logits, labels, what="focalloss"):
    _require_gpu("focal loss", logits, labels)
    if labels.shape != logits.shape:
        raise RuntimeError("%s: labels and logits must have the same shape" % what)
    a = FocalArgs()
    a.dtype = logits.dtype
    if logits.dtype == labels.dtype and logits.dtype in _DTYPE_TAGS:
        a.x, a.y, a.tag = logits.contiguous(), labels.contiguous(), _DTYPE_TAGS[logits.dtype]
    else:
        a.x, a.y, a.tag = _f32c(logits), _f32c(labels), 0
    return a


def focal_forward(logits, labels, gamma, alpha, args=None):
    a = args or focal_args(logits, labels, "focalloss_forward")
    losses = torch.empty(a.x.shape, dtype=torch.float32, device=a.x.device)
    if a.x.numel():
        _call(a.x, "plh_focal_forward", _ptr(a.x), a.tag, _ptr(a.y), _ptr(losses), a.x.numel(), float(gamma),
              float(alpha))
    return _back_to(losses, _loss_dtype(a.dtype))


def focal_backward(logits, labels, gamma, alpha, grad_output=None, args=None):
    a = args or focal_args(logits, labels, "focalloss_backward")
    grad = torch.empty_like(a.x)
    if a.x.numel():
        go, stride = _upstream(grad_output, a.x.shape)
        _call(a.x, "plh_focal_backward", _ptr(a.x), a.tag, _ptr(a.y), _ptr(go), stride, _ptr(grad), a.x.numel(),
              float(gamma), float(alpha))
    return _back_to(grad, a.dtype)


def focal_forward_backward(logits, labels, gamma, alpha):
    a = focal_args(logits, labels, "focalloss_forward_backward")
    losses = torch.empty(a.x.shape, dtype=torch.float32, device=a.x.device)
    grad = torch.empty_like(a.x)
    if a.x.numel():
        _call(a.x, "plh_focal_forward_backward", _ptr(a.x), a.tag, _ptr(a.y), _ptr(losses), _ptr(grad), a.x.numel(),
              float(gamma), float(alpha))
    return _back_to(losses, _loss_dtype(a.dtype)), _back_to(grad, a.dtype)


def focal_forward_backward_reduced(logits, labels, gamma, alpha, mean):
    """One pass: -> (loss: the sum or the mean, gradient under an upstream gradient of 1, dtype tag of the gradient or None)."""
    a = focal_args(logits, labels, "focalloss_forward_backward")
    loss = torch.empty((), dtype=torch.float32, device=a.x.device)
    grad = torch.empty_like(a.x)
    ws, ws_bytes = _reduce_workspace(a.x.numel(), a.x.device)
    _call(a.x, "plh_focal_forward_backward_reduced", _ptr(a.x), a.tag, _ptr(a.y), _ptr(loss), _ptr(grad), 1 if mean else 0,
          _ptr(ws), ws_bytes, a.x.numel(), float(gamma), float(alpha))
    return _back_to(loss, _loss_dtype(a.dtype)), _back_to(grad, a.dtype), (a.tag if a.x.dtype == a.dtype else None)


def focal_forward_reduced(logits, labels, gamma, alpha, mean, args=None):
    a = args or focal_args(logits, labels, "focalloss_forward")
    loss = torch.empty((), dtype=torch.float32, device=a.x.device)
    ws, ws_bytes = _reduce_workspace(a.x.numel(), a.x.device)
    _call(a.x, "plh_focal_forward_reduced", _ptr(a.x), a.tag, _ptr(a.y), None, _ptr(loss), 1 if mean else 0, _ptr(ws),
          ws_bytes, a.x.numel(), float(gamma), float(alpha))
    return _back_to(loss, _loss_dtype(a.dtype))


def focal_backward_scaled(logits, labels, gamma, alpha, grad_scalar, scale, args=None):
    a = args or focal_args(logits, labels, "focalloss_backward")
    grad = torch.empty_like(a.x)
    if a.x.numel():
        go = _scalar_f32(grad_scalar)
        _call(a.x, "plh_focal_backward_scaled", _ptr(a.x), a.tag, _ptr(a.y), _ptr(go), float(scale), _ptr(grad),
              a.x.numel(), float(gamma), float(alpha))
    return _back_to(grad, a.dtype)


# --------------------------------------------------------------- lovasz ----

def lovasz_args(logits, labels):
    # same limits and wording as csrc/lovasz_softmax.cu:664-665
    if logits.numel() >= (1 << 31):
        raise RuntimeError("lovasz_softmax: input tensor too large, int32 type will overflow")
    if logits.dim() >= 2 and logits.shape[1] >= 512:
        raise RuntimeError("lovasz_softmax: num of classes should be less than BLOCKSIZE")
    return seg_args(logits, labels, "lovasz softmax function", "lovasz_softmax")


def lovasz_forward(logits, labels, ignore_index, args=None, look_back=False):
    """-> (losses[C], jacc[C, N*M] fp32). look_back=True runs the sort passes in their decoupled look-back form
    (same results bit for bit, slower; see plh_lovasz_forward_lookback)."""
    a = args or lovasz_args(logits, labels)
    entry, sizer = (("plh_lovasz_forward_lookback", "plh_lovasz_lookback_workspace_bytes") if look_back
                    else ("plh_lovasz_forward", "plh_lovasz_workspace_bytes"))
    losses = torch.empty((a.c,), dtype=torch.float32, device=a.x.device)
    jacc = torch.empty((a.c, a.n * a.m), dtype=torch.float32, device=a.x.device)
    if a.x.numel() == 0:
        return _back_to(losses.zero_(), _loss_dtype(a.dtype)), jacc
    ws_bytes = int(getattr(load(), sizer)(a.n, a.c, a.m))
    if ws_bytes < 0:
        _check(ws_bytes)
    workspace = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=a.x.device)
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(losses), _ptr(jacc), _ptr(workspace), ws_bytes,
          a.n, a.c, a.m, int(ignore_index))
    return _back_to(losses, _loss_dtype(a.dtype)), jacc


def lovasz_backward(grad_output, logits, labels, jacc, ignore_index, args=None):
    a = args or lovasz_args(logits, labels)
    _require_gpu("lovasz softmax function", a.x, grad_output, jacc)
    grad = torch.empty_like(a.x)
    if a.x.numel() == 0:
        return _back_to(grad, a.dtype)
    go = _f32c(grad_output.expand((a.c,)) if grad_output.numel() == 1 else grad_output)
    if go.numel() != a.c or jacc.numel() != a.c * a.n * a.m or jacc.dtype != torch.float32:
        raise RuntimeError("lovasz_softmax_backward: grad_output must have C elements and jacc C*N*M fp32 elements")
    jc = jacc.contiguous()
    _call(a.x, "plh_lovasz_backward", _ptr(go), _ptr(a.x), a.tag, _ptr(a.lb), _ptr(jc), _ptr(grad), a.n, a.c, a.m,
          int(ignore_index))
    return _back_to(grad, a.dtype)


# ----------------------------------------------------------------- ohem ----

def ohem_args(logits, labels):
    if labels.numel() > (1 << 31) - 1024:
        raise RuntimeError("score_ohem_label: too many pixels, int32 type will overflow")
    return seg_args(logits, labels, "ohem method", "score_ohem_label")


def _ohem_workspace(n_pixels, device):
    nbytes = int(load().plh_ohem_workspace_bytes(int(n_pixels)))
    if nbytes < 0:
        _check(nbytes)
    return torch.empty((nbytes,), dtype=torch.uint8, device=device), nbytes


def ohem_scores(logits, labels, ignore_index):
    """softmax(logits)[label] per pixel as fp32, 1 at ignored pixels."""
    a = ohem_args(logits, labels)
    scores = torch.empty(a.lb.shape, dtype=torch.float32, device=a.x.device)
    if a.x.numel():
        _call(a.x, "plh_ohem_scores", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(scores), a.n, a.c, a.m, int(ignore_index))
    return scores


def ohem_select_labels(scores, labels, ignore_index, score_thresh, n_min):
    _require_gpu("ohem method", scores, labels)
    if scores.shape != labels.shape or scores.dtype != torch.float32 or labels.dtype != torch.int64:
        raise RuntimeError("ohem_select_labels: scores (fp32) and labels (int64) must have the same shape")
    sc, lb = scores.contiguous(), labels.contiguous()
    out = torch.empty_like(lb)
    if lb.numel():
        ws, ws_bytes = _ohem_workspace(lb.numel(), lb.device)
        _call(lb, "plh_ohem_select_labels", _ptr(sc), _ptr(lb), _ptr(out), _ptr(ws), ws_bytes, lb.numel(),
              int(ignore_index), float(score_thresh), int(n_min))
    return out


def ohem_score_label(logits, labels, ignore_index, score_thresh, n_min):
    """-> new int64 labels of labels' shape; the inputs are left untouched."""
    a = ohem_args(logits, labels)
    out = torch.empty_like(a.lb)
    if a.lb.numel() == 0:
        return out
    n_pixels = a.n * a.m
    scores = torch.empty((n_pixels if n_min < n_pixels else 1,), dtype=torch.float32, device=a.x.device)
    ws, ws_bytes = _ohem_workspace(n_pixels, a.x.device)
    _call(a.x, "plh_ohem_score_label", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(out), _ptr(scores), _ptr(ws), ws_bytes,
          a.n, a.c, a.m, int(ignore_index), float(score_thresh), int(n_min))
    return out


def ohem_ce_forward(logits, labels, ignore_index, score_thresh, n_min, lam=None):
    """Selection of the hard pixels and mean loss over them, with one pass over the logits: cross entropy, or
    the large-margin loss when `lam` is given.
    -> (loss 0-dim, n_valid 0-dim int64, args, kept: one byte per pixel, 1 where the pixel takes part)."""
    a = ohem_args(logits, labels)
    dev = a.x.device
    n_pixels = a.n * a.m
    loss = torch.empty((), dtype=torch.float32, device=dev)
    n_valid = torch.empty((), dtype=torch.int64, device=dev)
    kept = torch.empty((max(n_pixels, 1),), dtype=torch.uint8, device=dev)
    scratch = torch.empty((2, max(n_pixels, 1)), dtype=torch.float32, device=dev)
    nbytes = int(load().plh_ohem_ce_workspace_bytes(n_pixels))
    if nbytes < 0:
        _check(nbytes)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    head = (_ptr(a.x), a.tag, _ptr(a.lb), _ptr(kept), _ptr(scratch[0]), _ptr(scratch[1]), _ptr(loss), _ptr(n_valid),
            _ptr(ws), nbytes, a.n, a.c, a.m, int(ignore_index))
    if lam is None:
        _call(a.x, "plh_ohem_ce_forward_kept", *head, float(score_thresh), int(n_min))
    else:
        _call(a.x, "plh_ohem_lmargin_forward_kept", *head, float(lam), float(score_thresh), int(n_min))
    return _back_to(loss, _loss_dtype(a.dtype)), n_valid, a, kept


def ohem_backward(args, kept, ignore_index, grad_scalar, n_valid, lam=None):
    """Gradient of the mean loss over the kept pixels: the cross-entropy (label smoothing 0) or large-margin
    backward on the original labels, pixels whose byte in `kept` is 0 taking no part."""
    a = args
    grad = torch.empty_like(a.x)
    if a.x.numel() == 0:
        return _back_to(grad, a.dtype)
    go = _scalar_f32(grad_scalar)
    entry, param = ("plh_lsr_backward_kept", 0.0) if lam is None else ("plh_lmargin_backward_kept", float(lam))
    _call(a.x, entry, _ptr(a.x), a.tag, _ptr(a.lb), _ptr(kept), _ptr(go), 1.0, _ptr(n_valid), _ptr(grad), a.n, a.c, a.m,
          int(ignore_index), param)
    return _back_to(grad, a.dtype)


# --------------------------------------------------------------- taylor ----

def _check_order(n):
    if n <= 0 or n % 2 != 0:
        raise AssertionError("taylor softmax: n must be a positive even number")   # taylor_softmax.py:36


def _around_dim(t, dim):
    if t.dim() == 0:
        raise RuntimeError("taylor softmax: input needs at least one dimension")
    dim = dim % t.dim()
    n_size = 1
    for d in t.shape[:dim]:
        n_size *= int(d)
    m_size = 1
    for d in t.shape[dim + 1:]:
        m_size *= int(d)
    return n_size, int(t.shape[dim]), m_size


def taylor_softmax_forward(feat, dim, n, use_log):
    _require_gpu("taylor softmax function", feat)
    _check_order(n)
    x, tag = _logits(feat)
    n_size, dimsize, m_size = _around_dim(x, dim)
    out = torch.empty_like(x)
    if x.numel():
        _call(x, "plh_taylor_softmax_forward", _ptr(x), tag, _ptr(out), n_size, dimsize, m_size, int(n),
              1 if use_log else 0)
    return _back_to(out, feat.dtype) if out.dtype != feat.dtype else out


def taylor_softmax_backward(grad_output, feat, dim, n, use_log):
    _require_gpu("taylor softmax function", feat, grad_output)
    _check_order(n)
    x, tag = _logits(feat)
    g = grad_output if grad_output.dtype == x.dtype else grad_output.to(x.dtype)
    g = g.expand(x.shape).contiguous()
    n_size, dimsize, m_size = _around_dim(x, dim)
    out = torch.empty_like(x)
    if x.numel():
        _call(x, "plh_taylor_softmax_backward", _ptr(g), _ptr(x), tag, _ptr(out), n_size, dimsize, m_size, int(n),
              1 if use_log else 0)
    return out if out.dtype == feat.dtype else out.to(feat.dtype)


def taylor_args(logits, labels):
    return seg_args(logits, labels, "taylor cross entropy", "taylor_ce")


def taylor_ce_forward(logits, labels, n, ignore_index, reduction, args=None):
    """-> (loss, n_valid or None). reduction 'mean' / 'sum' give a 0-dim loss, anything else per pixel."""
    _check_order(n)
    a = args or taylor_args(logits, labels)
    reduced = reduction in ("mean", "sum") and a.x.numel() > 0
    dev = a.x.device
    if reduced:
        loss = torch.empty((), dtype=torch.float32, device=dev)
        n_valid = torch.empty((), dtype=torch.int64, device=dev)
        ws, ws_bytes = _reduce_workspace(a.n * a.m, dev)
        _call(a.x, "plh_taylor_ce_forward", _ptr(a.x), a.tag, _ptr(a.lb), None, _ptr(loss), _ptr(n_valid),
              1 if reduction == "mean" else 0, _ptr(ws), ws_bytes, a.n, a.c, a.m, int(n), int(ignore_index))
        return _back_to(loss, _loss_dtype(a.dtype)), n_valid
    losses = torch.empty(a.lb.shape, dtype=torch.float32, device=dev)
    if a.x.numel():
        _call(a.x, "plh_taylor_ce_forward", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(losses), None, None, 0, None, 0,
              a.n, a.c, a.m, int(n), int(ignore_index))
    else:
        losses.zero_()
    return _back_to(losses, _loss_dtype(a.dtype)), None


def taylor_ce_forward_reduced_sums(logits, labels, n, ignore_index, mean, args=None):
    """The reduced forward that also leaves each row's sum of f for the backward, where the shape has a backward that
    uses it (long (N, C) rows, see plh_taylor_ce_saves_sums). -> (loss, n_valid, sums or None)."""
    _check_order(n)
    a = args or taylor_args(logits, labels)
    if a.x.numel() == 0 or not load().plh_taylor_ce_saves_sums(a.tag, a.n, a.c, a.m):
        loss, n_valid = taylor_ce_forward(logits, labels, n, ignore_index, "mean" if mean else "sum", args=a)
        return loss, n_valid, None
    dev = a.x.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    n_valid = torch.empty((), dtype=torch.int64, device=dev)
    sums = torch.empty((a.n * a.m,), dtype=torch.float32, device=dev)
    ws, ws_bytes = _reduce_workspace(a.n * a.m, dev)
    _call(a.x, "plh_taylor_ce_forward_reduced_sums", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(sums), _ptr(loss), _ptr(n_valid),
          1 if mean else 0, _ptr(ws), ws_bytes, a.n, a.c, a.m, int(n), int(ignore_index))
    return _back_to(loss, _loss_dtype(a.dtype)), n_valid, sums


def taylor_ce_backward_scaled_sums(sums, n, ignore_index, grad_scalar, divide_by, args):
    """The gradient from the forward's row sums (taylor_ce_forward_reduced_sums), for one scalar upstream gradient."""
    a = args
    grad = torch.empty_like(a.x)
    go = _scalar_f32(grad_scalar)
    _call(a.x, "plh_taylor_ce_backward_scaled_sums", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(sums), _ptr(go), 1.0,
          _ptr(divide_by), _ptr(grad), a.n, a.c, a.m, int(n), int(ignore_index))
    return _back_to(grad, a.dtype)


def taylor_ce_backward(logits, labels, n, ignore_index, grad_output, divide_by=None, args=None):
    a = args or taylor_args(logits, labels)
    grad = torch.empty_like(a.x)
    if a.x.numel() == 0:
        return _back_to(grad, a.dtype)
    if grad_output.numel() == 1:
        go, stride = _scalar_f32(grad_output), 0
    else:
        go, stride = _upstream(grad_output, a.lb.shape)
    _call(a.x, "plh_taylor_ce_backward", _ptr(a.x), a.tag, _ptr(a.lb), _ptr(go), stride, 1.0, _ptr(divide_by),
          _ptr(grad), a.n, a.c, a.m, int(n), int(ignore_index))
    return _back_to(grad, a.dtype)


# ------------------------------------------------------------ soft dice ----

def soft_dice_forward(logits, labels, p, smooth):
    """(N, L) logits and float labels -> (losses (N,), stats (N, 2) = numer, denor per row, marshalled inputs)."""
    if logits.shape != labels.shape or logits.dim() != 2:
        raise AssertionError("soft dice: logits and labels must both be (N, L)")     # soft_dice_loss.py:152
    a = focal_args(logits, labels, "soft_dice_forward")
    n, length = int(a.x.shape[0]), int(a.x.shape[1])
    losses = torch.empty((n,), dtype=torch.float32, device=a.x.device)
    stats = torch.empty((n, 2), dtype=torch.float32, device=a.x.device)
    if n:
        nbytes = int(load().plh_soft_dice_workspace_bytes(n, length))
        if nbytes < 0:
            _check(nbytes)
        ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=a.x.device)
        _call(a.x, "plh_soft_dice_forward", _ptr(a.x), a.tag, _ptr(a.y), _ptr(losses), _ptr(stats), _ptr(ws), nbytes,
              n, length, float(p), float(smooth))
    return _back_to(losses, _loss_dtype(a.dtype)), stats, a


def soft_dice_backward(grad_output, stats, p, args):
    a = args
    n, length = int(a.x.shape[0]), int(a.x.shape[1])
    grad = torch.empty_like(a.x)
    if a.x.numel():
        go = _f32c(grad_output.expand((n,)) if grad_output.numel() == 1 else grad_output.reshape(n))
        _call(a.x, "plh_soft_dice_backward", _ptr(go), _ptr(a.x), a.tag, _ptr(a.y), _ptr(stats), _ptr(grad), n, length,
              float(p))
    return _back_to(grad, a.dtype)


# -------------------------------------------------------------- one-hot ----

def onehot(labels, n_classes, smooth, ignore_index, check=True):
    """(N, *) int64 labels -> (N, n_classes, *) fp32 targets. check=True reads the two range flags
    back (one small device-to-host copy, as the reference's max/min test does) and raises."""
    _require_gpu("onehot method", labels)
    if labels.dtype != torch.int64:
        raise RuntimeError("label_one_hot: date type should be kLong")      # csrc/one_hot_kernel.cu:271
    lb = labels.contiguous()
    n_size = int(lb.shape[0]) if lb.dim() else 1
    m_size = lb.numel() // max(1, n_size)
    shape = (n_size, int(n_classes)) + tuple(lb.shape[1:])
    out = torch.empty(shape, dtype=torch.float32, device=lb.device)
    flags = torch.empty((2,), dtype=torch.int32, device=lb.device) if check else None
    _call(lb, "plh_onehot", _ptr(lb), _ptr(out), _ptr(flags), n_size, int(n_classes), m_size, int(ignore_index),
          float(smooth))
    if check:
        too_big, negative = flags.tolist()
        if too_big:
            raise RuntimeError("label should be less than min_len")           # csrc/one_hot_kernel.cu:301
        if negative:
            raise RuntimeError("label should be more than 0")                 # csrc/one_hot_kernel.cu:302
    return out


def stream_copy(src, dst):
    _require_gpu("stream copy", src, dst)
    assert src.dtype == torch.float32 and dst.dtype == torch.float32 and src.numel() == dst.numel()
    assert src.is_contiguous() and dst.is_contiguous()
    _call(src, "plh_stream_copy", _ptr(src), _ptr(dst), src.numel())


# ----------------------------------------------------------- layer norm ----

def layer_norm_forward(x, eps):
    """(N, C, M) normalised over C. -> (out, the contiguous input the backward reads, dtype tag)."""
    _require_gpu("layernorm loss", x)                                  # csrc/layer_norm.cu:380
    if x.dim() != 3:
        raise RuntimeError("layer norm: expected a (N, C, M) tensor, got %s" % (tuple(x.shape),))
    xc, tag = _logits(x)
    out = torch.empty_like(xc)
    if xc.numel():
        n, c, m = xc.shape
        _call(xc, "plh_layer_norm_forward", _ptr(xc), tag, _ptr(out), n, c, m, float(eps))
    return out.to(_loss_dtype(x.dtype)), xc, tag


def layer_norm_backward(grad_output, xc, tag, eps, dtype):
    g = grad_output if grad_output.dtype == xc.dtype else grad_output.to(xc.dtype)
    g = g.expand(xc.shape).contiguous()
    out = torch.empty_like(xc)
    if xc.numel():
        n, c, m = xc.shape
        _call(xc, "plh_layer_norm_backward", _ptr(g), _ptr(xc), tag, _ptr(out), n, c, m, float(eps))
    return out if out.dtype == dtype else out.to(dtype)
