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

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpytorch_loss_hip.so")
ABI_VERSION = 2

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
    "plh_lsr_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_focal_forward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _f32, _f32, _p]),
    "plh_focal_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _p, _i64, _f32, _f32, _p]),
    "plh_focal_forward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _i32, _p, _i64, _i64, _f32, _f32, _p]),
    "plh_focal_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _i64, _f32, _f32, _p]),
    "plh_focal_forward_backward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _i64, _f32, _f32, _p]),
    "plh_lmargin_forward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward": (ctypes.c_int, [_p, _i32, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_forward_reduced": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_backward_scaled": (ctypes.c_int, [_p, _i32, _p, _p, _f32, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lmargin_forward_backward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _f32, _p]),
    "plh_lovasz_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "plh_lovasz_forward": (ctypes.c_int, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "plh_lovasz_backward": (ctypes.c_int, [_p, _p, _i32, _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
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


def _stream():
    return _p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return _p(t.data_ptr()) if t is not None else _p(0)


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


def _loss_dtype(logits):
    """dtype of the returned losses: the logits' own, except under autocast, where the reference's
    custom_fwd(cast_inputs=float32) makes the whole op fp32."""
    return torch.float32 if torch.is_autocast_enabled("cuda") else logits.dtype


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

def _pixel_forward(entry, what, logits, labels, ignore_index, param):
    _require_gpu(what, logits, labels)
    n, c, m = _dims(logits, entry)
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, entry)
    losses = torch.empty(lb.shape, dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return _back_to(losses.zero_(), _loss_dtype(logits))
    with torch.cuda.device_of(x):
        _check(getattr(load(), entry)(_ptr(x), tag, _ptr(lb), _ptr(losses), n, c, m, int(ignore_index), float(param),
                                      _stream()))
    return _back_to(losses, _loss_dtype(logits))


def _pixel_backward(entry, what, logits, labels, ignore_index, param, grad_output):
    """dloss/dlogits, already multiplied by ``grad_output`` (None = unit upstream gradient)."""
    _require_gpu(what, logits, labels)
    n, c, m = _dims(logits, entry)
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, entry)
    grad = torch.empty_like(x)
    if x.numel() == 0:
        return _back_to(grad, logits.dtype)
    go, stride = _upstream(grad_output, lb.shape)
    with torch.cuda.device_of(x):
        _check(getattr(load(), entry)(_ptr(x), tag, _ptr(lb), _ptr(go), stride, _ptr(grad), n, c, m,
                                      int(ignore_index), float(param), _stream()))
    return _back_to(grad, logits.dtype)


def _reduce_workspace(units, device):
    nbytes = int(load().plh_reduce_workspace_bytes(int(units)))
    if nbytes < 0:
        _check(nbytes)
    return torch.empty((nbytes,), dtype=torch.uint8, device=device), nbytes


def _scalar_f32(t):
    """A 0-dim upstream gradient as one fp32 value in device memory."""
    t = t.reshape(-1)[:1]
    return t if (t.dtype == torch.float32 and t.is_contiguous()) else t.float().contiguous()


def _pixel_forward_reduced(entry, what, logits, labels, ignore_index, param, mean):
    """-> (loss 0-dim, n_valid 0-dim int64)."""
    _require_gpu(what, logits, labels)
    n, c, m = _dims(logits, entry)
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, entry)
    loss = torch.empty((), dtype=torch.float32, device=x.device)
    n_valid = torch.empty((), dtype=torch.int64, device=x.device)
    ws, ws_bytes = _reduce_workspace(n * m, x.device)
    with torch.cuda.device_of(x):
        _check(getattr(load(), entry)(_ptr(x), tag, _ptr(lb), None, _ptr(loss), _ptr(n_valid), 1 if mean else 0,
                                      _ptr(ws), ws_bytes, n, c, m, int(ignore_index), float(param), _stream()))
    return _back_to(loss, _loss_dtype(logits)), n_valid


def _pixel_backward_scaled(entry, what, logits, labels, ignore_index, param, grad_scalar, divide_by):
    _require_gpu(what, logits, labels)
    n, c, m = _dims(logits, entry)
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, entry)
    grad = torch.empty_like(x)
    if x.numel() == 0:
        return _back_to(grad, logits.dtype)
    go = _scalar_f32(grad_scalar)
    with torch.cuda.device_of(x):
        _check(getattr(load(), entry)(_ptr(x), tag, _ptr(lb), _ptr(go), 1.0, _ptr(divide_by), _ptr(grad), n, c, m,
                                      int(ignore_index), float(param), _stream()))
    return _back_to(grad, logits.dtype)


def lsr_forward(logits, labels, ignore_index, smooth):
    return _pixel_forward("plh_lsr_forward", "LSR loss", logits, labels, ignore_index, smooth)


def lsr_backward(logits, labels, ignore_index, smooth, grad_output=None):
    return _pixel_backward("plh_lsr_backward", "LSR loss", logits, labels, ignore_index, smooth, grad_output)


def lsr_forward_reduced(logits, labels, ignore_index, smooth, mean):
    return _pixel_forward_reduced("plh_lsr_forward_reduced", "LSR loss", logits, labels, ignore_index, smooth, mean)


def lsr_backward_scaled(logits, labels, ignore_index, smooth, grad_scalar, divide_by=None):
    return _pixel_backward_scaled("plh_lsr_backward_scaled", "LSR loss", logits, labels, ignore_index, smooth,
                                  grad_scalar, divide_by)


# -------------------------------------------------------------- lmargin ----

def lmargin_forward(logits, labels, lam, ignore_index):
    return _pixel_forward("plh_lmargin_forward", "large margin loss", logits, labels, ignore_index, lam)


def lmargin_backward(logits, labels, lam, ignore_index, grad_output=None):
    return _pixel_backward("plh_lmargin_backward", "large margin loss", logits, labels, ignore_index, lam,
                           grad_output)


def lmargin_forward_reduced(logits, labels, lam, ignore_index, mean):
    return _pixel_forward_reduced("plh_lmargin_forward_reduced", "large margin loss", logits, labels, ignore_index,
                                  lam, mean)


def lmargin_backward_scaled(logits, labels, lam, ignore_index, grad_scalar, divide_by=None):
    return _pixel_backward_scaled("plh_lmargin_backward_scaled", "large margin loss", logits, labels, ignore_index,
                                  lam, grad_scalar, divide_by)


def lmargin_forward_backward(logits, labels, lam, ignore_index):
    """-> (losses, grad under unit upstream gradient, valid_cnt int64[1])"""
    _require_gpu("large margin loss", logits, labels)
    n, c, m = _dims(logits, "l_margin_forward_backward")
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, "l_margin_forward_backward")
    losses = torch.empty(lb.shape, dtype=torch.float32, device=x.device)
    grad = torch.empty_like(x)
    cnt = torch.zeros(1, dtype=torch.int64, device=x.device)
    if x.numel():
        with torch.cuda.device_of(x):
            _check(load().plh_lmargin_forward_backward(_ptr(x), tag, _ptr(lb), _ptr(losses), _ptr(grad), _ptr(cnt),
                                                       n, c, m, int(ignore_index), float(lam), _stream()))
    else:
        losses.zero_()
    return _back_to(losses, _loss_dtype(logits)), _back_to(grad, logits.dtype), cnt


# ---------------------------------------------------------------- focal ----

def _focal_pair(logits, labels, what):
    """Logits and labels in one dtype the kernels read; mixed or exotic dtypes are computed from fp32 copies."""
    _require_gpu("focal loss", logits, labels)
    if tuple(labels.shape) != tuple(logits.shape):
        raise RuntimeError("%s: labels and logits must have the same shape" % what)
    if logits.dtype == labels.dtype and logits.dtype in _DTYPE_TAGS:
        return logits.contiguous(), labels.contiguous(), _DTYPE_TAGS[logits.dtype]
    return _f32c(logits), _f32c(labels), 0


def focal_forward(logits, labels, gamma, alpha):
    x, y, tag = _focal_pair(logits, labels, "focalloss_forward")
    losses = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    if x.numel():
        with torch.cuda.device_of(x):
            _check(load().plh_focal_forward(_ptr(x), tag, _ptr(y), _ptr(losses), x.numel(),
                                            float(gamma), float(alpha), _stream()))
    return _back_to(losses, _loss_dtype(logits))


def focal_backward(logits, labels, gamma, alpha, grad_output=None):
    x, y, tag = _focal_pair(logits, labels, "focalloss_backward")
    grad = torch.empty_like(x)
    if x.numel():
        go, stride = _upstream(grad_output, x.shape)
        with torch.cuda.device_of(x):
            _check(load().plh_focal_backward(_ptr(x), tag, _ptr(y), _ptr(go), stride, _ptr(grad), x.numel(),
                                             float(gamma), float(alpha), _stream()))
    return _back_to(grad, logits.dtype)


def focal_forward_backward(logits, labels, gamma, alpha):
    x, y, tag = _focal_pair(logits, labels, "focalloss_forward_backward")
    losses = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    grad = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device_of(x):
            _check(load().plh_focal_forward_backward(_ptr(x), tag, _ptr(y), _ptr(losses), _ptr(grad), x.numel(),
                                                     float(gamma), float(alpha), _stream()))
    return _back_to(losses, _loss_dtype(logits)), _back_to(grad, logits.dtype)


def focal_forward_reduced(logits, labels, gamma, alpha, mean):
    x, y, tag = _focal_pair(logits, labels, "focalloss_forward")
    loss = torch.empty((), dtype=torch.float32, device=x.device)
    ws, ws_bytes = _reduce_workspace(x.numel(), x.device)
    with torch.cuda.device_of(x):
        _check(load().plh_focal_forward_reduced(_ptr(x), tag, _ptr(y), None, _ptr(loss), 1 if mean else 0, _ptr(ws),
                                                ws_bytes, x.numel(), float(gamma), float(alpha), _stream()))
    return _back_to(loss, _loss_dtype(logits))


def focal_backward_scaled(logits, labels, gamma, alpha, grad_scalar, scale):
    x, y, tag = _focal_pair(logits, labels, "focalloss_backward")
    grad = torch.empty_like(x)
    if x.numel():
        go = _scalar_f32(grad_scalar)
        with torch.cuda.device_of(x):
            _check(load().plh_focal_backward_scaled(_ptr(x), tag, _ptr(y), _ptr(go), float(scale), _ptr(grad),
                                                    x.numel(), float(gamma), float(alpha), _stream()))
    return _back_to(grad, logits.dtype)


# --------------------------------------------------------------- lovasz ----

def _lovasz_limits(logits, what):
    # same limits and wording as csrc/lovasz_softmax.cu:664-665
    if logits.numel() >= (1 << 31):
        raise RuntimeError("%s: input tensor too large, int32 type will overflow" % what)
    if logits.dim() >= 2 and logits.shape[1] >= 512:
        raise RuntimeError("%s: num of classes should be less than BLOCKSIZE" % what)


def lovasz_forward(logits, labels, ignore_index):
    """-> (losses[C], jacc[C, N*M] fp32)"""
    _require_gpu("lovasz softmax function", logits, labels)
    _lovasz_limits(logits, "lovasz_softmax_forward")
    n, c, m = _dims(logits, "lovasz_softmax_forward")
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, "lovasz_softmax_forward")
    losses = torch.empty((c,), dtype=torch.float32, device=x.device)
    jacc = torch.empty((c, n * m), dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return _back_to(losses.zero_(), _loss_dtype(logits)), jacc
    lib = load()
    ws_bytes = int(lib.plh_lovasz_workspace_bytes(n, c, m))
    if ws_bytes < 0:
        _check(ws_bytes)
    workspace = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    with torch.cuda.device_of(x):
        _check(lib.plh_lovasz_forward(_ptr(x), tag, _ptr(lb), _ptr(losses), _ptr(jacc), _ptr(workspace), ws_bytes,
                                      n, c, m, int(ignore_index), _stream()))
    return _back_to(losses, _loss_dtype(logits)), jacc


def lovasz_backward(grad_output, logits, labels, jacc, ignore_index):
    _require_gpu("lovasz softmax function", logits, labels, grad_output, jacc)
    n, c, m = _dims(logits, "lovasz_softmax_backward")
    x, tag = _logits(logits)
    lb = _labels_i64(labels, logits, "lovasz_softmax_backward")
    grad = torch.empty_like(x)
    if x.numel() == 0:
        return _back_to(grad, logits.dtype)
    go = _f32c(grad_output.expand((c,)) if grad_output.numel() == 1 else grad_output)
    if go.numel() != c or jacc.numel() != c * n * m or jacc.dtype != torch.float32:
        raise RuntimeError("lovasz_softmax_backward: grad_output must have C elements and jacc C*N*M fp32 elements")
    jc = jacc.contiguous()
    with torch.cuda.device_of(x):
        _check(load().plh_lovasz_backward(_ptr(go), _ptr(x), tag, _ptr(lb), _ptr(jc), _ptr(grad), n, c, m,
                                          int(ignore_index), _stream()))
    return _back_to(grad, logits.dtype)


def stream_copy(src, dst):
    _require_gpu("stream copy", src, dst)
    assert src.dtype == torch.float32 and dst.dtype == torch.float32 and src.numel() == dst.numel()
    assert src.is_contiguous() and dst.is_contiguous()
    with torch.cuda.device_of(src):
        _check(load().plh_stream_copy(_ptr(src), _ptr(dst), src.numel(), _stream()))
