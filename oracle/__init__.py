"""CPU oracle for the fused-loss path -- TEST INFRASTRUCTURE ONLY.

ctypes front end over ``liboracle.so`` (built from ``plo_oracle.c`` by
``oracle/build.py``).  Nothing in the shipped package may import this module;
it is the checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.

All functions take and return numpy arrays.  The arithmetic type follows the
dtype of ``logits`` (float32 -> the ``_f32`` restatement, float64 -> ``_f64``).
Shapes follow the reference: logits ``(N, C, *)``, integer labels ``(N, *)``
(csrc/lsr_kernel.cu:199-202 flattens to n_size, dimsize, m_size the same way).
"""
import ctypes
import os

import numpy as np

from . import build as _build

_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        path = _build.LIB
        if not os.path.exists(path):
            path = _build.build()
        _LIB = ctypes.CDLL(path)
        assert _LIB.oracle_abi_version() == 1
    return _LIB


def _suffix(a):
    if a.dtype == np.float32:
        return "_f32", ctypes.c_float
    if a.dtype == np.float64:
        return "_f64", ctypes.c_double
    raise TypeError("oracle works on float32 or float64 logits, got %s" % a.dtype)


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _dims(logits):
    n_size = int(logits.shape[0])
    dimsize = int(logits.shape[1])
    m_size = int(logits.size // max(1, n_size * dimsize)) if logits.size else 0
    return n_size, dimsize, m_size


def _prep(logits, labels):
    logits = np.ascontiguousarray(logits)
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    assert labels.shape == logits.shape[:1] + logits.shape[2:], (labels.shape, logits.shape)
    return logits, labels


def _call(name, *args):
    fn = getattr(lib(), name)
    fn.restype = ctypes.c_int
    return fn(*args)


i64 = ctypes.c_int64
f64 = ctypes.c_double


def lsr_forward(logits, labels, ignore_index=-100, smooth=0.1):
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    out = np.zeros(labels.shape, dtype=logits.dtype)
    if logits.size:
        _call("oracle_lsr_forward" + sfx, _ptr(logits), _ptr(labels), _ptr(out),
              i64(n), i64(c), i64(m), i64(ignore_index), f64(smooth))
    return out


def lsr_backward(logits, labels, ignore_index=-100, smooth=0.1, grad_out=None):
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    if grad_out is not None:
        grad_out = np.ascontiguousarray(np.broadcast_to(grad_out, labels.shape), dtype=logits.dtype)
    out = np.zeros_like(logits)
    if logits.size:
        _call("oracle_lsr_backward" + sfx, _ptr(logits), _ptr(labels), _ptr(grad_out), _ptr(out),
              i64(n), i64(c), i64(m), i64(ignore_index), f64(smooth))
    return out


def focal_forward(logits, labels, alpha=0.25, gamma=2.0):
    logits = np.ascontiguousarray(logits)
    labels = np.ascontiguousarray(labels, dtype=logits.dtype)
    assert labels.shape == logits.shape
    sfx, _ = _suffix(logits)
    out = np.zeros_like(logits)
    if logits.size:
        _call("oracle_focal_forward" + sfx, _ptr(logits), _ptr(labels), _ptr(out),
              i64(logits.size), f64(alpha), f64(gamma))
    return out


def focal_backward(logits, labels, alpha=0.25, gamma=2.0, grad_out=None):
    logits = np.ascontiguousarray(logits)
    labels = np.ascontiguousarray(labels, dtype=logits.dtype)
    sfx, _ = _suffix(logits)
    if grad_out is not None:
        grad_out = np.ascontiguousarray(np.broadcast_to(grad_out, logits.shape), dtype=logits.dtype)
    out = np.zeros_like(logits)
    if logits.size:
        _call("oracle_focal_backward" + sfx, _ptr(logits), _ptr(labels), _ptr(grad_out), _ptr(out),
              i64(logits.size), f64(alpha), f64(gamma))
    return out


def lmargin_forward(logits, labels, lam=0.3, ignore_index=255):
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    out = np.zeros(labels.shape, dtype=logits.dtype)
    if logits.size:
        _call("oracle_lmargin_forward" + sfx, _ptr(logits), _ptr(labels), _ptr(out),
              i64(n), i64(c), i64(m), i64(ignore_index), f64(lam))
    return out


def lmargin_backward(logits, labels, lam=0.3, ignore_index=255, grad_out=None):
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    if grad_out is not None:
        grad_out = np.ascontiguousarray(np.broadcast_to(grad_out, labels.shape), dtype=logits.dtype)
    out = np.zeros_like(logits)
    if logits.size:
        _call("oracle_lmargin_backward" + sfx, _ptr(logits), _ptr(labels), _ptr(grad_out), _ptr(out),
              i64(n), i64(c), i64(m), i64(ignore_index), f64(lam))
    return out


def lovasz_forward(logits, labels, ignore_index=-100):
    """-> (losses[C], jacc[C, P]); jacc holds the Jaccard differences in pixel order."""
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    assert c < 512
    losses = np.zeros((c,), dtype=logits.dtype)
    jacc = np.zeros((c, n * m), dtype=logits.dtype)
    if logits.size:
        rc = _call("oracle_lovasz_forward" + sfx, _ptr(logits), _ptr(labels), _ptr(losses), _ptr(jacc),
                   i64(n), i64(c), i64(m), i64(ignore_index))
        if rc != 0:
            raise MemoryError("oracle_lovasz_forward ran out of memory")
    return losses, jacc


def lovasz_backward(grad_out, logits, labels, jacc, ignore_index=-100):
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    grad_out = np.ascontiguousarray(np.broadcast_to(grad_out, (c,)), dtype=logits.dtype)
    jacc = np.ascontiguousarray(jacc, dtype=logits.dtype)
    out = np.zeros_like(logits)
    if logits.size:
        _call("oracle_lovasz_backward" + sfx, _ptr(grad_out), _ptr(logits), _ptr(labels), _ptr(jacc),
              _ptr(out), i64(n), i64(c), i64(m), i64(ignore_index))
    return out


def ohem_scores(logits, labels, ignore_index=255):
    """Softmax probability at the label, 1 for ignored pixels (csrc/ohem_label_kernel.cu:112-151)."""
    logits, labels = _prep(logits, labels)
    sfx, _ = _suffix(logits)
    n, c, m = _dims(logits)
    out = np.ones(labels.shape, dtype=logits.dtype)
    if logits.size:
        _call("oracle_ohem_scores" + sfx, _ptr(logits), _ptr(labels), _ptr(out), i64(n), i64(c), i64(m),
              i64(ignore_index))
    return out


def ohem_select(scores, labels, ignore_index, score_thresh, n_min):
    """Labels with every pixel beyond the n_min lowest scores whose score exceeds the threshold set to
    ignore_index (csrc/ohem_label_kernel.cu:155-168, 247-262)."""
    scores = np.ascontiguousarray(scores)
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    assert scores.shape == labels.shape
    sfx, _ = _suffix(scores)
    out = np.empty_like(labels)
    rc = _call("oracle_ohem_select" + sfx, _ptr(scores), _ptr(labels), _ptr(out), i64(labels.size),
               i64(ignore_index), f64(score_thresh), i64(n_min))
    if rc != 0:
        raise MemoryError("oracle_ohem_select ran out of memory")
    return out


def ohem_score_label(logits, labels, ignore_index, score_thresh, n_min):
    """ohem_cpp.score_ohem_label (csrc/ohem_label_kernel.cu:171-263)."""
    return ohem_select(ohem_scores(logits, labels, ignore_index), labels, ignore_index, score_thresh, n_min)


def onehot(labels, n_classes, smooth=0.0, ignore_index=-1, dtype=np.float32):
    """(N, *) int labels -> (N, n_classes, *) targets: 1 - smooth at the label, smooth / n_classes
    elsewhere, all zeros at ignored pixels (csrc/one_hot_kernel.cu:231-261, 305-306)."""
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    n = int(labels.shape[0]) if labels.ndim else 1
    m = int(labels.size // max(1, n))
    out = np.zeros((n, n_classes) + tuple(labels.shape[1:]), dtype=dtype)
    if labels.size:
        _call("oracle_onehot" + ("_f32" if dtype == np.float32 else "_f64"), _ptr(labels), _ptr(out), i64(n),
              i64(n_classes), i64(m), i64(ignore_index), f64(smooth))
    return out


def _around(a, dim):
    dim = dim % a.ndim
    n = int(np.prod(a.shape[:dim], dtype=np.int64))
    m = int(np.prod(a.shape[dim + 1:], dtype=np.int64))
    return n, int(a.shape[dim]), m


def taylor_forward(feat, dim=1, order=2, use_log=False):
    """Taylor softmax of even `order` along `dim` (csrc/taylor_softmax.cu:50-86)."""
    feat = np.ascontiguousarray(feat)
    sfx, _ = _suffix(feat)
    n, d, m = _around(feat, dim)
    out = np.empty_like(feat)
    if feat.size:
        _call("oracle_taylor_forward" + sfx, _ptr(feat), _ptr(out), i64(n), i64(d), i64(m), i64(order),
              ctypes.c_int(1 if use_log else 0))
    return out


def taylor_backward(grad, feat, dim=1, order=2, use_log=False):
    feat = np.ascontiguousarray(feat)
    grad = np.ascontiguousarray(grad, dtype=feat.dtype)
    sfx, _ = _suffix(feat)
    n, d, m = _around(feat, dim)
    out = np.empty_like(feat)
    if feat.size:
        _call("oracle_taylor_backward" + sfx, _ptr(grad), _ptr(feat), _ptr(out), i64(n), i64(d), i64(m), i64(order),
              ctypes.c_int(1 if use_log else 0))
    return out


def taylor_ce(logits, labels, order=2, ignore_index=-1):
    """Per-pixel -log_taylor_softmax(logits)[label], 0 at ignored pixels: what F.nll_loss(reduction=
    'none') makes of the log form (pytorch_loss/taylor_softmax.py:175-198)."""
    logits, labels = _prep(logits, labels)
    logp = taylor_forward(logits, 1, order, True)
    safe = np.where(labels == ignore_index, 0, labels)
    picked = np.take_along_axis(logp, np.expand_dims(safe, 1), 1).squeeze(1)
    return np.where(labels == ignore_index, 0, -picked).astype(logits.dtype)


def taylor_ce_backward(logits, labels, order, ignore_index, grad_out):
    """Gradient of taylor_ce under the per-pixel upstream gradient `grad_out`."""
    logits, labels = _prep(logits, labels)
    g = np.zeros_like(logits)
    go = np.broadcast_to(np.asarray(grad_out, dtype=logits.dtype), labels.shape)
    safe = np.where(labels == ignore_index, 0, labels)
    np.put_along_axis(g, np.expand_dims(safe, 1), np.expand_dims(np.where(labels == ignore_index, 0, -go), 1), 1)
    return taylor_backward(g, logits, 1, order, True)


def soft_dice_forward(logits, labels, p=1.0, smooth=1.0):
    """(N, L) -> (losses (N,), stats (N, 2) = numer, denor) (pytorch_loss/soft_dice_loss.py:72-93)."""
    logits = np.ascontiguousarray(logits)
    labels = np.ascontiguousarray(labels, dtype=logits.dtype)
    assert logits.ndim == 2 and logits.shape == labels.shape
    sfx, _ = _suffix(logits)
    n, length = logits.shape
    losses = np.zeros((n,), dtype=logits.dtype)
    stats = np.zeros((n, 2), dtype=logits.dtype)
    _call("oracle_soft_dice_forward" + sfx, _ptr(logits), _ptr(labels), _ptr(losses), _ptr(stats), i64(n), i64(length),
          f64(p), f64(smooth))
    return losses, stats


def soft_dice_backward(grad_out, logits, labels, stats, p=1.0):
    logits = np.ascontiguousarray(logits)
    labels = np.ascontiguousarray(labels, dtype=logits.dtype)
    sfx, _ = _suffix(logits)
    n, length = logits.shape
    grad_out = np.ascontiguousarray(np.broadcast_to(grad_out, (n,)), dtype=logits.dtype)
    stats = np.ascontiguousarray(stats, dtype=logits.dtype)
    out = np.zeros_like(logits)
    _call("oracle_soft_dice_backward" + sfx, _ptr(grad_out), _ptr(logits), _ptr(labels), _ptr(stats), _ptr(out),
          i64(n), i64(length), f64(p))
    return out


def layer_norm_forward(x, eps=1e-6):
    """(N, C, M) normalised over C (csrc/layer_norm.cu:102-129)."""
    x = np.ascontiguousarray(x)
    assert x.ndim == 3
    sfx, _ = _suffix(x)
    out = np.zeros_like(x)
    _call("oracle_layer_norm_forward" + sfx, _ptr(x), _ptr(out), i64(x.shape[0]), i64(x.shape[1]), i64(x.shape[2]),
          f64(eps))
    return out


def layer_norm_backward(grad, x, eps=1e-6):
    """What the reference's backward kernel returns (csrc/layer_norm.cu:200-216); see oracle_body.inc."""
    x = np.ascontiguousarray(x)
    grad = np.ascontiguousarray(grad, dtype=x.dtype)
    assert x.ndim == 3 and grad.shape == x.shape
    sfx, _ = _suffix(x)
    out = np.zeros_like(x)
    _call("oracle_layer_norm_backward" + sfx, _ptr(grad), _ptr(x), _ptr(out), i64(x.shape[0]), i64(x.shape[1]),
          i64(x.shape[2]), f64(eps))
    return out


# ---- module-level reductions (label_smooth.py:162-171, focal_loss.py(root):195-200,
# large_margin_softmax.py(root):221-229, lovasz_softmax.py:110-116) ----------------

def reduce_pixels(losses, labels, reduction, ignore_index):
    """'mean' divides by the count of non-ignored pixels; anything but 'mean'/'sum' is a pass-through."""
    if reduction == "sum":
        return losses.sum(dtype=losses.dtype)
    if reduction == "mean":
        n_valid = (np.asarray(labels) != ignore_index).sum()
        with np.errstate(invalid="ignore", divide="ignore"):
            return losses.sum(dtype=losses.dtype) / losses.dtype.type(n_valid)
    return losses


def reduce_all(losses, reduction):
    if reduction == "sum":
        return losses.sum(dtype=losses.dtype)
    if reduction == "mean":
        return losses.mean(dtype=losses.dtype)
    return losses
