"""Stands in for the extension built from csrc/ohem_label_kernel.cu (PYBIND11_MODULE at :279-281)."""
import torch

from ._abi import F32, I32, I64, P, bind, check, dims, gpu_only, native, stream
from ._abi import labels as int64_labels

_ws_bytes = bind("plh_ohem_workspace_bytes", [I64], I64)
_relabel = bind("plh_ohem_score_label", [P, I32, P, P, P, P, I64, I64, I64, I64, I64, F32, I64, P])


def score_ohem_label(logits, labels, ignore_index, score_thresh, n_min):
    """csrc/ohem_label_kernel.cu:267-277 -> new int64 labels: pixels whose probability at the label exceeds
    score_thresh and that are not among the n_min lowest are set to ignore_index; the inputs stay as they are."""
    gpu_only("ohem method", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    out = torch.empty_like(lb)
    if lb.numel() == 0:
        return out
    n, c, m = dims(x)
    nbytes = _ws_bytes(n * m)
    if nbytes < 0:
        check(int(nbytes))
    ws = torch.empty((max(int(nbytes), 1),), dtype=torch.uint8, device=x.device)
    scores = torch.empty((n * m,), dtype=torch.float32, device=x.device)
    with torch.cuda.device_of(x):
        check(_relabel(x.data_ptr(), tag, lb.data_ptr(), out.data_ptr(), scores.data_ptr(), ws.data_ptr(), int(nbytes),
                       n, c, m, ignore_index, score_thresh, n_min, stream()))
    return out
