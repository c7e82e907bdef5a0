"""Stands in for the extension built from csrc/lovasz_softmax.cu (PYBIND11_MODULE at :799-802).
Unlike the other three, the forward has a second output that the backward takes back (the Jaccard
differences in pixel order, `jacc` [C, P] fp32) and needs scratch memory, which the library asks
the caller for: plh_lovasz_workspace_bytes() bytes, allocated here through torch's caching allocator
(the reference allocates its own with thrust, :565)."""
import torch

from ._abi import I32, I64, P, bind, check, dims, gpu_only, native, stream
from ._abi import labels as int64_labels

_ws_bytes = bind("plh_lovasz_workspace_bytes", [I64, I64, I64], I64)
_fwd = bind("plh_lovasz_forward", [P, I32, P, P, P, P, I64, I64, I64, I64, I64, P])
_bwd = bind("plh_lovasz_backward", [P, P, I32, P, P, P, I64, I64, I64, I64, P])


def lovasz_softmax_forward(logits, labels, ignore_index):
    """-> (losses [C], jacc [C, P]), csrc/lovasz_softmax.cu:778-786."""
    gpu_only("lovasz softmax function", logits)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    n, c, m = dims(x)
    losses = torch.zeros(c, dtype=torch.float32, device=x.device)
    jacc = torch.zeros((c, n * m), dtype=torch.float32, device=x.device)
    if x.numel():
        need = _ws_bytes(n, c, m)
        if need < 0:
            check(int(need))
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, lb.data_ptr(), losses.data_ptr(), jacc.data_ptr(), ws.data_ptr(), need,
                       n, c, m, ignore_index, stream()))
    return losses.to(logits.dtype), jacc


def lovasz_softmax_backward(grad, logits, labels, jacc, ignore_index):
    """-> dloss/dlogits for the upstream gradient `grad` [C], csrc/lovasz_softmax.cu:788-797."""
    gpu_only("lovasz softmax function", logits, labels)
    (x, tag), lb = native(logits), int64_labels(labels, logits)
    out = torch.empty_like(x)
    go, dj = grad.float().contiguous(), jacc.float().contiguous()      # fp32 at the ABI
    if x.numel():
        with torch.cuda.device_of(x):
            check(_bwd(go.data_ptr(), x.data_ptr(), tag, lb.data_ptr(), dj.data_ptr(), out.data_ptr(), *dims(x),
                       ignore_index, stream()))
    return out.to(logits.dtype)
