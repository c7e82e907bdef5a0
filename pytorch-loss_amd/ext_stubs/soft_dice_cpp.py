"""Stands in for the extension built from csrc/soft_dice_kernel_v2.cu (PYBIND11_MODULE at :434-437)."""
import torch

from ._abi import F32, I32, I64, P, bind, check, gpu_only, native, stream

_ws_bytes = bind("plh_soft_dice_workspace_bytes", [I64, I64], I64)
_fwd = bind("plh_soft_dice_forward", [P, I32, P, P, P, P, I64, I64, I64, F32, F32, P])
_bwd = bind("plh_soft_dice_backward", [P, P, I32, P, P, P, I64, I64, F32, P])


def _forward(logits, labels, p, smooth):
    x, tag = native(logits)
    y = labels.to(x.dtype).contiguous()
    n = x.shape[0]
    length = x.numel() // max(1, n)
    losses = torch.empty((n,), dtype=torch.float32, device=x.device)
    stats = torch.empty((n, 2), dtype=torch.float32, device=x.device)      # numer, denor per row
    if n:
        nbytes = _ws_bytes(n, length)
        if nbytes < 0:
            check(int(nbytes))
        ws = torch.empty((max(int(nbytes), 1),), dtype=torch.uint8, device=x.device)
        with torch.cuda.device_of(x):
            check(_fwd(x.data_ptr(), tag, y.data_ptr(), losses.data_ptr(), stats.data_ptr(), ws.data_ptr(), int(nbytes),
                       n, length, p, smooth, stream()))
    return x, tag, y, losses, stats


def soft_dice_forward(logits, labels, p, smooth):
    """csrc/soft_dice_kernel_v2.cu:411-420 -> loss per row of the (N, L) inputs, dtype of logits."""
    gpu_only("dice loss", logits, labels)
    return _forward(logits, labels, p, smooth)[3].to(logits.dtype)


def soft_dice_backward(grad, logits, labels, p, smooth):
    """csrc/soft_dice_kernel_v2.cu:422-432 -> gradient with respect to logits. Like the reference's, this call
    forms the rows' numerators and denominators again (the C ABI takes them from the forward call)."""
    gpu_only("dice loss", logits, labels)
    x, tag, y, _, stats = _forward(logits, labels, p, smooth)
    n = x.shape[0]
    out = torch.empty_like(x)
    if x.numel():
        go = grad.float().reshape(-1).expand((n,)).contiguous()
        with torch.cuda.device_of(x):
            check(_bwd(go.data_ptr(), x.data_ptr(), tag, y.data_ptr(), stats.data_ptr(), out.data_ptr(), n,
                       x.numel() // n, p, stream()))
    return out.to(logits.dtype)
