"""Stand-ins for the reference's pybind11 extension modules of the fused-loss path and the ops next to
it, bound to libpytorch_loss_hip.so.

The reference's Python files import one CUDA extension per op at module level (`import lsr_cpp`,
pytorch_loss/label_smooth.py:125; `focal_cpp`, `large_margin_cpp`, `lovasz_softmax_cpp`, `ohem_cpp`,
`one_hot_cpp`, `taylor_softmax_cpp`, `soft_dice_cpp`, `layer_norm_cpp` likewise; setup.py:13-45 names them).
Each module here carries the same function names with the same positional arguments and return
values as the extension it replaces, so those files run unchanged once `install()` has put the
stand-ins into `sys.modules` (or this directory is on `sys.path` ahead of the built extensions):

    import ext_stubs; ext_stubs.install()
    import lsr_cpp                      # -> ext_stubs.lsr_cpp
    losses = lsr_cpp.lsr_forward(logits, labels, 255, 0.1)

They are plain ctypes over the C ABI of include/pytorch_loss_hip.h and use nothing of the
`pytorch_loss` package in this tree.
"""
import importlib
import sys

NAMES = ("lsr_cpp", "focal_cpp", "large_margin_cpp", "lovasz_softmax_cpp",
         "ohem_cpp", "one_hot_cpp", "taylor_softmax_cpp", "soft_dice_cpp", "layer_norm_cpp")


def install():
    """Register the stand-ins under the reference's extension module names."""
    mods = {}
    for name in NAMES:
        mods[name] = sys.modules[name] = importlib.import_module(__name__ + "." + name)
    return mods
