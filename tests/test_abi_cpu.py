"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares with the arity the binding assumes, rejects bad arguments before launching anything,
and the Python surface mirrors the reference's error behaviour.  No kernel runs here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pytorch_loss_hip.h")


def declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char \*)\s*(plh_\w+)\s*\(([^;{]*)\)\s*;", text):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return out


@pytest.fixture(scope="module")
def native():
    from pytorch_loss import _native
    return _native


def test_library_exports_every_declared_symbol(native):
    lib = native.load()
    decl = declared()
    assert len(decl) >= 20
    for name, n_args in decl.items():
        assert hasattr(lib, name), name
        assert name in native._SIGNATURES, "binding lacks " + name
        assert len(native._SIGNATURES[name][1]) == n_args, name
    assert set(native._SIGNATURES) == set(decl)
    assert lib.plh_abi_version() == native.ABI_VERSION == 5


def test_error_strings(native):
    lib = native.load()
    assert lib.plh_error_string(0) == b"ok"
    for code in range(-7, 0):
        assert len(lib.plh_error_string(code)) > 5
    assert b"512" in lib.plh_error_string(-4)
    assert lib.plh_error_string(-99) == b"unknown error code"


def test_arguments_are_rejected_before_any_launch(native):
    lib = native.load()
    buf = (ctypes.c_float * 64)()
    lab = (ctypes.c_int64 * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    lp = ctypes.cast(lab, ctypes.c_void_p)
    odd = ctypes.c_void_p(p.value + 2)
    # zero-sized problems are fine and launch nothing
    assert lib.plh_lsr_forward(None, 0, None, None, 0, 19, 16, 255, 0.1, None) == 0
    assert lib.plh_focal_forward(None, 1, None, None, 0, 2.0, 0.25, None) == 0
    assert lib.plh_lovasz_forward(None, 2, None, None, None, None, 0, 0, 19, 16, 255, None) == 0
    assert lib.plh_stream_copy(None, None, 0, None) == 0
    # NULL / negative / misaligned / stride / class-count / workspace
    assert lib.plh_lsr_forward(None, 0, lp, p, 1, 2, 2, 255, 0.1, None) == -1
    assert lib.plh_lsr_forward(p, 0, lp, p, -1, 2, 2, 255, 0.1, None) == -2
    assert lib.plh_lsr_forward(odd, 0, lp, p, 1, 2, 2, 255, 0.1, None) == -6
    assert lib.plh_lsr_backward(p, 0, lp, p, 2, p, 1, 2, 2, 255, 0.1, None) == -3
    assert lib.plh_lmargin_backward(p, 0, lp, p, 7, p, 1, 2, 2, 255, 0.3, None) == -3
    assert lib.plh_focal_backward(p, 0, p, p, 3, p, 4, 2.0, 0.25, None) == -3
    assert lib.plh_focal_forward(p, 0, None, p, 4, 2.0, 0.25, None) == -1
    assert lib.plh_lovasz_forward(p, 0, lp, p, p, p, 1 << 20, 1, 512, 2, 255, None) == -4
    assert lib.plh_lovasz_workspace_bytes(1, 512, 4) == -4
    assert lib.plh_lovasz_workspace_bytes(1 << 20, 19, 1 << 12) == -2       # numel >= 2^31
    need = lib.plh_lovasz_workspace_bytes(2, 19, 64)
    assert need > 3 * 4 * 2 * 19 * 64
    assert lib.plh_lovasz_forward(p, 0, lp, p, p, None, need, 2, 19, 64, 255, None) == -5
    assert lib.plh_lsr_forward_reduced(p, 0, lp, None, p, None, 1, None, 0, 1, 2, 2, 255, 0.1, None) == -5
    # element type tags other than fp32 / fp16 / bf16, on every op and before anything else is looked at
    for bad in (-1, 3, 7):
        assert lib.plh_lsr_forward(p, bad, lp, p, 1, 2, 2, 255, 0.1, None) == -7
        assert lib.plh_lsr_backward(p, bad, lp, None, 0, p, 1, 2, 2, 255, 0.1, None) == -7
        assert lib.plh_lmargin_forward(p, bad, lp, p, 1, 2, 2, 255, 0.3, None) == -7
        assert lib.plh_lmargin_forward_backward(p, bad, lp, p, p, p, 1, 2, 2, 255, 0.3, None) == -7
        assert lib.plh_focal_forward(p, bad, p, p, 4, 2.0, 0.25, None) == -7
        assert lib.plh_focal_forward_backward(p, bad, p, p, p, 4, 2.0, 0.25, None) == -7
        assert lib.plh_lovasz_forward(p, bad, lp, p, p, p, need, 2, 19, 64, 255, None) == -7
        assert lib.plh_lovasz_backward(p, p, bad, lp, p, p, 2, 19, 64, 255, None) == -7
    # the forward that keeps the log-sum-exp and the backward that uses it: where they apply, and refusals elsewhere
    assert lib.plh_lsr_saves_lse(0, 16, 19, 769 * 769) == 1 and lib.plh_lsr_saves_lse(0, 32, 24, 513 * 513) == 1
    assert lib.plh_lsr_saves_lse(0, 8, 19, 1024 * 1024) == 0 and lib.plh_lsr_saves_lse(0, 8, 25, 769 * 769) == 0
    assert lib.plh_lsr_saves_lse(1, 16, 19, 769 * 769) == 0 and lib.plh_lsr_saves_lse(2, 16, 19, 769 * 769) == 0
    assert lib.plh_lsr_saves_lse(0, 8, 19, 1022 * 1022) == 1           # even, but planes off the 128-byte lines
    assert lib.plh_lsr_saves_lse(0, 8, 150, 513 * 513) == 1 and lib.plh_lsr_saves_lse(0, 8, 150, 512 * 512) == 0
    assert lib.plh_lsr_saves_lse(0, 4, 600, 256 * 256) == 1 and lib.plh_lsr_saves_lse(2, 4, 600, 256 * 256) == 0
    assert lib.plh_lsr_saves_lse(0, 8, 300, 256 * 256) == 1 and lib.plh_lsr_saves_lse(0, 8, 256, 256 * 256) == 0
    assert lib.plh_lsr_saves_lse(2, 8192, 32000, 1) == 1 and lib.plh_lsr_saves_lse(0, 8192, 4096, 1) == 0 and lib.plh_lsr_saves_lse(2, 8192, 4096, 1) == 1     # rows
    assert lib.plh_lsr_saves_lse(0, 8192, 512, 1) == 0 and lib.plh_lsr_saves_lse(0, 8192, 1000, 1) == 1 and lib.plh_lsr_saves_lse(0, 8192, 32, 1) == 0
    assert lib.plh_lsr_saves_lse(2, 8192, 1000, 1) == 0 and lib.plh_lsr_saves_lse(2, 8192, 1100, 1) == 1 and lib.plh_lsr_saves_lse(1, 8192, 64, 1) == 1
    assert lib.plh_taylor_ce_saves_sums(0, 8192, 1000, 1) == 1 and lib.plh_taylor_ce_saves_sums(0, 8192, 256, 1) == 0
    assert lib.plh_taylor_ce_saves_sums(2, 8192, 1100, 1) == 1 and lib.plh_taylor_ce_saves_sums(2, 8192, 1000, 1) == 0 and lib.plh_taylor_ce_saves_sums(2, 8192, 2049, 1) == 1 and lib.plh_taylor_ce_saves_sums(2, 8192, 48, 1) == 1
    assert lib.plh_lmargin_saves_stats(1, 8192, 32000, 1) == 1 and lib.plh_lmargin_saves_stats(0, 8192, 1024, 1) == 0 and lib.plh_lmargin_saves_stats(0, 8192, 1000, 1) == 1 and lib.plh_lmargin_saves_stats(2, 8192, 1024, 1) == 1 and lib.plh_lmargin_saves_stats(2, 8192, 1100, 1) == 1 and lib.plh_lmargin_saves_stats(2, 8192, 4096, 1) == 1
    assert lib.plh_lmargin_saves_stats(0, 8, 5000, 64) == 0 and lib.plh_lmargin_saves_stats(9, 8192, 32000, 1) == 0
    assert lib.plh_lsr_saves_lse(0, 16, 19, 63 * 65) == 0 and lib.plh_lsr_saves_lse(7, 16, 19, 769 * 769) == 0
    assert lib.plh_lsr_forward_reduced_lse(p, 0, lp, p, p, None, 1, p, 1 << 20, 2, 19, 4096, 255, 0.1, None) == -2
    assert lib.plh_lsr_forward_reduced_lse(p, 0, lp, None, p, None, 1, p, 1 << 20, 2, 19, 4097, 255, 0.1, None) == -1
    assert lib.plh_lsr_backward_scaled_lse(p, 0, lp, p, None, p, 1.0, None, p, 2, 19, 4096, 255, 0.1, None) == -2
    assert lib.plh_lsr_backward_scaled_lse(p, 0, lp, None, None, p, 1.0, None, p, 2, 19, 4097, 255, 0.1, None) == -1
    # online hard example mining
    assert lib.plh_ohem_workspace_bytes(-1) == -2 and lib.plh_ohem_workspace_bytes(1 << 31) == -2
    ohem_need = lib.plh_ohem_workspace_bytes(4096)
    assert ohem_need >= 3 * 1024 * 4 + 4 * 4 and ohem_need % 256 == 0
    big = (ctypes.c_char * (ohem_need + 512))()
    wsp = ctypes.c_void_p((ctypes.addressof(big) + 255) & ~255)              # 256-byte aligned, as required
    assert lib.plh_ohem_scores(None, 0, None, None, 0, 19, 16, 255, None) == 0
    assert lib.plh_ohem_scores(p, 5, lp, p, 1, 2, 2, 255, None) == -7
    assert lib.plh_ohem_scores(p, 0, lp, None, 1, 2, 2, 255, None) == -1
    assert lib.plh_ohem_select_labels(None, None, None, None, 0, 0, 255, 0.7, 0, None) == 0
    assert lib.plh_ohem_select_labels(p, lp, None, wsp, ohem_need, 4, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_select_labels(p, lp, lp, None, 0, 4, 255, 0.7, 1, None) == -5
    assert lib.plh_ohem_select_labels(p, lp, lp, wsp, ohem_need, -4, 255, 0.7, 1, None) == -2
    assert lib.plh_ohem_score_label(p, 9, lp, lp, p, wsp, ohem_need, 1, 2, 2, 255, 0.7, 1, None) == -7
    assert lib.plh_ohem_score_label(p, 0, lp, lp, None, wsp, ohem_need, 1, 2, 2, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_score_label(p, 0, lp, lp, p, None, 0, 1, 2, 2, 255, 0.7, 1, None) == -5
    assert lib.plh_ohem_score_label(p, 0, lp, lp, p, ctypes.c_void_p(wsp.value + 8), ohem_need, 1, 2, 2, 255, 0.7, 1,
                                    None) == -5                                  # misaligned workspace
    # one-hot encoder
    assert lib.plh_onehot(None, None, None, 0, 19, 16, 255, 0.1, None) == 0
    assert lib.plh_onehot(lp, None, None, 1, 2, 2, 255, 0.1, None) == -1
    assert lib.plh_onehot(None, p, None, 1, 2, 2, 255, 0.1, None) == -1
    assert lib.plh_onehot(lp, p, None, 1, -2, 2, 255, 0.1, None) == -2
    assert lib.plh_onehot(lp, odd, None, 1, 2, 2, 255, 0.1, None) == -6
    assert lib.plh_onehot(lp, p, odd, 1, 2, 2, 255, 0.1, None) == -6
    # Taylor softmax and its cross entropy
    assert lib.plh_taylor_softmax_forward(None, 0, None, 0, 19, 16, 4, 0, None) == 0
    assert lib.plh_taylor_softmax_forward(p, 0, p, 1, 2, 2, 3, 0, None) == -2          # odd order
    assert lib.plh_taylor_softmax_forward(p, 0, p, 1, 2, 2, 0, 0, None) == -2
    assert lib.plh_taylor_softmax_forward(p, 4, p, 1, 2, 2, 2, 0, None) == -7
    assert lib.plh_taylor_softmax_forward(p, 0, None, 1, 2, 2, 2, 0, None) == -1
    assert lib.plh_taylor_softmax_forward(odd, 0, p, 1, 2, 2, 2, 0, None) == -6
    assert lib.plh_taylor_softmax_backward(None, p, 0, p, 1, 2, 2, 2, 1, None) == -1
    assert lib.plh_taylor_softmax_backward(odd, p, 0, p, 1, 2, 2, 2, 1, None) == -6
    assert lib.plh_taylor_ce_forward(p, 0, lp, None, None, None, 0, None, 0, 1, 2, 2, 2, 255, None) == -1
    assert lib.plh_taylor_ce_forward(p, 0, lp, None, p, None, 1, None, 0, 1, 2, 2, 2, 255, None) == -5
    assert lib.plh_taylor_ce_forward(p, 0, lp, p, None, None, 0, None, 0, 1, 2, 2, 5, 255, None) == -2
    assert lib.plh_taylor_ce_backward(p, 0, lp, p, 2, 1.0, None, p, 1, 2, 2, 2, 255, None) == -3
    assert lib.plh_taylor_ce_backward(p, 0, None, None, 0, 1.0, None, p, 1, 2, 2, 2, 255, None) == -1
    # soft dice
    assert lib.plh_soft_dice_workspace_bytes(-1, 4) == -2 and lib.plh_soft_dice_workspace_bytes(70000, 4) == -2
    dice_need = lib.plh_soft_dice_workspace_bytes(2, 5000)
    assert dice_need >= 2 * 5 * 8 and dice_need % 256 == 0
    assert lib.plh_soft_dice_forward(None, 0, None, None, None, None, 0, 0, 16, 1.0, 1.0, None) == 0
    assert lib.plh_soft_dice_forward(p, 3, p, p, p, wsp, dice_need, 2, 8, 1.0, 1.0, None) == -7
    assert lib.plh_soft_dice_forward(p, 0, None, p, p, wsp, dice_need, 2, 8, 1.0, 1.0, None) == -1
    assert lib.plh_soft_dice_forward(p, 0, p, p, None, wsp, dice_need, 2, 8, 1.0, 1.0, None) == -1
    assert lib.plh_soft_dice_forward(p, 0, p, p, p, None, 0, 2, 8, 1.0, 1.0, None) == -5
    assert lib.plh_soft_dice_forward(odd, 0, p, p, p, wsp, dice_need, 2, 8, 1.0, 1.0, None) == -6
    assert lib.plh_soft_dice_backward(None, p, 0, p, p, p, 2, 8, 1.0, None) == -1
    assert lib.plh_soft_dice_backward(p, p, 0, p, None, p, 2, 8, 1.0, None) == -1
    # fused OHEM cross entropy
    ce_need = lib.plh_ohem_ce_workspace_bytes(5000)
    assert ce_need >= lib.plh_ohem_workspace_bytes(5000) + 8 * 5 and ce_need % 256 == 0
    assert lib.plh_ohem_ce_workspace_bytes(-1) == -2
    assert lib.plh_ohem_ce_forward(p, 4, p, p, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -7
    assert lib.plh_ohem_ce_forward(p, 0, None, p, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_ce_forward(p, 0, p, p, p, p, None, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_ce_forward(p, 0, p, p, p, None, p, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_ce_forward(p, 0, p, p, p, p, p, p, None, 0, 1, 4, 16, 255, 0.7, 1, None) == -5
    assert lib.plh_ohem_ce_forward(p, 0, p, p, p, p, p, p, wsp, 16, 1, 4, 16, 255, 0.7, 1, None) == -5
    # fused OHEM large margin: the same checks behind one more scalar
    # the forwards that leave a byte mask instead of new labels, and the backwards that read it
    assert lib.plh_ohem_ce_forward_kept(p, 4, p, p, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -7
    assert lib.plh_ohem_ce_forward_kept(p, 0, p, None, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.7, 1, None) == -1
    assert lib.plh_ohem_ce_forward_kept(p, 0, p, p, p, p, p, p, wsp, 16, 1, 4, 16, 255, 0.7, 1, None) == -5
    assert lib.plh_ohem_lmargin_forward_kept(p, 0, p, None, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -1
    assert lib.plh_ohem_lmargin_forward_kept(p, 0, p, p, p, p, p, p, None, 0, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -5
    for back in (lib.plh_lsr_backward_kept, lib.plh_lmargin_backward_kept):
        assert back(p, 0, p, None, p, 1.0, None, p, 1, 4, 16, 255, 0.0, None) == -1
        assert back(p, 0, p, p, None, 1.0, None, p, 1, 4, 16, 255, 0.0, None) == -1
        assert back(p, 5, p, p, p, 1.0, None, p, 1, 4, 16, 255, 0.0, None) == -7
    assert lib.plh_ohem_lmargin_forward(p, 4, p, p, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -7
    assert lib.plh_ohem_lmargin_forward(p, 0, None, p, p, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -1
    assert lib.plh_ohem_lmargin_forward(p, 0, p, p, None, p, p, p, wsp, ce_need, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -1
    assert lib.plh_ohem_lmargin_forward(p, 0, p, p, p, p, p, p, wsp, 16, 1, 4, 16, 255, 0.3, 0.7, 1, None) == -5
    # layer norm
    assert lib.plh_layer_norm_forward(None, 0, None, 0, 4, 4, 1e-6, None) == 0
    assert lib.plh_layer_norm_forward(p, 5, p, 1, 4, 4, 1e-6, None) == -7
    assert lib.plh_layer_norm_forward(p, 0, None, 1, 4, 4, 1e-6, None) == -1
    assert lib.plh_layer_norm_forward(p, 0, p, -1, 4, 4, 1e-6, None) == -2
    assert lib.plh_layer_norm_forward(odd, 0, p, 1, 4, 4, 1e-6, None) == -6
    assert lib.plh_layer_norm_backward(None, p, 0, p, 1, 4, 4, 1e-6, None) == -1
    assert lib.plh_layer_norm_backward(p, p, 0, None, 1, 4, 4, 1e-6, None) == -1
    assert lib.plh_layer_norm_backward(odd, p, 0, p, 1, 4, 4, 1e-6, None) == -6
    # 16-bit logits need 2-byte alignment only; an odd address is still refused
    assert lib.plh_lsr_forward(ctypes.c_void_p(p.value + 1), 1, lp, p, 1, 2, 2, 255, 0.1, None) == -6
    assert lib.plh_reduce_workspace_bytes(100) == 8 * 16384
    assert lib.plh_reduce_workspace_bytes(-1) == -2


def test_python_surface_refuses_cpu_tensors():
    import pytorch_loss as pl
    x = torch.randn(2, 5, 4, 4, requires_grad=True)
    y = torch.randint(0, 5, (2, 4, 4))
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.LabelSmoothSoftmaxCEV3()(x, y)
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.LargeMarginSoftmaxV3()(x, y)
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.LovaszSoftmaxV3()(x, y)
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.FocalLossV3()(x, torch.rand_like(x))
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.LSRCrossEntropyFunctionV3.apply(x, y, 0.1, -100)


def test_constructor_defaults_match_the_reference():
    # pytorch_loss/label_smooth.py:150, focal_loss.py:177-180, large_margin_softmax.py:151,
    # lovasz_softmax.py:97
    import pytorch_loss as pl
    a = pl.LabelSmoothSoftmaxCEV3()
    assert (a.lb_smooth, a.reduction, a.lb_ignore) == (0.1, "mean", -100)
    b = pl.FocalLossV3()
    assert (b.alpha, b.gamma, b.reduction) == (0.25, 2, "mean")
    c = pl.LargeMarginSoftmaxV3()
    assert (c.lam, c.reduction, c.ignore_index) == (0.3, "mean", 255)
    d = pl.LovaszSoftmaxV3()
    assert (d.reduction, d.lb_ignore) == ("mean", -100)
    for name in ("LSRCrossEntropyFunctionV3", "FocalSigmoidLossFuncV3", "FocalSigmoidLossFuncV3FB",
                 "LargeMarginSoftmaxFuncV3", "LargeMarginSoftmaxFuncV3FB", "LovaszSoftmaxFunctionV3"):
        assert issubclass(getattr(pl, name), torch.autograd.Function)


def test_neighbouring_ops_mirror_the_reference_surface():
    # pytorch_loss/ohem_loss.py:15,32; one_hot.py:57-67; taylor_softmax.py:107,129,179; soft_dice_loss.py:117-123;
    # layer_norm.py:114-121
    import pytorch_loss as pl
    o = pl.OhemCELoss(0.7)
    assert (o.score_thresh, o.n_min, o.ignore_lb) == (0.7, None, 255)
    o = pl.OhemLargeMarginLoss(0.6, n_min=10, ignore_index=-1)
    assert (o.score_thresh, o.n_min, o.ignore_lb) == (0.6, 10, -1) and isinstance(o.criteria, pl.LargeMarginSoftmaxV3)
    e = pl.OnehotEncoder(19)
    assert (e.n_classes, e.lb_smooth, e.ignore_idx) == (19, 0., -1)
    for cls in (pl.TaylorSoftmaxV3, pl.LogTaylorSoftmaxV3):
        t = cls()
        assert (t.dim, t.n) == (1, 2)
    t = pl.TaylorCrossEntropyLossV3()
    assert (t.n, t.ignore_index, t.reduction) == (2, -1, "mean")
    d = pl.SoftDiceLossV3()
    assert (d.p, d.smooth) == (1, 1.)
    n = pl.LayerNormV3(8)
    assert (n.n_chan, n.affine, n.eps) == (8, True, 1e-6)
    assert n.weight.shape == (1, 8, 1) and n.bias.shape == (1, 8, 1)
    assert torch.equal(n.weight.data, torch.ones(1, 8, 1)) and torch.equal(n.bias.data, torch.zeros(1, 8, 1))
    assert pl.LayerNormV3(8, affine=False).weight is None
    for name in ("TaylorSoftmaxFunc", "TaylorCrossEntropyFunctionV3", "SoftDiceLossV3Func", "LayerNormV3Func"):
        assert issubclass(getattr(pl, name), torch.autograd.Function)
    x = torch.randn(2, 5, 4, 4)
    y = torch.randint(0, 5, (2, 4, 4))
    for call in (lambda: pl.OhemCELoss(0.7)(x, y), lambda: pl.OhemLargeMarginLoss(0.7)(x, y),
                 lambda: pl.OnehotEncoder(5)(y), lambda: pl.TaylorSoftmaxV3()(x), lambda: pl.LogTaylorSoftmaxV3()(x),
                 lambda: pl.TaylorCrossEntropyLossV3()(x, y), lambda: pl.SoftDiceLossV3()(x, torch.rand_like(x)),
                 lambda: pl.LayerNormV3(5)(x), lambda: pl.score_ohem_label(x, y, 255, 0.7, 2)):
        with pytest.raises(RuntimeError, match="only supports gpu mode"):
            call()
    # odd Taylor orders are refused before anything is launched (csrc/taylor_softmax.cu:295)
    with pytest.raises((RuntimeError, AssertionError)):
        pl.TaylorSoftmaxV3(n=3)(x)


def test_upstream_gradient_marshalling(native):
    like = (2, 3, 4)
    t, stride = native._upstream(None, like)
    assert t is None and stride == 0
    scalar = torch.tensor(0.5).expand(like)              # what sum()/mean() backward hands over
    t, stride = native._upstream(scalar, like)
    assert stride == 0 and t.numel() == 1 and t.item() == 0.5
    full = torch.rand(like)
    t, stride = native._upstream(full, like)
    assert stride == 1 and t.is_contiguous() and torch.equal(t, full)
    t, stride = native._upstream(full.double().transpose(1, 2).transpose(1, 2), like)
    assert stride == 1 and t.dtype == torch.float32
    assert native._dims(torch.zeros(3, 5), "x") == (3, 5, 1)
    assert native._dims(torch.zeros(3, 5, 2, 7), "x") == (3, 5, 14)
    with pytest.raises(RuntimeError):
        native._dims(torch.zeros(3), "x")
    with pytest.raises(RuntimeError, match="integer"):
        native._labels_i64(torch.zeros(3, 2, 7), torch.zeros(3, 5, 2, 7), "x")
    with pytest.raises(RuntimeError, match="do not match"):
        native._labels_i64(torch.zeros(3, 7, dtype=torch.long), torch.zeros(3, 5, 2, 7), "x")


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_taylor_orders_are_checked_where_the_reference_checks_them():
    """pytorch_loss/taylor_softmax.py: TaylorSoftmaxV3's constructor wants an even positive order (:85), the log
    module's and the cross entropy's only an even one (:131, :181); those two refuse n = 0 in their first forward (:50)."""
    import pytorch_loss as pl
    for bad in (0, 3, -2):
        with pytest.raises(AssertionError):
            pl.TaylorSoftmaxV3(dim=1, n=bad)
    for bad in (3, -1):
        with pytest.raises(AssertionError):
            pl.LogTaylorSoftmaxV3(dim=1, n=bad)
        with pytest.raises(AssertionError):
            pl.TaylorCrossEntropyLossV3(n=bad)
    x, y = torch.zeros(2, 3), torch.zeros(2, dtype=torch.int64)
    with pytest.raises(AssertionError):
        pl.LogTaylorSoftmaxV3(n=0)(x)
    with pytest.raises(AssertionError):
        pl.TaylorCrossEntropyLossV3(n=0)(x, y)
    assert pl.TaylorCrossEntropyLossV3(n=4).n == 4 and pl.LogTaylorSoftmaxV3(n=2).n == 2


def test_extension_stand_ins_refuse_labels_the_abi_would_misread():
    """The C ABI reads labels as int64, one per pixel: the stand-ins raise for another dtype (as the reference's
    data_ptr<int64_t>() does) or another element count before any pointer is handed over."""
    from ext_stubs import _abi
    x = torch.zeros(2, 3, 4)
    assert _abi.labels(torch.zeros(2, 4, dtype=torch.int64), x).dtype == torch.int64
    assert _abi.labels(torch.zeros(4, 2, dtype=torch.int64).t(), x).is_contiguous()
    for bad in (torch.zeros(2, 4, dtype=torch.int32), torch.zeros(2, 4, dtype=torch.uint8), torch.zeros(2, 4)):
        with pytest.raises(RuntimeError, match="Long"):
            _abi.labels(bad, x)
    for bad in (torch.zeros(2, 3, dtype=torch.int64), torch.zeros(2, 3, 4, dtype=torch.int64)):
        with pytest.raises(RuntimeError, match="do not go with"):
            _abi.labels(bad, x)
    assert _abi.labels(torch.zeros(5, dtype=torch.int64), torch.zeros(5, 7)).shape == (5,)


def test_extension_stand_ins_load_and_refuse_cpu_tensors():
    """The ctypes stand-ins for the reference's extension modules bind every entry point they use at import time
    (a misspelt or missing symbol fails here, without a GPU) and raise the extensions' own error for CPU tensors."""
    import sys
    import torch
    import ext_stubs
    saved = {n: sys.modules.get(n) for n in ext_stubs.NAMES}
    try:
        mods = ext_stubs.install()
        assert set(mods) == {"lsr_cpp", "focal_cpp", "large_margin_cpp", "lovasz_softmax_cpp", "ohem_cpp", "one_hot_cpp",
                             "taylor_softmax_cpp", "soft_dice_cpp", "layer_norm_cpp"}
        x = torch.zeros(2, 3, 4)
        y = torch.zeros(2, 4, dtype=torch.int64)
        calls = [
            lambda: mods["lsr_cpp"].lsr_forward(x, y, 255, 0.1),
            lambda: mods["lsr_cpp"].lsr_backward(x, y, 255, 0.1),
            lambda: mods["focal_cpp"].focalloss_forward(x, x, 2.0, 0.25),
            lambda: mods["focal_cpp"].focalloss_backward(x, x, 2.0, 0.25),
            lambda: mods["focal_cpp"].focalloss_forward_backward(x, x, 2.0, 0.25),
            lambda: mods["large_margin_cpp"].l_margin_forward(x, y, 0.3, 255),
            lambda: mods["large_margin_cpp"].l_margin_backward(x, y, 0.3, 255),
            lambda: mods["large_margin_cpp"].l_margin_forward_backward(x, y, 0.3, 255),
            lambda: mods["lovasz_softmax_cpp"].lovasz_softmax_forward(x, y, 255),
            lambda: mods["ohem_cpp"].score_ohem_label(x, y, 255, 0.7, 2),
            lambda: mods["one_hot_cpp"].label_one_hot(y, 255, 0.1, 3),
            lambda: mods["taylor_softmax_cpp"].taylor_softmax_forward(x, 1, 2, False),
            lambda: mods["taylor_softmax_cpp"].taylor_softmax_backward(x, x, 1, 2, False),
            lambda: mods["soft_dice_cpp"].soft_dice_forward(x[0], x[0], 1.0, 1.0),
            lambda: mods["soft_dice_cpp"].soft_dice_backward(torch.ones(3), x[0], x[0], 1.0, 1.0),
            lambda: mods["layer_norm_cpp"].layer_norm_forward(x, 1e-6),
            lambda: mods["layer_norm_cpp"].layer_norm_backward(x, x, 1e-6),
        ]
        for call in calls:
            with pytest.raises(RuntimeError, match="only supports gpu mode"):
                call()
    finally:
        for n, m in saved.items():
            if m is None:
                sys.modules.pop(n, None)
            else:
                sys.modules[n] = m
