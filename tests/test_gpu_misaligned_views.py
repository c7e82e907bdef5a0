"""Tensors that start one element into their storage (views of larger buffers): aligned to their element type,
as the C ABI requires, but to nothing wider. Every kernel that moves 8 or 16 bytes per access has to notice and take
its element-wise form; results against the CPU oracle to the usual bars."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

from .test_gpu_dtypes import ULP_REL
from .test_gpu_parity import close_grad, close_loss, seg_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def shifted(a, dt=None, by=1):
    """The array on the GPU as a contiguous view that starts `by` elements into a larger allocation."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dt is not None:
        t = t.to(dt)
    buf = torch.empty(t.numel() + by + 7, dtype=t.dtype, device="cuda")
    view = buf[by:by + t.numel()].view(t.shape)
    view.copy_(t)
    assert view.is_contiguous() and view.data_ptr() == buf.data_ptr() + by * t.element_size()
    return view


SHAPES = [(2, 19, 32, 32), (2, 19, 65, 65), (2, 40, 16, 16), (2, 40, 64, 64), (1, 150, 65, 63), (1, 300, 8, 8), (37, 100), (5, 4104),
          (2, 50001), (300, 19)]


@pytest.mark.parametrize("which", ["logits", "labels", "both"])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("kind", ["lsr", "lmargin", "taylor"])
def test_channel_softmax_losses(pl, kind, shape, dt, which):
    x, y = seg_inputs(700, shape, 255, 0.1)
    xt = shifted(x, dt, 1 if which != "labels" else 0)
    yt = shifted(y, None, 1 if which != "logits" else 0)
    xr = xt.float().cpu().numpy()
    xt.requires_grad_()
    if kind == "lsr":
        losses = pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, 255)
        want = oracle.lsr_forward(xr, y, 255, 0.1)
        grad_of = lambda g: oracle.lsr_backward(xr, y, 255, 0.1, g)
    elif kind == "lmargin":
        losses = pl.LargeMarginSoftmaxFuncV3.apply(xt, yt, 0.3, 255)
        want = oracle.lmargin_forward(xr, y, 0.3, 255)
        grad_of = lambda g: oracle.lmargin_backward(xr, y, 0.3, 255, g)
    else:
        losses = pl.TaylorCrossEntropyFunctionV3.apply(xt, yt, 4, 255, "none")
        want = oracle.taylor_ce(xr.astype(np.float64), y, 4, 255)
        grad_of = lambda g: oracle.taylor_ce_backward(xr.astype(np.float64), y, 4, 255, g.astype(np.float64))
    got = losses.detach().float().cpu().numpy()
    if dt == torch.float32:
        close_loss(got, want, kind)
    else:
        assert np.all(np.abs(got - want) <= ULP_REL[dt] * np.abs(want) + 1e-6)
    go = synth.normal(700, 3, y.shape, 0.0, 1.0)
    got = shifted(go, losses.dtype, 1)              # the upstream gradient too
    losses.backward(got)
    want_g = np.asarray(grad_of(got.float().cpu().numpy()))
    g = xt.grad.float().cpu().numpy().astype(np.float64)
    if dt == torch.float32:
        if kind == "taylor":
            assert np.abs(g - want_g).max() <= 1e-5 * max(1.0, np.abs(want_g).max())
        else:
            close_grad(g, want_g, kind)
    else:
        assert np.all(np.abs(g - want_g) <= ULP_REL[dt] * np.abs(want_g) + 1e-7 + 1e-6 * np.abs(want_g).max())
    # the module's fused mean on the same views
    crit = {"lsr": lambda: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, ignore_index=255),
            "lmargin": lambda: pl.LargeMarginSoftmaxV3(lam=0.3, ignore_index=255),
            "taylor": lambda: pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255)}[kind]()
    mean = crit(xt.detach(), yt)
    want_mean = want.sum(dtype=np.float64) / max(1, int((y != 255).sum()))
    assert abs(mean.item() - want_mean) <= (1e-5 + (ULP_REL[dt] if dt != torch.float32 else 0)) * abs(want_mean)


@pytest.mark.parametrize("dt", [torch.float32, torch.float16], ids=["fp32", "fp16"])
def test_focal_lovasz_ohem_onehot(pl, dt):
    from pytorch_loss import _native
    # focal: logits and float labels
    shape = (3, 7, 33, 31)
    x = synth.normal(701, 1, shape, -1.0, 2.0)
    y = synth.bernoulli(701, 2, shape, 0.2).astype(np.float32)
    xt, yt = shifted(x, dt), shifted(y, dt)
    xr = xt.float().cpu().numpy()
    xt.requires_grad_()
    loss = pl.FocalSigmoidLossFuncV3.apply(xt, yt, 0.25, 2.0)
    want = oracle.focal_forward(xr, y, 0.25, 2.0)
    tol = 1e-6 if dt == torch.float32 else ULP_REL[dt]
    assert np.all(np.abs(loss.detach().float().cpu().numpy() - want) <= 1e-5 * np.abs(want) + tol * np.abs(want) + 1e-6)
    loss.sum().backward()
    want_g = oracle.focal_backward(xr, y, 0.25, 2.0, np.float32(1.0))
    assert np.all(np.abs(xt.grad.float().cpu().numpy() - want_g) <= (ULP_REL.get(dt, 0.0)) * np.abs(want_g) + 1e-5)
    # Lovasz, OHEM scores and relabelling
    shape = (2, 19, 40, 41)
    x, lb = seg_inputs(702, shape, 255, 0.1)
    xt, lt = shifted(x, dt), shifted(lb)
    xr = xt.float().cpu().numpy()
    losses, jacc = _native.lovasz_forward(xt, lt, 255)
    l64, _ = oracle.lovasz_forward(xr.astype(np.float64), lb, 255)
    np.testing.assert_allclose(losses.float().cpu().numpy(), l64, rtol=1e-5 + (ULP_REL[dt] if dt != torch.float32 else 0))
    assert (jacc.cpu().numpy()[:, lb.reshape(-1) == 255] == 0).all()
    scores = _native.ohem_scores(xt, lt, 255).cpu().numpy()
    assert np.abs(scores - oracle.ohem_scores(xr, lb, 255)).max() <= 1e-6
    new = _native.ohem_score_label(xt, lt, 255, 0.7, lb.size // 8).cpu().numpy()
    assert np.array_equal(new, oracle.ohem_select(scores, lb, 255, 0.7, lb.size // 8))
    assert np.array_equal(lt.cpu().numpy(), lb)
    # one-hot from shifted labels
    got = pl.OnehotEncoder(19, lb_smooth=0.1, ignore_idx=255)(lt).cpu().numpy()
    assert np.array_equal(got, oracle.onehot(lb, 19, 0.1, 255))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_taylor_softmax_dice_layernorm(pl, dt):
    rel = 1e-5 if dt == torch.float32 else ULP_REL[dt]
    for shape in ((2, 19, 130), (3, 100, 7), (40, 1000, 1)):
        x = synth.normal(703, 1, shape, 0.0, 1.0)
        g = synth.normal(703, 2, shape, 0.0, 1.0)
        xt, gt = shifted(x, dt), shifted(g, dt)
        xr, gr = xt.float().cpu().numpy().astype(np.float64), gt.float().cpu().numpy().astype(np.float64)
        xt.requires_grad_()
        out = pl.TaylorSoftmaxFunc.apply(xt, 1, 4, True)
        want = oracle.taylor_forward(xr, 1, 4, True)
        assert np.all(np.abs(out.detach().float().cpu().numpy() - want) <= rel * np.abs(want) + 1e-5), shape
        out.backward(gt)
        want_g = oracle.taylor_backward(gr, xr, 1, 4, True)
        assert np.all(np.abs(xt.grad.float().cpu().numpy() - want_g) <= rel * np.abs(want_g) + 1e-5 * max(1.0, np.abs(want_g).max())), shape
        x2 = shifted(x, dt).requires_grad_()
        ln = pl.LayerNormV3Func.apply(x2, 1e-6)
        want = oracle.layer_norm_forward(xr, 1e-6)
        assert np.all(np.abs(ln.detach().float().cpu().numpy() - want) <= rel * np.abs(want) + 1e-5), shape
        ln.backward(gt)
        want_g = oracle.layer_norm_backward(gr, xr, 1e-6)
        assert np.all(np.abs(x2.grad.float().cpu().numpy() - want_g) <= rel * np.abs(want_g) + 1e-5 * np.abs(want_g).max()), shape
    n, length = 3, 10_001
    x = synth.normal(704, 1, (n, length), 0.0, 2.0)
    y = synth.uniform01(704, 2, n * length).reshape(n, length).astype(np.float32)
    xt, yt = shifted(x, dt), shifted(y, dt)
    xr, yr = xt.float().cpu().numpy().astype(np.float64), yt.float().cpu().numpy().astype(np.float64)
    xt.requires_grad_()
    loss = pl.SoftDiceLossV3Func.apply(xt, yt, 2.0, 1.0)
    want, stats = oracle.soft_dice_forward(xr, yr, 2.0, 1.0)
    assert np.all(np.abs(loss.detach().float().cpu().numpy() - want) <= (1e-5 + (rel if dt != torch.float32 else 0)) * np.abs(want) + 1e-7)
    loss.sum().backward()
    want_g = oracle.soft_dice_backward(np.ones(n), xr, yr, stats, 2.0)
    assert np.all(np.abs(xt.grad.float().cpu().numpy() - want_g) <= rel * np.abs(want_g) + 1e-5 * np.abs(want_g).max() + 1e-12)
