"""A seeded sweep over shapes nobody picked by hand: every launch shape has its boundaries in the tables of
test_gpu_parity.py; this walks random points between them (channel counts 1..600, odd and even planes on both
sides of the 4096-pixel limit of the per-image form, (N, C) rows up to 6000, all three storage types, the three
ignore conventions) for the four channel-softmax losses and the OHEM scores, against the CPU oracle to the usual bars."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

from .test_gpu_dtypes import ULP_REL, close_grad_stored
from .test_gpu_parity import close_grad, close_loss, dev, seg_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _draw(seed):
    r = np.random.RandomState(1000 + seed)
    kind = ("lsr", "lmargin", "taylor", "ohem")[seed % 4]
    family = r.randint(5)
    if family == 0:            # segmentation, channels in registers
        shape = (int(r.randint(1, 4)), int(r.randint(1, 33)), int(r.randint(1, 70)), int(r.randint(1, 70)))
    elif family == 1:          # fp32 planes around the per-image form: odd lengths of 4096 pixels or more, C <= 24 and just above
        h = int(r.randint(60, 100)) | 1
        w = int(r.randint(64, 100)) | 1
        shape = (int(r.randint(1, 4)), int(r.randint(2, 27)), h, w)
    elif family == 2:          # channels shared out over the wavefronts of a block (33..512) and a lane per pixel beyond
        shape = (int(r.randint(1, 3)), int(r.randint(33, 600)), int(r.randint(1, 24)), int(r.randint(1, 24)))
    elif family == 3:          # (N, C) rows: a wavefront or a block per row
        shape = (int(r.randint(1, 40)), int(r.choice([r.randint(1, 33), r.randint(33, 2049), r.randint(2049, 6000)])))
    else:                      # 5-D and 3-D inputs
        shape = (int(r.randint(1, 3)), int(r.randint(2, 80))) + tuple(int(v) for v in r.randint(1, 9, size=int(r.choice([1, 3]))))
    ignore = int(r.choice([255, -100, 0]))
    frac = float(r.choice([0.0, 0.1, 0.5]))
    dt = (torch.float32, torch.float32, torch.bfloat16, torch.float16)[int(r.randint(4))]
    gain = float(r.choice([1.0, 1.0, 5.0, 20.0]))      # logits 2 N(0,1) times this: up to saturated softmaxes
    return kind, shape, ignore, frac, dt, gain


@pytest.mark.parametrize("seed", range(160))
def test_random_shape(pl, seed):
    from pytorch_loss import _native
    kind, shape, ignore, frac, dt, gain = _draw(seed)
    if kind == "lmargin" and shape[1] < 2:
        shape = (shape[0], 2) + shape[2:]           # 1 / (C - 1)
    if kind == "taylor":
        gain = min(gain, 5.0)                       # the series is a polynomial: |x| = 100 is outside its use
    x, y = seg_inputs(300 + seed, shape, ignore, frac)
    x = x * np.float32(gain)
    xt = dev(x).to(dt)
    xr = xt.float().cpu().numpy()                   # what the kernels see, widened
    yt = dev(y)
    what = "%s %s %s ignore=%d gain=%g" % (kind, shape, str(dt)[6:], ignore, gain)
    if kind == "ohem":
        got = _native.ohem_scores(xt, yt, ignore).cpu().numpy()
        assert np.abs(got - oracle.ohem_scores(xr, y, ignore)).max() <= 1e-6, what
        return
    xt.requires_grad_()
    if kind == "lsr":
        losses = pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, ignore)
        want = oracle.lsr_forward(xr, y, ignore, 0.1)
        grad_of = lambda g: oracle.lsr_backward(xr, y, ignore, 0.1, g)
    elif kind == "lmargin":
        losses = pl.LargeMarginSoftmaxFuncV3.apply(xt, yt, 0.3, ignore)
        want = oracle.lmargin_forward(xr, y, 0.3, ignore)
        grad_of = lambda g: oracle.lmargin_backward(xr, y, 0.3, ignore, g)
    else:
        losses = pl.TaylorCrossEntropyFunctionV3.apply(xt, yt, 4, ignore, "none")
        want = oracle.taylor_ce(xr.astype(np.float64), y, 4, ignore)
        grad_of = lambda g: oracle.taylor_ce_backward(xr.astype(np.float64), y, 4, ignore, g.astype(np.float64))
    assert losses.shape == yt.shape, what
    got = losses.detach().float().cpu().numpy()
    if dt == torch.float32:
        close_loss(got, want, what)
    else:                                           # losses come back in the storage type: one rounding of it
        assert np.all(np.abs(got - want) <= ULP_REL[dt] * np.abs(want) + 1e-6), what
    assert (got[y == ignore] == 0).all(), what
    go = synth.normal(300 + seed, 3, y.shape, 0.0, 1.0)
    losses.backward(dev(go).to(losses.dtype))
    go_seen = dev(go).to(losses.dtype).float().cpu().numpy()
    want_g = np.asarray(grad_of(go_seen))
    if dt == torch.float32:
        if kind == "taylor":                        # gradients through log f grow where f comes close to 0
            err = np.abs(xt.grad.cpu().numpy() - want_g).max() if want_g.size else 0.0
            assert err <= 1e-5 * max(1.0, np.abs(want_g).max()), (what, err)
        elif gain > 1:                              # large-margin gradients grow with the logits: relative to the largest
            err = np.abs(xt.grad.cpu().numpy() - want_g).max() if want_g.size else 0.0
            assert err <= 1e-5 * max(1.0, np.abs(want_g).max()), (what, err)
        else:
            close_grad(xt.grad.cpu().numpy(), want_g, what)
    else:
        got_g = xt.grad.float().cpu().numpy().astype(np.float64)
        assert xt.grad.dtype == dt, what
        slack = 1e-7 + 1e-6 * (np.abs(want_g).max() if want_g.size else 0.0)       # fp32 evaluation in front of the rounding
        assert np.all(np.abs(got_g - want_g) <= ULP_REL[dt] * np.abs(want_g) + slack), what
    g = xt.grad.float().cpu().numpy()
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all(), what


@pytest.mark.parametrize("seed", range(40))
def test_random_shape_lovasz(pl, seed):
    """The sort pipeline at random row lengths and class counts (tiles that end anywhere, rows shorter than a
    tile, classes without positives, one to three storage types): loss per class against the fp64 restatement,
    Jaccard differences mostly bit-equal to the fp32 one, exact zeros at ignored pixels, and the gradient to the
    bound that near-ties allow."""
    from pytorch_loss import _native
    r = np.random.RandomState(5000 + seed)
    shape = (int(r.randint(1, 4)), int(r.randint(1, 41)), int(r.randint(1, 90)), int(r.randint(1, 90)))
    ignore = int(r.choice([255, -100]))
    frac = float(r.choice([0.0, 0.1, 0.6]))
    scale = float(r.choice([0.5, 2.0, 6.0]))
    dt = (torch.float32, torch.float32, torch.bfloat16)[int(r.randint(3))]
    x = synth.normal(400 + seed, 1, shape, 0.0, scale)
    y = synth.seg_labels(400 + seed, shape[:1] + shape[2:], shape[1], ignore, frac)
    xt = dev(x).to(dt)
    xr = xt.float().cpu().numpy()
    what = "lovasz %s %s ignore=%d scale=%g" % (shape, str(dt)[6:], ignore, scale)
    losses, jacc = _native.lovasz_forward(xt, dev(y), ignore)
    jacc = jacc.cpu().numpy()
    l64, j64 = oracle.lovasz_forward(xr.astype(np.float64), y, ignore)
    rtol = 3e-4 if scale > 2 else 1e-5              # confident logits: 1 - p carries p's fp32 rounding enlarged
    if dt != torch.float32:
        rtol += ULP_REL[dt]                         # the losses come back in the storage type
    np.testing.assert_allclose(losses.float().cpu().numpy(), l64, rtol=rtol, atol=1e-7, err_msg=what)
    assert (jacc[:, y.reshape(-1) == ignore] == 0).all(), what
    if (y != ignore).any():
        np.testing.assert_allclose(jacc.sum(axis=1, dtype=np.float64), 1.0, rtol=1e-4, err_msg=what)
    _, j32 = oracle.lovasz_forward(xr, y, ignore)
    assert (jacc.view(np.uint32) == j32.view(np.uint32)).mean() > 0.99, what
    xt.requires_grad_()
    out = pl.LovaszSoftmaxFunctionV3.apply(xt, dev(y), ignore)
    w = synth.normal(400 + seed, 4, (shape[1],), 0.5, 1.0)
    out.backward(dev(w).to(out.dtype))
    w_seen = dev(w).to(out.dtype).float().cpu().numpy().astype(np.float64)
    want_g = oracle.lovasz_backward(w_seen, xr.astype(np.float64), y, j64, ignore)
    g = xt.grad.float().cpu().numpy()
    bound = max(1e-5, 2e-3 * np.abs(j64).max() * np.abs(w_seen).max())
    if dt != torch.float32:
        bound += ULP_REL[dt] * np.abs(want_g).max()
    assert np.abs(g - want_g).max() <= bound, (what, np.abs(g - want_g).max(), bound)
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all(), what


@pytest.mark.parametrize("seed", range(80))
def test_random_shape_neighbouring_ops(pl, seed):
    """Focal, Taylor softmax, soft dice and layer norm at random sizes (element counts that end anywhere inside a
    vector, a wavefront or a block; channel counts on both sides of every launch shape of the layer norm)."""
    r = np.random.RandomState(7000 + seed)
    kind = ("focal", "taylor_sm", "dice", "layernorm")[seed % 4]
    if kind == "focal":
        shape = tuple(int(v) for v in r.randint(1, 40, size=int(r.randint(1, 5))))
        x = synth.normal(500 + seed, 1, shape, -1.0, 2.0)
        if seed % 8 < 4:
            y = synth.bernoulli(500 + seed, 2, shape, 0.2).astype(np.float32)
        else:
            y = synth.uniform01(500 + seed, 2, int(np.prod(shape))).reshape(shape).astype(np.float32)
        alpha, gamma = float(r.choice([0.25, 0.6])), float(r.choice([0.0, 1.5, 2.0]))
        xt = dev(x).requires_grad_()
        loss = pl.FocalSigmoidLossFuncV3.apply(xt, dev(y), alpha, gamma)
        close_loss(loss.detach().cpu().numpy(), oracle.focal_forward(x, y, alpha, gamma), "focal %s" % (shape,))
        go = synth.normal(500 + seed, 3, shape, 0.0, 1.0)
        loss.backward(dev(go))
        close_grad(xt.grad.cpu().numpy(), oracle.focal_backward(x, y, alpha, gamma, go), "focal %s" % (shape,))
    elif kind == "taylor_sm":
        shape = (int(r.randint(1, 4)), int(r.choice([r.randint(1, 33), r.randint(33, 300), r.randint(300, 3000)])),
                 int(r.choice([1, r.randint(1, 70)])))
        order, use_log = int(r.choice([2, 4, 6])), bool(r.randint(2))
        x = synth.normal(500 + seed, 1, shape, 0.0, 1.0)
        g = synth.normal(500 + seed, 2, shape, 0.0, 1.0)
        xt = dev(x).requires_grad_()
        out = pl.TaylorSoftmaxFunc.apply(xt, 1, order, use_log)
        want = oracle.taylor_forward(x.astype(np.float64), 1, order, use_log)
        assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-5 * max(1.0, np.abs(want).max()), shape
        out.backward(dev(g))
        want_g = oracle.taylor_backward(g.astype(np.float64), x.astype(np.float64), 1, order, use_log)
        assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * max(1.0, np.abs(want_g).max()), shape
    elif kind == "dice":
        n, length = int(r.randint(1, 9)), int(r.choice([r.randint(1, 100), r.randint(100, 70000)]))
        p, smooth = float(r.choice([1.0, 2.0, 1.5])), float(r.choice([1.0, 0.1]))
        x = synth.normal(500 + seed, 1, (n, length), 0.0, 2.0)
        y = synth.uniform01(500 + seed, 2, n * length).reshape(n, length).astype(np.float32)
        xt = dev(x).requires_grad_()
        loss = pl.SoftDiceLossV3Func.apply(xt, dev(y), p, smooth)
        want, stats = oracle.soft_dice_forward(x.astype(np.float64), y.astype(np.float64), p, smooth)
        assert np.abs(loss.detach().cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max() + 1e-7, (n, length)
        go = synth.normal(500 + seed, 3, (n,), 0.5, 1.0)
        loss.backward(dev(go))
        want_g = oracle.soft_dice_backward(go.astype(np.float64), x.astype(np.float64), y.astype(np.float64), stats, p)
        assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * np.abs(want_g).max() + 1e-12, (n, length)
    else:
        shape = (int(r.randint(1, 4)), int(r.choice([r.randint(1, 33), r.randint(33, 513), r.randint(513, 1500)])),
                 int(r.choice([1, r.randint(1, 200)])))
        x = synth.normal(500 + seed, 1, shape, 0.3, 1.5)
        g = synth.normal(500 + seed, 2, shape, 0.0, 1.0)
        xt = dev(x).requires_grad_()
        out = pl.LayerNormV3Func.apply(xt, 1e-6)
        if shape[1] > 1:
            assert np.abs(out.detach().cpu().numpy() - oracle.layer_norm_forward(x.astype(np.float64), 1e-6)).max() <= 1e-5, shape
        out.backward(dev(g))
        want_g = oracle.layer_norm_backward(g.astype(np.float64), x.astype(np.float64), 1e-6)
        assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * np.abs(want_g).max(), shape


@pytest.mark.parametrize("seed", range(60))
def test_random_shape_module_reductions(pl, seed):
    """'mean' / 'sum' of the modules (per-block partials inside the forward kernel, a fixed-order finish, the
    upstream scalar and 1 / n_valid folded into the backward) at random shapes large enough for many blocks, on every
    launch shape: loss and gradient against the oracle's reduction of its per-pixel values."""
    r = np.random.RandomState(9000 + seed)
    kind = ("lsr", "lmargin", "taylor", "ohem_ce")[seed % 4]
    family = r.randint(4)
    if family == 0:
        shape = (int(r.randint(1, 5)), int(r.randint(2, 33)), int(r.randint(20, 200)), int(r.randint(20, 200)))
    elif family == 1:          # odd planes: the per-image form for fp32
        shape = (int(r.randint(1, 5)), int(r.randint(2, 25)), int(r.randint(64, 160)) | 1, int(r.randint(64, 160)) | 1)
    elif family == 2:
        shape = (int(r.randint(1, 3)), int(r.randint(33, 520)), int(r.randint(8, 40)), int(r.randint(8, 40)))
    else:
        shape = (int(r.randint(100, 3000)), int(r.choice([r.randint(2, 33), r.randint(33, 1200)])))
    ignore = int(r.choice([255, -100]))
    reduction = ("mean", "sum")[int(r.randint(2))]
    dt = (torch.float32, torch.float32, torch.bfloat16)[int(r.randint(3))]
    x, y = seg_inputs(600 + seed, shape, ignore, 0.1)
    xt = dev(x).to(dt)
    xr = xt.float().cpu().numpy()
    xt.requires_grad_()
    yt = dev(y)
    what = "%s %s %s %s" % (kind, shape, reduction, str(dt)[6:])
    n_valid = int((y != ignore).sum())
    if kind == "lsr":
        crit = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=reduction, ignore_index=ignore)
        per = oracle.lsr_forward(xr.astype(np.float64), y, ignore, 0.1)
        grad_of = lambda g: oracle.lsr_backward(xr, y, ignore, 0.1, g)
    elif kind == "lmargin":
        crit = pl.LargeMarginSoftmaxV3(lam=0.3, reduction=reduction, ignore_index=ignore)
        per = oracle.lmargin_forward(xr.astype(np.float64), y, 0.3, ignore)
        grad_of = lambda g: oracle.lmargin_backward(xr, y, 0.3, ignore, g)
    elif kind == "taylor":
        crit = pl.TaylorCrossEntropyLossV3(n=4, ignore_index=ignore, reduction=reduction)
        per = oracle.taylor_ce(xr.astype(np.float64), y, 4, ignore)
        grad_of = lambda g: oracle.taylor_ce_backward(xr.astype(np.float64), y, 4, ignore, g)
    else:
        # OhemCELoss with a threshold no score exceeds keeps every label: plain cross entropy, mean over the valid pixels
        crit = pl.OhemCELoss(score_thresh=2.0, n_min=1, ignore_index=ignore)
        reduction = "mean"
        per = oracle.lsr_forward(xr.astype(np.float64), y, ignore, 0.0)
        grad_of = lambda g: oracle.lsr_backward(xr, y, ignore, 0.0, g)
    loss = crit(xt, yt)
    assert loss.dim() == 0, what
    want = per.sum(dtype=np.float64) / (n_valid if reduction == "mean" else 1)
    rtol = 1e-5 + (ULP_REL[dt] if dt != torch.float32 else 0.0)
    assert abs(loss.item() - want) <= rtol * abs(want), (what, loss.item(), want)
    loss.backward()
    scale = np.float32(1.0 / n_valid) if reduction == "mean" else np.float32(1.0)
    want_g = np.asarray(grad_of(np.full(y.shape, scale, dtype=np.float32)))
    if dt == torch.float32:
        err = np.abs(xt.grad.cpu().numpy() - want_g).max()
        assert err <= 2e-5 * np.abs(want_g).max() + 1e-12, (what, err, np.abs(want_g).max())
    else:
        close_grad_stored(xt.grad, want_g, dt, what)


@pytest.mark.parametrize("seed", range(48))
def test_random_shape_fused_variants(pl, seed):
    """The forward+backward-in-one-pass Functions (focal, large margin with its valid count) and the OHEM modules
    (relabelling and loss in one forward pass) at random shapes: against the oracle, and the OHEM losses against the
    composition of the separately tested relabelling with the plain loss on the new labels."""
    from pytorch_loss import _native
    r = np.random.RandomState(11000 + seed)
    kind = ("focal_fb", "lmargin_fb", "ohem_ce", "ohem_lm")[seed % 4]
    if kind == "focal_fb":
        shape = tuple(int(v) for v in r.randint(1, 50, size=int(r.randint(1, 5))))
        x = synth.normal(800 + seed, 1, shape, -1.0, 2.0)
        y = synth.bernoulli(800 + seed, 2, shape, 0.3).astype(np.float32)
        alpha, gamma = float(r.choice([0.25, 0.5])), float(r.choice([0.0, 1.0, 2.0, 3.0]))
        xt = dev(x).requires_grad_()
        loss = pl.FocalSigmoidLossFuncV3FB.apply(xt, dev(y), alpha, gamma)
        close_loss(loss.detach().cpu().numpy(), oracle.focal_forward(x, y, alpha, gamma), "focal fb %s" % (shape,))
        go = synth.normal(800 + seed, 3, shape, 0.0, 1.0)
        loss.backward(dev(go))
        close_grad(xt.grad.cpu().numpy(), oracle.focal_backward(x, y, alpha, gamma, go), "focal fb %s" % (shape,))
        return
    family = r.randint(3)
    if family == 0:
        shape = (int(r.randint(1, 4)), int(r.randint(2, 33)), int(r.randint(1, 90)), int(r.randint(1, 90)))
    elif family == 1:
        shape = (int(r.randint(1, 3)), int(r.randint(33, 520)), int(r.randint(8, 24)), int(r.randint(8, 24)))
    else:
        shape = (int(r.randint(16, 600)), int(r.choice([r.randint(2, 33), r.randint(33, 3000)])))
    ignore = int(r.choice([255, -100]))
    x, y = seg_inputs(800 + seed, shape, ignore, 0.1)
    x = x * np.float32(r.choice([1.0, 2.0]))
    xt = dev(x).requires_grad_()
    yt = dev(y)
    what = "%s %s ignore=%d" % (kind, shape, ignore)
    if kind == "lmargin_fb":
        losses, cnt = pl.LargeMarginSoftmaxFuncV3FB.apply(xt, yt, 0.3, ignore)
        assert cnt.dtype == torch.int64 and int(cnt.item()) == int((y != ignore).sum()), what
        close_loss(losses.detach().cpu().numpy(), oracle.lmargin_forward(x, y, 0.3, ignore), what)
        go = synth.normal(800 + seed, 3, y.shape, 0.0, 1.0)
        losses.backward(dev(go))
        close_grad(xt.grad.cpu().numpy(), oracle.lmargin_backward(x, y, 0.3, ignore, go), what)
        return
    thresh = float(r.choice([0.3, 0.7, 0.9]))
    n_min = int(y.size // int(r.choice([4, 16, 64]))) + 1
    crit = (pl.OhemCELoss if kind == "ohem_ce" else pl.OhemLargeMarginLoss)(thresh, n_min, ignore)
    loss = crit(xt, yt)
    new = _native.ohem_score_label(xt.detach(), yt, ignore, thresh, n_min).cpu().numpy()
    assert np.array_equal(yt.cpu().numpy(), y), what
    n_valid = int((new != ignore).sum())
    assert n_valid >= min(n_min, int((y != ignore).sum())) - 0, what
    if kind == "ohem_ce":
        per = oracle.lsr_forward(x.astype(np.float64), new, ignore, 0.0)
        grad_of = lambda g: oracle.lsr_backward(x, new, ignore, 0.0, g)
    else:
        per = oracle.lmargin_forward(x.astype(np.float64), new, 0.3, ignore)
        grad_of = lambda g: oracle.lmargin_backward(x, new, 0.3, ignore, g)
    want = per.sum(dtype=np.float64) / max(n_valid, 1)
    if n_valid == 0:
        assert np.isnan(loss.item()), what
        return
    assert abs(loss.item() - want) <= 1e-5 * abs(want), (what, loss.item(), want)
    loss.backward()
    want_g = np.asarray(grad_of(np.full(y.shape, np.float32(1.0 / n_valid), dtype=np.float32)))
    err = np.abs(xt.grad.cpu().numpy() - want_g).max()
    assert err <= 2e-5 * np.abs(want_g).max() + 1e-12, (what, err)
