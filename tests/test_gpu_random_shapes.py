"""Seeded sweep over small random shapes: every op against the CPU oracle on sizes nobody picked
by hand (odd extents, one channel, one pixel, tiles that end mid-wave, channel counts on both
sides of every kernel-shape boundary). Same tolerances as the hand-picked parity tests."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth
from .test_gpu_parity import close_grad, close_loss, dev, seg_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _shapes(seed, count, max_c, max_m):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        n = int(rng.integers(1, 4))
        c = int(rng.choice([1, 2, 3, int(rng.integers(4, max_c + 1))]))
        m = int(rng.choice([1, 2, int(rng.integers(3, 70)), int(rng.integers(70, max_m + 1))]))
        out.append((n, c, m))
    return out


@pytest.mark.parametrize("shape", _shapes(1, 24, 40, 700))
def test_pixel_losses(pl, shape):
    n, c, m = shape
    x, y = seg_inputs(200 + n * c * m, (n, c, m), 255, 0.1)
    yt = dev(y)
    go = synth.normal(201, 3, y.shape, 0.0, 1.0)
    for name, fn, fwd, bwd in (
            ("lsr", lambda t: pl.LSRCrossEntropyFunctionV3.apply(t, yt, 0.1, 255),
             lambda: oracle.lsr_forward(x, y, 255, 0.1), lambda: oracle.lsr_backward(x, y, 255, 0.1, go)),
            ("lmargin", lambda t: pl.LargeMarginSoftmaxFuncV3.apply(t, yt, 0.3, 255),
             lambda: oracle.lmargin_forward(x, y, 0.3, 255), lambda: oracle.lmargin_backward(x, y, 0.3, 255, go)),
            ("taylor", lambda t: pl.TaylorCrossEntropyFunctionV3.apply(t, yt, 4, 255, "none"),
             lambda: oracle.taylor_ce(x, y, 4, 255), lambda: oracle.taylor_ce_backward(x, y, 4, 255, go))):
        if c == 1 and name == "lmargin":
            continue    # the margin term carries 1 / (C - 1) (csrc/large_margin_kernel.cu:100): undefined for one class
        xt = dev(x).requires_grad_()
        out = fn(xt)
        if c == 1:      # a single class: every loss is exactly 0; the kernels' exp2/log2 pair leaves ~5e-8
            assert np.abs(out.detach().cpu().numpy() - fwd()).max() <= 1e-6
        else:
            close_loss(out.detach().cpu().numpy(), fwd(), "%s %s" % (name, shape))
        out.backward(dev(go))
        if c == 1:      # and every gradient is exactly 0: what is left on either side is rounding
            assert np.abs(xt.grad.cpu().numpy() - bwd()).max() <= 1e-5
        else:
            close_grad(xt.grad.cpu().numpy(), bwd(), "%s %s" % (name, shape))


@pytest.mark.parametrize("shape", _shapes(2, 16, 24, 500))
def test_lovasz_and_relabelling(pl, shape):
    n, c, m = shape
    x, y = seg_inputs(300 + n * c * m, (n, c, m), 255, 0.1)
    xt, yt = dev(x).requires_grad_(), dev(y)
    losses = pl.LovaszSoftmaxFunctionV3.apply(xt, yt, 255)
    want, want_jacc = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    assert np.abs(losses.detach().cpu().numpy() - want).max() <= 1e-5 * max(1e-30, np.abs(want).max())
    n_min = max(1, y.size // 8)
    got = pl.score_ohem_label(xt.detach(), yt, 255, 0.4, n_min).cpu().numpy()
    scores = oracle.ohem_scores(x, y, 255)
    # the selection is exact on given scores; scores themselves may differ in the last bit, so compare
    # wherever no score sits within 1e-6 of the threshold or of the n_min-th smallest score
    order = np.sort(scores.reshape(-1))
    cut = order[min(n_min, order.size) - 1]
    sure = (np.abs(scores - 0.4) > 1e-6) & (np.abs(scores - cut) > 1e-6)
    want_lab = oracle.ohem_score_label(x, y, 255, 0.4, n_min)
    assert np.array_equal(got[sure], want_lab[sure])
    onehot = pl.OnehotEncoder(c, lb_smooth=0.1, ignore_idx=255)(yt).cpu().numpy()
    assert np.array_equal(onehot, oracle.onehot(y, c, 0.1, 255))


@pytest.mark.parametrize("shape", _shapes(3, 24, 150, 400))
def test_layer_norm_taylor_softmax(pl, shape):
    x = synth.normal(400 + sum(shape), 1, shape, 0.2, 1.5)
    g = synth.normal(401, 2, shape, 0.0, 1.0)
    xt = dev(x).requires_grad_()
    out = pl.LayerNormV3Func.apply(xt, 1e-5)
    if shape[1] > 1:
        # fp32 carries x - mean to about one spacing of |x|, and the output multiplies that by
        # 1/sqrt(var + eps), which is large where the channels of a pixel nearly coincide
        rstd = 1.0 / np.sqrt(x.astype(np.float64).var(axis=1) + 1e-5)
        bound = 1e-5 + 2.4e-7 * np.abs(x).max() * rstd.max()
        assert np.abs(out.detach().cpu().numpy() - oracle.layer_norm_forward(x.astype(np.float64), 1e-5)).max() <= bound
    out.backward(dev(g))
    want = oracle.layer_norm_backward(g.astype(np.float64), x.astype(np.float64), 1e-5)
    assert np.abs(xt.grad.cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max() + 1e-12
    for use_log, mod in ((False, pl.TaylorSoftmaxV3(dim=1, n=2)), (True, pl.LogTaylorSoftmaxV3(dim=1, n=2))):
        xt = dev(x).requires_grad_()
        out = mod(xt)
        want = oracle.taylor_forward(x.astype(np.float64), 1, 2, use_log)
        assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
        out.backward(dev(g))
        want_g = oracle.taylor_backward(g.astype(np.float64), x.astype(np.float64), 1, 2, use_log)
        assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * max(1.0, np.abs(want_g).max())


@pytest.mark.parametrize("shape", _shapes(4, 16, 12, 3000))
def test_elementwise_ops(pl, shape):
    x = synth.normal(500 + sum(shape), 1, shape, -1.0, 1.5)
    y = synth.bernoulli(501, 2, shape, 0.25).astype(np.float32)
    go = synth.normal(502, 3, shape, 0.0, 1.0)
    xt = dev(x).requires_grad_()
    out = pl.FocalSigmoidLossFuncV3.apply(xt, dev(y), 0.25, 2)
    close_loss(out.detach().cpu().numpy(), oracle.focal_forward(x, y, 0.25, 2), "focal %s" % (shape,))
    out.backward(dev(go))
    close_grad(xt.grad.cpu().numpy(), oracle.focal_backward(x, y, 0.25, 2, go), "focal %s" % (shape,))
    rows = x.reshape(shape[0], -1)
    xt = dev(rows).requires_grad_()
    loss = pl.SoftDiceLossV3Func.apply(xt, dev(y.reshape(shape[0], -1)), 2, 0.5)
    want, stats = oracle.soft_dice_forward(rows.astype(np.float64), y.reshape(shape[0], -1).astype(np.float64), 2, 0.5)
    assert np.abs(loss.detach().cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max() + 1e-7
    gr = synth.normal(503, 4, (shape[0],), 0.5, 1.0)
    loss.backward(dev(gr))
    want_g = oracle.soft_dice_backward(gr.astype(np.float64), rows.astype(np.float64),
                                       y.reshape(shape[0], -1).astype(np.float64), stats, 2)
    assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * np.abs(want_g).max() + 1e-12


@pytest.mark.parametrize("shape", _shapes(7, 24, 48, 5000))
def test_one_pass_fb_modules_match_the_two_pass_modules(pl, shape):
    """LSR, large margin and focal with fb=True ('mean' and 'sum', an upstream scalar of 1 and another one) against
    the same modules with fb=False, which the tests above hold to the oracle."""
    n, c, m = shape
    x, y = seg_inputs(300 + n * c * m, (n, c, m), 255, 0.1)
    yt = dev(y)
    soft = dev((synth.uniform01(301, 4, x.size).reshape(x.shape) < 0.2).astype(np.float32))
    for name, make, labels in (
            ("lsr", lambda fb, r: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=r, ignore_index=255, fb=fb), yt),
            ("lmargin", lambda fb, r: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=r, ignore_index=255, fb=fb), yt),
            ("focal", lambda fb, r: pl.FocalLossV3(alpha=0.25, gamma=2, reduction=r, fb=fb), soft)):
        if c == 1 and name == "lmargin":
            continue
        for reduction, factor in (("mean", 1.0), ("sum", 1.0), ("mean", 0.3)):
            got = []
            for fb in (True, False):
                xt = dev(x).requires_grad_()
                loss = make(fb, reduction)(xt, labels)
                (loss * factor if factor != 1.0 else loss).backward()
                got.append((float(loss.detach()), xt.grad))
            (la, ga), (lb, gb) = got
            what = "%s %s %s x%g" % (name, shape, reduction, factor)
            if np.isnan(lb):
                assert np.isnan(la), what          # nothing valid under 'mean'
            else:
                assert abs(la - lb) <= 1e-6 * abs(lb) + 1e-7, what
            # (one class: every gradient is an exact 0 and what either side leaves is rounding)
            assert (ga - gb).abs().max().item() <= 2e-6 * gb.abs().max().item() + (1e-7 if c == 1 else 1e-12), what
