"""GPU parity: the HIP path (through the C ABI, via the drop-in Python surface) against the CPU oracle.

Tolerances are the ones the scope states: loss within 1e-5 relative, gradients within
1e-5 max-abs in fp32, masks exact (zeros at ignored pixels are bit-exact zeros, the valid
count is an exact integer).  Because a 'mean' over millions of pixels makes the absolute
gradient bound vacuous, gradients are also held to a relative max-norm bound under unit
upstream gradient ('sum'/'none').
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-5
GRAD_REL = 2e-5      # max|got - want| / max|want|


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def close_loss(got, want, what=""):
    """Reduced losses (and the sum of unreduced ones): 1e-5 relative.  Single elements of an
    unreduced loss tensor: 1e-5 relative plus an absolute allowance of 1e-6 of the tensor's mean
    magnitude, because an element such as -|y-p|^g * ce near y == p is itself the result of a
    cancellation and no fp32 evaluation, the oracle's included, has a relative error bound there."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    if want.ndim == 0:
        assert abs(got - want) <= LOSS_RTOL * abs(want), "%s loss %r vs %r" % (what, got, want)
        return
    if want.size == 0:
        assert got.size == 0
        return
    floor = 1e-6 * np.abs(want).mean()
    err = np.abs(got - want) - (LOSS_RTOL * np.abs(want) + floor)
    assert np.all(err <= 0), "%s loss element err exceeds bound by %.3e" % (what, err.max())
    assert abs(got.sum() - want.sum()) <= LOSS_RTOL * np.abs(want).sum(), "%s summed loss" % what


def close_grad(got, want, what=""):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64)).max() if got.size else 0.0
    assert err <= GRAD_ATOL, "%s grad max-abs err %.3e" % (what, err)
    ref = np.abs(want).max() if want.size else 0.0
    if ref > 0:
        assert err / ref <= GRAD_REL, "%s grad rel err %.3e" % (what, err / ref)


SEG_CASES = [
    # (shape, ignore_index, ignore_frac)            execution shape
    ((2, 19, 64, 64), 255, 0.05),                   # 4 pixels per thread, channels in registers
    ((2, 19, 7, 9), 255, 0.1),                      # odd spatial size -> 1 pixel per thread
    ((3, 2, 5, 8), -100, 0.2),
    ((4, 32, 4, 4), 255, 0.0),
    ((2, 3, 1, 1), 255, 0.0),
    ((37, 10), -100, 0.1),                          # (N, C) classification input, C <= 32: a wavefront moves
    ((300, 19), 255, 0.1),                          #   its 64 rows through LDS; full and partly filled wavefronts,
    ((1000, 32), -100, 0.1),                        #   even and odd row lengths
    ((129, 2), 255, 0.2),
    ((33, 100), -100, 0.1),                         # (N, C): one wavefront per row
    ((5, 1000), 255, 0.3),
    ((9, 77), -100, 0.1),                           # ... rows of 33..2048 channels sit in a wavefront's registers:
    ((6, 501), 255, 0.2),                           #   2 .. 32 steps, element by element for odd lengths (in pieces of
    ((7, 201), 255, 0.1),                           #   8, 4 or 2 bytes when only those divide a row's bytes),
    ((70, 33), -100, 0.1),                          #   rows of up to 256 channels: four rows per wavefront,
    ((21, 136), 255, 0.1),                          #   the last wavefront partly filled
    ((3, 256), 255, 0.0),
    ((5, 260), 255, 0.2),
    ((9, 264), 255, 0.1),                           #   16-bit rows of 257..512 elements in whole chunks: 16 lanes too
    ((6, 512), -100, 0.1),
    ((5, 200), 255, 0.1),                           #   short rows in whole chunks that end inside a 128-byte line
    ((7, 301), 255, 0.1),                           #   257..512 elements in short pieces: 16 lanes, 32 single elements,
    ((5, 258), -100, 0.1),                          #   16 pieces of two, 8 of four (16-bit 300 and 500)
    ((4, 500), 255, 0.1),
    ((4, 1001), -100, 0.1),
    ((3, 2047), 255, 0.1),                          #   16-byte chunks otherwise
    ((2, 2048), 255, 0.0),
    ((7, 150), 255, 0.1),                           #   lengths that are a multiple of 2 but not of 4 (and of 4 but not of 8):
    ((5, 34), -100, 0.1),                           #   pieces of two fp32 elements, of two or four 16-bit ones
    ((3, 1002), 255, 0.1),
    ((4, 2046), -100, 0.0),
    ((6, 300), 255, 0.1),
    ((9, 151), 255, 0.1),                           #   129..160 elements in short pieces: 5 steps of two, 10 of one
    ((5, 130), -100, 0.1),
    ((7, 143), 255, 0.1),
    ((2, 2049), -100, 0.0),                         # one channel more: staged or swept rows
    ((4, 3000), -100, 0.1),                         # 16-bit rows in whole chunks stay in a wavefront's registers up to
    ((3, 4096), 255, 0.1),                          #   4096 elements (8 steps of 8); fp32 rows take a block per row
    ((3, 4100), 255, 0.0),                          # row longer than the LDS staging buffer
    ((5, 4104), 255, 0.2),                          # ... a multiple of 8 elements: 16-byte chunks for 16-bit rows too
    ((2, 4099), -100, 0.0),                         # ... an odd length: element by element
    ((3, 50000), 255, 0.3),                         # a vocabulary
    ((2, 60000), 255, 0.0),                         #   one whose 16-bit rows exceed the 256-thread blocks' 112 KiB as well
    ((2, 33, 6, 7), 255, 0.2),                      # deep channel dim in NCHW: one lane per pixel
    ((2, 227, 5, 5), 255, 0.1),
    ((1, 64, 2, 3, 4), 0, 0.3),                     # 5-D input, ignore_index inside the class range
    ((2, 33, 9, 8), -100, 0.2),                     # 33..256 channels, 64 pixels or more per image: the channels of
    ((2, 40, 16, 16), 255, 0.1),                    #   a pixel are shared out over the 8 wavefronts of a block;
    ((3, 100, 10, 10), 255, 0.1),                   #   slots per wavefront 8 .. 32, last wavefronts partly or
    ((1, 150, 12, 16), 255, 0.05),                  #   wholly empty, pixel counts that leave lanes idle
    ((2, 256, 8, 8), 255, 0.1),
    ((2, 52, 8, 8), 255, 0.1),                      #   more channel counts of real label sets: the last
    ((2, 65, 8, 8), 255, 0.1),                      #   wavefront that holds channels holds 1 .. all of its slots
    ((1, 73, 8, 16), -100, 0.1),
    ((1, 112, 8, 8), 255, 0.1),
    ((1, 133, 8, 8), 255, 0.1),
    ((1, 171, 8, 8), 255, 0.1),
    ((1, 200, 8, 8), 255, 0.1),
    ((2, 257, 8, 8), 255, 0.1),                     # 257..512 channels: the same with up to 64 slots per wavefront
    ((1, 300, 9, 8), 255, 0.1),                     #   and half the pixels per lane (LSR, large-margin); slot counts
    ((2, 321, 8, 8), -100, 0.2),                    #   40, 48, 56, 64, last wavefronts partly or wholly empty,
    ((1, 400, 8, 9), 255, 0.1),                     #   pixel counts that leave lanes idle
    ((1, 449, 8, 8), 255, 0.1),
    ((1, 512, 8, 8), 255, 0.1),
    ((1, 513, 8, 8), 255, 0.1),                     # one channel more: a lane per pixel
    ((2, 19, 65, 65), 255, 0.05),                   # fp32 planes of odd length, 4096 pixels or more: tiles per
    ((3, 5, 71, 61), -100, 0.1),                    #   image, 4 pixels per lane; the last lane of an image holds
    ((2, 24, 4097, 1), 255, 0.1),                   #   1 or 3 pixels; the widest slice that takes this form,
    ((1, 25, 65, 65), 255, 0.1),                    #   one channel more and one pixel fewer than its limits
    ((2, 24, 63, 65), 255, 0.1),
    ((2, 32, 65, 65), 255, 0.1),                    # 16-bit slices take that form up to 32 channels (8-byte accesses
    ((1, 29, 67, 63), -100, 0.1),                   #   on 2-byte boundaries); fp32 keeps one pixel per lane here
    ((2, 150, 65, 65), 255, 0.05),                  # 33..256 channels on planes of odd length, 4096 pixels or more: the
    ((1, 33, 67, 63), -100, 0.1),                   #   split shape in tiles per image; the last lane of an image holds
    ((2, 256, 4097, 1), 255, 0.1),                  #   1, 2 or 3 pixels; both ends of the channel range
    ((3, 60, 65, 63), 255, 0.1),
    ((2, 100, 65, 65), -100, 0.1),                  #   97..160 channels: four fp32 pixels per lane in the LSR kernels
    ((1, 160, 71, 61), 255, 0.1),
    ((1, 257, 65, 65), 255, 0.1),                   #   one channel more: a lane per pixel
    ((2, 19, 66, 66), 255, 0.1),                    # planes of even length that do not start on 128-byte lines take
    ((2, 60, 66, 66), -100, 0.1),                   #   the tiles-per-image forms as well (4356 pixels: 17424 or 8712 bytes)
    ((1, 28, 66, 66), 255, 0.1),                    #   ... but not where that form does not reach (28 channels in fp32)
    ((2, 19, 16, 16), 255, 1.0),                    # everything ignored
]


def seg_inputs(seed, shape, ignore, frac):
    n_cls = shape[1]
    x = synth.normal(seed, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(seed, shape[:1] + shape[2:], n_cls, ignore, frac)
    if ignore == 0 and frac < 1.0:
        y[y == 0] = 1 if n_cls > 1 else 0
        y[synth.bernoulli(seed, 12, y.shape, frac)] = 0
    return x, y


# ------------------------------------------------------------------ LSR ----

@pytest.mark.parametrize("shape,ignore,frac", SEG_CASES)
def test_lsr_function_matches_oracle(pl, shape, ignore, frac):
    x, y = seg_inputs(21, shape, ignore, frac)
    xt = dev(x).requires_grad_()
    yt = dev(y)
    losses = pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, ignore)
    want = oracle.lsr_forward(x, y, ignore, 0.1)
    assert losses.shape == yt.shape and losses.dtype == torch.float32
    close_loss(losses.detach().cpu().numpy(), want, "lsr")
    assert (losses.detach().cpu().numpy()[y == ignore] == 0).all()
    go = synth.normal(5, 3, y.shape, 0.0, 1.0)
    losses.backward(dev(go))
    close_grad(xt.grad.cpu().numpy(), oracle.lsr_backward(x, y, ignore, 0.1, go), "lsr")
    g = xt.grad.cpu().numpy()
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
@pytest.mark.parametrize("smooth", [0.0, 0.1, 0.4])
def test_lsr_module_reductions(pl, reduction, smooth):
    x, y = seg_inputs(22, (2, 19, 32, 32), 255, 0.05)
    xt = dev(x).requires_grad_()
    crit = pl.LabelSmoothSoftmaxCEV3(lb_smooth=smooth, reduction=reduction, ignore_index=255)
    out = crit(xt, dev(y))
    per = oracle.lsr_forward(x, y, 255, smooth)
    want = oracle.reduce_pixels(per, y, reduction, 255)
    close_loss(out.detach().cpu().numpy(), want, "lsr " + reduction)
    (out.sum() if reduction == "none" else out).backward()
    scale = 1.0 / (y != 255).sum() if reduction == "mean" else 1.0
    want_g = oracle.lsr_backward(x, y, 255, smooth, np.float32(scale))
    close_grad(xt.grad.cpu().numpy(), want_g, "lsr " + reduction)
    assert np.abs(xt.grad.sum(dim=1).cpu().numpy()).max() < 1e-5     # gradient rows sum to zero


@pytest.mark.parametrize("shape,ignore,frac", SEG_CASES)
@pytest.mark.parametrize("kind", ["lsr", "lmargin"])
def test_fused_reductions_on_every_execution_shape(pl, kind, shape, ignore, frac):
    """'mean' / 'sum' come from per-block partials inside the forward kernel: every launch shape
    (registers, wavefront per row, lane per pixel, ragged tails) must agree with the unreduced path."""
    x, y = seg_inputs(25, shape, ignore, frac)
    yt = dev(y)
    if frac >= 1.0:
        # every pixel ignored: 'sum' is an exact 0 with an exactly zero gradient, 'mean' is 0 / 0 = NaN, as in the
        # reference's modules (pytorch_loss/label_smooth.py:169-170, pytorch_loss/large_margin_softmax.py:170-171)
        assert int((y != ignore).sum()) == 0
        for red in ("sum", "mean"):
            crit = (pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=ignore) if kind == "lsr"
                    else pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=ignore))
            xt = dev(x).requires_grad_()
            out = crit(xt, yt)
            if red == "sum":
                assert out.item() == 0.0
                out.backward()
                assert xt.grad.abs().max().item() == 0.0
            else:
                assert torch.isnan(out).item()
        return
    if kind == "lsr":
        make = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=ignore)
        per = oracle.lsr_forward(x.astype(np.float64), y, ignore, 0.1)
        grad_of = lambda g: oracle.lsr_backward(x, y, ignore, 0.1, g)
    else:
        make = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=ignore)
        per = oracle.lmargin_forward(x.astype(np.float64), y, 0.3, ignore)
        grad_of = lambda g: oracle.lmargin_backward(x, y, 0.3, ignore, g)
    n_valid = int((y != ignore).sum())
    for red in ("sum", "mean"):
        xt = dev(x).requires_grad_()
        out = make(red)(xt, yt)
        assert out.dim() == 0
        want = per.sum() / (n_valid if red == "mean" else 1)
        assert abs(out.item() - want) <= 1e-5 * abs(want), (red, out.item(), want)
        (out * 3.0).backward()                      # a non-unit upstream scalar
        scale = 3.0 / (n_valid if red == "mean" else 1)
        close_grad(xt.grad.cpu().numpy(), grad_of(np.float32(scale)), kind + " " + red)


def test_lsr_all_ignored_mean_is_nan(pl):
    x, y = seg_inputs(23, (2, 19, 8, 8), 255, 1.0)
    out = pl.LabelSmoothSoftmaxCEV3(ignore_index=255)(dev(x), dev(y))
    assert torch.isnan(out).item()


def test_lsr_default_ignore_index_and_noncontiguous(pl):
    x = synth.normal(24, 1, (2, 8, 8, 19), 0.0, 2.0)      # channels-last storage
    xt = dev(x).permute(0, 3, 1, 2)                       # logical (2, 19, 8, 8), non-contiguous
    y = synth.randint(24, 11, (2, 8, 8), 0, 19)
    y[0, 0, :3] = -100
    out = pl.LabelSmoothSoftmaxCEV3()(xt, dev(y))
    per = oracle.lsr_forward(np.ascontiguousarray(x.transpose(0, 3, 1, 2)), y, -100, 0.1)
    close_loss(out.item(), oracle.reduce_pixels(per, y, "mean", -100), "lsr nc")


# ---------------------------------------------------------------- focal ----

FOCAL_SHAPES = [(2, 8, 16, 16), (17, 3, 15, 13), (5,), (1, 1, 1, 3), (3, 1025)]


@pytest.mark.parametrize("shape", FOCAL_SHAPES)
@pytest.mark.parametrize("alpha,gamma", [(0.25, 2), (0.5, 1), (0.75, 3.0), (0.3, 0.5), (0.25, 2.5), (0.25, 0)])
@pytest.mark.parametrize("soft", [False, True])
def test_focal_functions_match_oracle(pl, shape, alpha, gamma, soft):
    x = synth.normal(31, 1, shape, -2.0, 1.5)
    if soft:
        y = synth.uniform01(31, 2, int(np.prod(shape))).reshape(shape).astype(np.float32)
    else:
        y = synth.bernoulli(31, 2, shape, 0.2).astype(np.float32)
    want_l = oracle.focal_forward(x, y, alpha, gamma)
    go = synth.normal(6, 3, shape, 0.0, 1.0)
    want_g = oracle.focal_backward(x, y, alpha, gamma, go)
    # |y-p|^gamma with gamma < 1 is not Lipschitz at y == p (its derivative is singular there):
    # with soft labels, compare only where the function is well conditioned
    well = np.ones(shape, dtype=bool)
    if soft and gamma < 1:
        well = np.abs(y - 1.0 / (1.0 + np.exp(-x.astype(np.float64)))) > 1e-2
    for fn in (pl.FocalSigmoidLossFuncV3, pl.FocalSigmoidLossFuncV3FB):
        xt = dev(x).requires_grad_()
        loss = fn.apply(xt, dev(y), alpha, gamma)
        close_loss(loss.detach().cpu().numpy()[well], want_l[well], fn.__name__)
        loss.backward(dev(go))
        close_grad(xt.grad.cpu().numpy()[well], want_g[well], fn.__name__)


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_focal_module_reductions(pl, reduction):
    w = synth.workload("cfg3", scale=0.25, batch=2)
    x, y = w["logits"], w["labels"]
    xt = dev(x).requires_grad_()
    out = pl.FocalLossV3(alpha=0.25, gamma=2, reduction=reduction)(xt, dev(y))
    per = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, 2.0)
    close_loss(out.detach().cpu().numpy(), oracle.reduce_all(per, reduction), "focal " + reduction)
    (out.sum() if reduction == "none" else out).backward()
    scale = 1.0 / x.size if reduction == "mean" else 1.0
    close_grad(xt.grad.cpu().numpy(), oracle.focal_backward(x, y, 0.25, 2.0, np.float32(scale)), "focal " + reduction)


@pytest.mark.parametrize("shape", FOCAL_SHAPES)
@pytest.mark.parametrize("gamma", [2, 1, 1.5])
def test_focal_fused_reductions(pl, shape, gamma):
    x = synth.normal(32, 1, shape, -2.0, 1.5)
    y = synth.bernoulli(32, 2, shape, 0.2).astype(np.float32)
    per = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, gamma)
    for red in ("sum", "mean"):
        xt = dev(x).requires_grad_()
        out = pl.FocalLossV3(alpha=0.25, gamma=gamma, reduction=red)(xt, dev(y))
        want = per.sum() / (x.size if red == "mean" else 1)
        assert abs(out.item() - want) <= 1e-5 * abs(want)
        (out * -2.0).backward()
        scale = -2.0 / (x.size if red == "mean" else 1)
        close_grad(xt.grad.cpu().numpy(), oracle.focal_backward(x, y, 0.25, gamma, np.float32(scale)), "focal " + red)


def test_focal_extreme_logits_stay_finite(pl):
    x = np.array([-120.0, -90.0, -60.0, -30.0, 0.0, 30.0, 60.0, 90.0, 120.0] * 2, dtype=np.float32)
    y = np.array([0.0] * 9 + [1.0] * 9, dtype=np.float32)
    xt = dev(x).requires_grad_()
    loss = pl.FocalSigmoidLossFuncV3.apply(xt, dev(y), 0.25, 2)
    loss.sum().backward()
    got, g = loss.detach().cpu().numpy(), xt.grad.cpu().numpy()
    assert np.isfinite(got).all() and np.isfinite(g).all()
    close_loss(got, oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, 2.0), "focal extreme")


# -------------------------------------------------------------- lmargin ----

@pytest.mark.parametrize("shape,ignore,frac", SEG_CASES)
@pytest.mark.parametrize("fb", [False, True])
def test_lmargin_functions_match_oracle(pl, shape, ignore, frac, fb):
    if shape[1] < 2:
        pytest.skip("needs at least two classes")
    x, y = seg_inputs(41, shape, ignore, frac)
    xt = dev(x).requires_grad_()
    yt = dev(y)
    if fb:
        losses, cnt = pl.LargeMarginSoftmaxFuncV3FB.apply(xt, yt, 0.3, ignore)
        assert cnt.dtype == torch.int64 and cnt.item() == int((y != ignore).sum())
    else:
        losses = pl.LargeMarginSoftmaxFuncV3.apply(xt, yt, 0.3, ignore)
    want = oracle.lmargin_forward(x, y, 0.3, ignore)
    close_loss(losses.detach().cpu().numpy(), want, "lmargin")
    assert (losses.detach().cpu().numpy()[y == ignore] == 0).all()
    go = synth.normal(7, 3, y.shape, 0.0, 1.0)
    losses.backward(dev(go))
    g = xt.grad.cpu().numpy()
    close_grad(g, oracle.lmargin_backward(x, y, 0.3, ignore, go), "lmargin")
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
@pytest.mark.parametrize("fb", [False, True])
@pytest.mark.parametrize("lam", [0.0, 0.3, 1.0])
def test_lmargin_module_reductions(pl, reduction, fb, lam):
    x, y = seg_inputs(42, (2, 19, 32, 32), 255, 0.05)
    xt = dev(x).requires_grad_()
    out = pl.LargeMarginSoftmaxV3(lam=lam, reduction=reduction, ignore_index=255, fb=fb)(xt, dev(y))
    per = oracle.lmargin_forward(x, y, lam, 255)
    close_loss(out.detach().cpu().numpy(), oracle.reduce_pixels(per, y, reduction, 255), "lmargin " + reduction)
    (out.sum() if reduction == "none" else out).backward()
    scale = 1.0 / (y != 255).sum() if reduction == "mean" else 1.0
    close_grad(xt.grad.cpu().numpy(), oracle.lmargin_backward(x, y, lam, 255, np.float32(scale)), "lmargin")


def test_lmargin_dominant_target_stays_finite(pl):
    x = np.zeros((1, 4, 1, 4), dtype=np.float32)
    x[0, 2] = 200.0
    x[0, 0, 0, 1] = -150.0
    y = np.full((1, 1, 4), 2, dtype=np.int64)
    for fb in (False, True):
        xt = dev(x).requires_grad_()
        out = pl.LargeMarginSoftmaxV3(reduction="none", fb=fb)(xt, dev(y))
        out.sum().backward()
        assert torch.isfinite(out).all() and torch.isfinite(xt.grad).all()
        close_loss(out.detach().cpu().numpy(), oracle.lmargin_forward(x.astype(np.float64), y, 0.3, 255), "dominant")


# --------------------------------------------------------------- lovasz ----

LOVASZ_CASES = [
    ((2, 19, 64, 64), 255, 0.05),
    ((2, 19, 7, 9), 255, 0.1),
    ((3, 2, 5, 8), -100, 0.2),
    ((1, 4, 70, 64), 255, 0.0),       # a little over one sort tile per class
    ((2, 5, 100, 100), 255, 0.3),     # several tiles, last one ragged
    ((37, 10), -100, 0.1),
    ((2, 33, 6, 7), 255, 0.2),
    ((2, 227, 5, 5), 255, 0.1),
    ((1, 8, 4, 4), 0, 0.3),
    ((2, 19, 16, 16), 255, 1.0),
]


@pytest.mark.parametrize("shape,ignore,frac", LOVASZ_CASES)
def test_lovasz_function_matches_oracle(pl, shape, ignore, frac):
    x, y = seg_inputs(51, shape, ignore, frac)
    xt = dev(x).requires_grad_()
    losses = pl.LovaszSoftmaxFunctionV3.apply(xt, dev(y), ignore)
    want, want_jacc = oracle.lovasz_forward(x.astype(np.float64), y, ignore)
    assert losses.shape == (shape[1],)
    got = losses.detach().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-5 * max(1e-30, np.abs(want).max()), np.abs(got - want).max()
    w = synth.normal(8, 3, (shape[1],), 0.5, 1.0)
    losses.backward(dev(w))
    g = xt.grad.cpu().numpy()
    want_g = oracle.lovasz_backward(w.astype(np.float64), x.astype(np.float64), y, want_jacc, ignore)
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()
    # near-ties may be ordered differently in fp32 and fp64; that moves single Jaccard
    # differences between neighbouring pixels, bounded by the largest difference in the class
    err = np.abs(g - want_g)
    assert np.median(err) <= 1e-6
    assert err.max() <= max(GRAD_ATOL, 2.0 * np.abs(want_jacc).max() * np.abs(w).max() * 1e-3), err.max()


def test_lovasz_jacc_is_exact_for_the_computed_order(pl):
    """Sort, scan and Jaccard differences are integer/rank work: given the fp32 errors the GPU
    itself computed, the saved differences must equal the fp32 CPU restatement bit for bit."""
    from pytorch_loss import _native
    x, y = seg_inputs(52, (2, 5, 100, 100), 255, 0.2)
    losses, jacc = _native.lovasz_forward(dev(x), dev(y), 255)
    jacc = jacc.cpu().numpy()
    l32, j32 = oracle.lovasz_forward(x, y, 255)
    same = (jacc.view(np.uint32) == j32.view(np.uint32)).mean()
    assert same > 0.995, same                       # the rest: 1-ulp differences in expf reorder near-ties
    assert (jacc[:, y.reshape(-1) == 255] == 0).all()
    np.testing.assert_allclose(jacc.sum(axis=1), 1.0, rtol=1e-4)
    # the fp32 restatement sums 16k products serially; hold the loss to the fp64 one instead
    l64, _ = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(losses.cpu().numpy(), l64, rtol=1e-5)
    np.testing.assert_allclose(l32, l64, rtol=1e-4)


def test_lovasz_errors_spread_over_many_binades(pl):
    """Logits of a saturated model: errors from 1e-30 to 1, some exactly 0 (softmax rounds to 1), so
    nothing can be left out of the sort and the top digit takes dozens of values per wavefront."""
    from pytorch_loss import _native
    x, y = seg_inputs(57, (2, 19, 128, 128), 255, 0.05)
    x = (x * 8.0).astype(np.float32)
    losses, jacc = _native.lovasz_forward(dev(x), dev(y), 255)
    jacc = jacc.cpu().numpy()
    l64, _ = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(losses.cpu().numpy(), l64, rtol=1e-5)
    _, j32 = oracle.lovasz_forward(x, y, 255)
    assert (jacc.view(np.uint32) == j32.view(np.uint32)).mean() > 0.99
    np.testing.assert_allclose(jacc.sum(axis=1), 1.0, rtol=1e-4)
    assert (jacc[:, y.reshape(-1) == 255] == 0).all()


@pytest.mark.parametrize("case", ["confident", "one_positive", "absent_and_present", "ties_at_the_limit"])
def test_lovasz_keys_left_out_of_the_sort_get_exact_zeros(pl, case):
    """The kernels sort only the keys that can have a non-zero Jaccard difference (those not ranked
    after the class's last positive).  What they leave out must come back as exact zeros, and what
    they keep must match the oracle, which sorts everything."""
    from pytorch_loss import _native
    shape = (2, 6, 96, 96)
    x, y = seg_inputs(53, shape, 255, 0.1)
    if case == "confident":                      # a trained model: the label's logit dominates
        onehot = (np.arange(shape[1])[None, :, None, None] == np.where(y == 255, 0, y)[:, None]).astype(np.float32)
        x = (x * 0.5 + 6.0 * onehot).astype(np.float32)
    elif case == "one_positive":                 # class 5 has a single, well classified pixel
        y[y == 5] = 4
        y[0, 3, 7] = 5
        x[0, 5, 3, 7] = 9.0
    elif case == "absent_and_present":           # classes 4 and 5 never occur
        y[(y == 4) | (y == 5)] = 1
    elif case == "ties_at_the_limit":            # identical pixels: every error is tied with the last positive's
        x[:] = x[0:1, :, 0:1, 0:1]
    losses, jacc = _native.lovasz_forward(dev(x), dev(y), 255)
    jacc = jacc.cpu().numpy()
    l64, j64 = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    _, j32 = oracle.lovasz_forward(x, y, 255)
    np.testing.assert_allclose(losses.cpu().numpy(), l64, rtol=1e-5, atol=1e-7)
    # wherever the oracle's difference is an exact zero the kernel's must be too, and vice versa
    # (up to near-tie reorderings, which never cross the zero / non-zero boundary by more than a pixel)
    assert ((jacc == 0) != (j32 == 0)).mean() < 1e-3
    if case != "ties_at_the_limit":              # with all-equal errors the order is pixel order in both
        same = (jacc.view(np.uint32) == j32.view(np.uint32)).mean()
        assert same > 0.99, same
    else:
        assert np.array_equal(jacc.view(np.uint32), j32.view(np.uint32))
    np.testing.assert_allclose(jacc.sum(axis=1), 1.0, rtol=1e-4)
    if case == "confident":
        assert (jacc == 0).mean() > 0.15          # a good part of the keys was not sorted at all
    # gradient through the public surface
    xt = dev(x).requires_grad_()
    out = pl.LovaszSoftmaxV3(reduction="mean", ignore_index=255)(xt, dev(y))
    out.backward()
    want_g = oracle.lovasz_backward(np.full(shape[1], 1.0 / shape[1]), x.astype(np.float64), y, j64, 255)
    err = np.abs(xt.grad.cpu().numpy() - want_g)
    assert np.median(err) <= 1e-7 and err.max() <= max(GRAD_ATOL, 2e-3 * np.abs(j64).max() / shape[1]), err.max()


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_lovasz_module_reductions(pl, reduction):
    w = synth.workload("cfg5", scale=1 / 16, batch=2)
    x, y = w["logits"], w["labels"]
    xt = dev(x).requires_grad_()
    out = pl.LovaszSoftmaxV3(reduction=reduction, ignore_index=255)(xt, dev(y))
    per, jacc = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    want = oracle.reduce_all(per, reduction)
    got = out.detach().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    (out.sum() if reduction == "none" else out).backward()
    scale = 1.0 / 19 if reduction == "mean" else 1.0
    want_g = oracle.lovasz_backward(np.full(19, scale), x.astype(np.float64), y, jacc, 255)
    err = np.abs(xt.grad.cpu().numpy() - want_g)
    assert err.max() <= GRAD_ATOL and np.median(err) <= 1e-7


def test_lovasz_limits_raise(pl):
    x = torch.zeros(1, 512, 2, 2, device="cuda")
    y = torch.zeros(1, 2, 2, dtype=torch.long, device="cuda")
    with pytest.raises(RuntimeError, match="num of classes"):
        pl.LovaszSoftmaxV3()(x, y)


# ------------------------------------------------ shared surface behaviour ----

def test_empty_inputs_return_empty(pl):
    x = torch.zeros(0, 19, 4, 4, device="cuda", requires_grad=True)
    y = torch.zeros(0, 4, 4, dtype=torch.long, device="cuda")
    assert pl.LSRCrossEntropyFunctionV3.apply(x, y, 0.1, 255).numel() == 0
    assert pl.LargeMarginSoftmaxFuncV3.apply(x, y, 0.3, 255).numel() == 0
    assert pl.FocalSigmoidLossFuncV3.apply(x, x.detach(), 0.25, 2).numel() == 0


def test_half_and_double_inputs_are_computed_in_fp32(pl):
    x, y = seg_inputs(61, (2, 19, 8, 8), 255, 0.1)
    for dt in (torch.float16, torch.bfloat16, torch.float64):
        xt = dev(x).to(dt).requires_grad_()
        out = pl.LabelSmoothSoftmaxCEV3(ignore_index=255)(xt, dev(y))
        out.backward()
        assert xt.grad.dtype == dt and out.dtype == dt
        xr = xt.detach().float().cpu().numpy()
        per = oracle.lsr_forward(xr, y, 255, 0.1)
        assert abs(out.item() - oracle.reduce_pixels(per, y, "mean", 255)) < 2e-2


def test_autocast_casts_to_fp32(pl):
    x, y = seg_inputs(62, (2, 19, 8, 8), 255, 0.1)
    xt = dev(x).half().requires_grad_()
    with torch.autocast("cuda", dtype=torch.float16):
        out = pl.LabelSmoothSoftmaxCEV3(ignore_index=255)(xt, dev(y))
    assert out.dtype == torch.float32
    out.backward()
    assert xt.grad.dtype == torch.float16


def test_runs_on_a_side_stream(pl):
    x, y = seg_inputs(63, (2, 19, 64, 64), 255, 0.05)
    xt, yt = dev(x), dev(y)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out = pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, 255)
    side.synchronize()
    close_loss(out.cpu().numpy(), oracle.lsr_forward(x, y, 255, 0.1), "side stream")


@pytest.mark.parametrize("n_cls,masked", [(5000, 4200), (40000, 33000), (3001, 1500)])
def test_rows_with_masked_vocabulary_entries_stay_finite(pl, n_cls, masked):
    """(N, C) rows of more than 2048 logits whose leading entries are -inf (a masked vocabulary): whole
    16-byte chunks of -inf reach a lane before its first finite value. Cross entropy (smoothing 0), its
    gradient and the OHEM scores stay finite and match the oracle, as for the shorter row shapes (the
    smoothed loss itself is 0 * inf = NaN there in the reference's arithmetic too)."""
    from pytorch_loss import _native
    x = synth.normal(77, 1, (6, n_cls), 0.0, 2.0)
    x[:, :masked] = -np.inf
    x[1, masked:masked + 7] = -np.inf
    y = synth.randint(77, 11, (6,), masked + 7, n_cls)
    y[4] = 255
    xt, yt = dev(x), dev(y)
    # OhemCELoss with a threshold nothing exceeds: the mean cross entropy of the valid rows
    xr = xt.clone().requires_grad_()
    loss = pl.OhemCELoss(score_thresh=2.0, n_min=1, ignore_index=255)(xr, yt)
    x64 = x.astype(np.float64)
    keep = y != 255
    mx = x64.max(axis=1)
    lse = np.log(np.exp(x64 - mx[:, None]).sum(axis=1)) + mx
    want = (lse - x64[np.arange(6), np.where(keep, y, 0)])[keep].mean()
    close_loss(loss.item(), want, "masked rows, OhemCELoss")
    loss.backward()
    assert torch.isfinite(xr.grad).all()
    close_grad(xr.grad.cpu().numpy(), oracle.lsr_backward(x, y, 255, 0.0, np.float32(1.0 / keep.sum())), "masked rows, OhemCELoss")
    grad = _native.lsr_backward(xt, yt, 255, 0.0).cpu().numpy()
    assert np.isfinite(grad).all() and np.all(grad[:, :masked] == 0)
    close_grad(grad, oracle.lsr_backward(x, y, 255, 0.0), "masked rows")
    scores = _native.ohem_scores(xt, yt, 255).cpu().numpy()
    assert np.isfinite(scores).all()
    np.testing.assert_allclose(scores, oracle.ohem_scores(x, y, 255), rtol=2e-5, atol=1e-7)


@pytest.mark.parametrize("shape", [(6, 100), (5, 300), (9, 1000), (6, 150), (4, 5000)])
def test_large_margin_rows_with_a_masked_class(pl, shape):
    """A logit of -inf among the classes other than the target: that class has q = 0 and the margin term
    (0 - coeff) * log 0 = +inf (root large_margin_softmax.py:84-90, csrc/large_margin_kernel.cu:183-190). The
    forward-only kernels of the (N, C) shapes take the margin term in closed form; a row with a masked class must
    come out as it does from the kernels that also produce the gradient, and the rows around it must not notice."""
    x = synth.normal(91, 1, shape, 0.0, 2.0)
    y = synth.randint(91, 11, shape[:1], 0, shape[1])
    y[0] = 255
    masked_row = 2
    col = (int(y[masked_row]) + 3) % shape[1]
    x[masked_row, col] = -np.inf
    want = oracle.lmargin_forward(x.astype(np.float64), y, 0.3, 255)
    assert np.isposinf(want[masked_row]) and np.isfinite(np.delete(want, masked_row)).all()
    xt, yt = dev(x), dev(y)
    fwd = pl.LargeMarginSoftmaxFuncV3.apply(xt, yt, 0.3, 255).cpu().numpy()
    both = pl.LargeMarginSoftmaxFuncV3FB.apply(xt.clone().requires_grad_(), yt, 0.3, 255)[0].detach().cpu().numpy()
    for got, what in ((fwd, "forward"), (both, "forward+backward")):
        assert np.isposinf(got[masked_row]), (what, got[masked_row])
        close_loss(np.delete(got, masked_row), np.delete(want, masked_row), "masked class, " + what)


def _prototype_logits(seed, shape, n_proto):
    """Pixels draw their logit vector from a small set of prototypes. Pixels of one prototype get bit-equal
    errors on the GPU and in the oracle alike (exact ties, ordered by pixel index on both sides); errors of
    different prototypes are far apart, so no rounding difference can reorder them."""
    n, c = shape[0], shape[1]
    protos = synth.normal(seed, 5, (n_proto, c), 0.0, 2.0)
    which = synth.randint(seed, 6, (n,) + tuple(shape[2:]), 0, n_proto)
    x = np.moveaxis(protos[which], -1, 1)
    return np.ascontiguousarray(x, dtype=np.float32), which


def _errors_well_separated(x, y, ignore):
    """fp64: within every class, two distinct errors differ by more than ten times what fp32 rounding can
    move them by (relative 1e-6 for an error p, absolute 1e-6 for an error 1 - p)."""
    p = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    yy = y.reshape(-1)
    for c in range(x.shape[1]):
        pc = np.moveaxis(p, 1, 0)[c].reshape(-1)
        hot = (yy == c)[yy != ignore]
        e = np.where(yy == c, 1.0 - pc, pc)[yy != ignore]
        order = np.argsort(e, kind="stable")
        e, hot = e[order], hot[order]
        d = np.diff(e)
        tol = np.where(hot, 1e-5, 1e-5 * e)
        if np.any((d > 1e-12 * e[1:]) & (d <= tol[:-1] + tol[1:])):
            return False
    return True


@pytest.mark.parametrize("shape,n_proto", [((2, 19, 64, 64), 16), ((2, 19, 16, 16), 24), ((3, 5, 33, 17), 48)])
def test_lovasz_gradient_without_near_ties(pl, shape, n_proto):
    """Where no two distinct errors of a class come close, the fp32 order is the fp64 order and the gradient is
    held to 1e-5 max-abs, the bar the other losses meet (the looser bound of test_lovasz_function_matches_oracle
    applies only where near-ties exist)."""
    ignore = 255
    for seed in range(70, 100):
        x, which = _prototype_logits(seed, shape, n_proto)
        y = synth.seg_labels(seed, shape[:1] + shape[2:], shape[1], ignore, 0.05)
        ok = _errors_well_separated(x, y, ignore)
        if ok:
            break
    assert ok, "no seed in range gave well separated errors"
    xt = dev(x).requires_grad_()
    losses = pl.LovaszSoftmaxFunctionV3.apply(xt, dev(y), ignore)
    want, want_jacc = oracle.lovasz_forward(x.astype(np.float64), y, ignore)
    assert np.abs(losses.detach().cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max()
    w = synth.normal(8, 3, (shape[1],), 0.5, 1.0)
    losses.backward(dev(w))
    want_g = oracle.lovasz_backward(w.astype(np.float64), x.astype(np.float64), y, want_jacc, ignore)
    err = np.abs(xt.grad.cpu().numpy() - want_g).max()
    assert err <= GRAD_ATOL, err
    # and with the module's 'mean' over classes
    xt.grad = None
    pl.LovaszSoftmaxV3(reduction="mean", ignore_index=ignore)(xt, dev(y)).backward()
    want_g = oracle.lovasz_backward(np.full(shape[1], 1.0 / shape[1]), x.astype(np.float64), y, want_jacc, ignore)
    assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= GRAD_ATOL


def _one_rounding(got, want, dtype):
    """|got - want| within one rounding step of `dtype` at want's magnitude (plus a denormal-sized floor)."""
    eps = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    return np.all(np.abs(got - want) <= eps * np.abs(want) + 1e-7)


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("in_dtype", ["amp", torch.float32])
@pytest.mark.parametrize("op", ["lsr", "focal", "lmargin", "lovasz"])
def test_autocast_gives_fp32_losses_and_input_typed_gradients(pl, op, in_dtype, amp_dtype):
    """What custom_fwd(cast_inputs=torch.float32) / custom_bwd give in the reference
    (pytorch_loss/label_smooth.py:131,139): under autocast the loss is fp32 whatever the logits' type, the
    gradient comes back in the logits' type, and the values are those of the fp32 op on the widened inputs."""
    in_dtype = amp_dtype if in_dtype == "amp" else in_dtype
    if op == "focal":
        shape = (2, 8, 16, 16)
        x = synth.normal(64, 1, shape, -2.0, 1.5)
        y = synth.bernoulli(64, 2, shape, 0.2).astype(np.float32)
        yt = dev(y)                                            # fp32 labels next to 16-bit logits: both are widened
    else:
        x, y = seg_inputs(64, (2, 19, 16, 16), 255, 0.1)
        yt = dev(y)
    xt = dev(x).to(in_dtype).requires_grad_()
    xw = xt.detach().float().cpu().numpy()                     # the widened inputs the oracle sees
    crit = {"lsr": lambda: pl.LabelSmoothSoftmaxCEV3(ignore_index=255),
            "focal": lambda: pl.FocalLossV3(),
            "lmargin": lambda: pl.LargeMarginSoftmaxV3(ignore_index=255),
            "lovasz": lambda: pl.LovaszSoftmaxV3(ignore_index=255)}[op]()
    with torch.autocast("cuda", dtype=amp_dtype):
        out = crit(xt, yt)
        assert out.dtype == torch.float32
        out.backward()
    assert xt.grad.dtype == in_dtype
    n_valid = (y != 255).sum() if op != "focal" else y.size
    if op == "lsr":
        want = oracle.reduce_pixels(oracle.lsr_forward(xw.astype(np.float64), y, 255, 0.1), y, "mean", 255)
        want_g = oracle.lsr_backward(xw.astype(np.float64), y, 255, 0.1, 1.0 / n_valid)
    elif op == "lmargin":
        want = oracle.reduce_pixels(oracle.lmargin_forward(xw.astype(np.float64), y, 0.3, 255), y, "mean", 255)
        want_g = oracle.lmargin_backward(xw.astype(np.float64), y, 0.3, 255, 1.0 / n_valid)
    elif op == "focal":
        want = oracle.focal_forward(xw.astype(np.float64), y.astype(np.float64), 0.25, 2.0).mean()
        want_g = oracle.focal_backward(xw.astype(np.float64), y.astype(np.float64), 0.25, 2.0, 1.0 / y.size)
    else:
        l64, j64 = oracle.lovasz_forward(xw.astype(np.float64), y, 255)
        want = l64.mean()
        want_g = oracle.lovasz_backward(np.full(19, 1.0 / 19), xw.astype(np.float64), y, j64, 255)
    assert abs(out.item() - want) <= LOSS_RTOL * abs(want), (op, out.item(), want)
    got_g = xt.grad.float().cpu().numpy()
    if in_dtype == torch.float32:
        tol = GRAD_ATOL if op != "lovasz" else max(GRAD_ATOL, 2e-3 * np.abs(j64).max() / 19)
        assert np.abs(got_g - want_g).max() <= tol
    elif op == "lovasz":
        # near-ties may swap neighbours' Jaccard differences (see test_lovasz_function_matches_oracle)
        assert np.median(np.abs(got_g - want_g)) <= 1e-6
    else:
        assert _one_rounding(got_g, want_g, in_dtype)


@pytest.mark.parametrize("n_cls,scale,boost,passes", [(400, 0.002, 0.0, 2), (120, 0.3, 0.0, 3), (120, 1.0, 12.0, 4)])
def test_lovasz_sort_passes_follow_the_key_width(pl, n_cls, scale, boost, passes):
    """The sort looks only at the key bits below a class's limit: near-uniform predictions over many classes
    (best positive's error above 0.996: at most 16 key bits) take two passes, soft ones three, confident ones
    all four. Every plan against the fp32 restatement bit for bit, and the loss against the fp64 one."""
    from pytorch_loss import _native
    shape = (2, n_cls, 40, 50)
    y = synth.seg_labels(53, (2, 40, 50), n_cls, 255, 0.1)
    x = synth.normal(53, 1, shape, 0.0, scale)
    if boost:
        onehot = np.moveaxis(np.eye(n_cls, dtype=np.float32)[np.where(y == 255, 0, y)], -1, 1)
        x = x + np.float32(boost) * onehot
    # the number of passes each class with positives takes, from the key of its best classified positive
    p = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    need = []
    for c in range(n_cls):
        hot = (y == c)
        if hot.any():
            err = np.float32(1.0) - np.moveaxis(p, 1, 0)[c][hot].astype(np.float32)
            key = int(np.float32(1.0).view(np.uint32)) - int(np.float32(err.min()).view(np.uint32))
            width = max(1, key.bit_length())
            need.append(2 if width <= 16 else (3 if width <= 24 else 4))
    assert need.count(passes) > 0.9 * len(need), {k: need.count(k) for k in set(need)}
    losses, jacc = _native.lovasz_forward(dev(x), dev(y), 255)
    jacc = jacc.cpu().numpy()
    l32, j32 = oracle.lovasz_forward(x, y, 255)
    assert (jacc.view(np.uint32) == j32.view(np.uint32)).mean() > 0.995
    assert (jacc[:, y.reshape(-1) == 255] == 0).all()
    l64, _ = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    # confident predictions: a positive's error 1 - p with p = 0.9993 carries p's fp32 rounding 1400 times enlarged,
    # in the reference's fp32 kernels too; the loss, which those errors make up, inherits it
    np.testing.assert_allclose(losses.cpu().numpy(), l64, rtol=3e-4 if boost else 1e-5)
