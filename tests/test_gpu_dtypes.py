"""GPU parity for fp16 / bf16 logits read and gradients written in their own type.

The kernels widen every element to fp32 on load, do all arithmetic in fp32 and narrow only the
gradient on store (the reference dispatches its kernels on the logits' scalar type and accumulates
in the type itself, csrc/lsr_kernel.cu:236-262; computing in fp32 is the stricter of the two).
So against the oracle evaluated on the widened inputs:
  - losses, which stay fp32 (taken under autocast, where the reference's
    custom_fwd(cast_inputs=float32) makes the op's outputs fp32), hold the fp32 bar of 1e-5;
  - gradients hold one rounding step of the storage type: |got - want| <= ulp(want) + 1e-7,
    i.e. 2^-10 relative for fp16 and 2^-7 for bf16.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth
from .test_gpu_parity import FOCAL_SHAPES, LOVASZ_CASES, SEG_CASES, close_loss, dev, seg_inputs

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.bfloat16]
ULP_REL = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def rounded(a, dt):
    """-> (tensor of type dt on the GPU, the same values widened back to a float32 numpy array)."""
    t = dev(a).to(dt)
    return t, t.float().cpu().numpy()


def close_grad_stored(got_t, want, dt, what=""):
    assert got_t.dtype == dt, (what, got_t.dtype)
    got = got_t.float().cpu().numpy().astype(np.float64)
    want = want.astype(np.float64)
    bound = ULP_REL[dt] * np.abs(want) + 1e-7
    err = np.abs(got - want) - bound
    assert np.all(err <= 0), "%s grad exceeds one storage rounding by %.3e" % (what, err.max())


@pytest.mark.parametrize("dt", DTYPES, ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape,ignore,frac", SEG_CASES)
@pytest.mark.parametrize("kind", ["lsr", "lmargin"])
def test_pixel_losses_native_16bit(pl, kind, shape, ignore, frac, dt):
    x, y = seg_inputs(71, shape, ignore, frac)
    xt, xr = rounded(x, dt)
    xt.requires_grad_()
    yt = dev(y)
    go = synth.normal(5, 3, y.shape, 0.0, 1.0)
    if kind == "lsr":
        apply = lambda: pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, ignore)
        want = oracle.lsr_forward(xr, y, ignore, 0.1)
        want_g = oracle.lsr_backward(xr, y, ignore, 0.1, go)
    else:
        apply = lambda: pl.LargeMarginSoftmaxFuncV3.apply(xt, yt, 0.3, ignore)
        want = oracle.lmargin_forward(xr, y, 0.3, ignore)
        want_g = oracle.lmargin_backward(xr, y, 0.3, ignore, go)
    with torch.autocast("cuda", dtype=dt):
        losses = apply()
    assert losses.dtype == torch.float32 and losses.shape == yt.shape
    close_loss(losses.detach().cpu().numpy(), want, kind)
    losses.backward(dev(go))
    close_grad_stored(xt.grad, want_g, dt, kind)
    g = xt.grad.float().cpu().numpy()
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()
    # outside autocast the losses come back in the logits' type, like the reference's
    plain = apply()
    assert plain.dtype == dt
    assert torch.equal(plain, losses.detach().to(dt))


@pytest.mark.parametrize("dt", DTYPES, ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape,ignore,frac", [c for c in SEG_CASES if c[2] < 1.0])
@pytest.mark.parametrize("kind", ["lsr", "lmargin"])
def test_fused_reductions_native_16bit(pl, kind, shape, ignore, frac, dt):
    x, y = seg_inputs(72, shape, ignore, frac)
    xt, xr = rounded(x, dt)
    yt = dev(y)
    if kind == "lsr":
        make = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=ignore)
        per = oracle.lsr_forward(xr.astype(np.float64), y, ignore, 0.1)
        grad_of = lambda g: oracle.lsr_backward(xr, y, ignore, 0.1, g)
    else:
        make = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=ignore)
        per = oracle.lmargin_forward(xr.astype(np.float64), y, 0.3, ignore)
        grad_of = lambda g: oracle.lmargin_backward(xr, y, 0.3, ignore, g)
    n_valid = int((y != ignore).sum())
    for red in ("sum", "mean"):
        leaf = xt.clone().requires_grad_()
        with torch.autocast("cuda", dtype=dt):
            out = make(red)(leaf, yt)
        assert out.dim() == 0 and out.dtype == torch.float32
        want = per.sum() / (n_valid if red == "mean" else 1)
        assert abs(out.item() - want) <= 1e-5 * abs(want), (red, out.item(), want)
        out.backward()
        close_grad_stored(leaf.grad, grad_of(np.float32(1.0 / (n_valid if red == "mean" else 1))), dt, kind + red)


@pytest.mark.parametrize("dt", DTYPES, ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", FOCAL_SHAPES)
@pytest.mark.parametrize("alpha,gamma", [(0.25, 2), (0.5, 1), (0.25, 2.5)])
@pytest.mark.parametrize("soft", [False, True])
def test_focal_native_16bit(pl, shape, alpha, gamma, soft, dt):
    x = synth.normal(33, 1, shape, -2.0, 1.5)
    if soft:
        y = synth.uniform01(33, 2, int(np.prod(shape))).reshape(shape).astype(np.float32)
    else:
        y = synth.bernoulli(33, 2, shape, 0.2).astype(np.float32)
    xt, xr = rounded(x, dt)
    yt, yr = rounded(y, dt)
    go = synth.normal(6, 3, shape, 0.0, 1.0)
    want_l = oracle.focal_forward(xr, yr, alpha, gamma)
    want_g = oracle.focal_backward(xr, yr, alpha, gamma, go)
    for fn in (pl.FocalSigmoidLossFuncV3, pl.FocalSigmoidLossFuncV3FB):
        leaf = xt.clone().requires_grad_()
        with torch.autocast("cuda", dtype=dt):
            loss = fn.apply(leaf, yt, alpha, gamma)
        assert loss.dtype == torch.float32
        close_loss(loss.detach().cpu().numpy(), want_l, fn.__name__)
        loss.backward(dev(go))
        close_grad_stored(leaf.grad, want_g, dt, fn.__name__)
    for red in ("mean", "sum"):
        leaf = xt.clone().requires_grad_()
        with torch.autocast("cuda", dtype=dt):
            out = pl.FocalLossV3(alpha=alpha, gamma=gamma, reduction=red)(leaf, yt)
        want = want_l.astype(np.float64).sum() / (want_l.size if red == "mean" else 1)
        assert abs(out.item() - want) <= 1e-5 * abs(want)
        out.backward()
        scale = np.float32(1.0 / (want_l.size if red == "mean" else 1))
        close_grad_stored(leaf.grad, oracle.focal_backward(xr, yr, alpha, gamma, scale), dt, "focal " + red)


def test_focal_mixed_types_take_the_fp32_path(pl):
    shape = (2, 5, 8, 8)
    x = synth.normal(34, 1, shape, -2.0, 1.5)
    y = synth.bernoulli(34, 2, shape, 0.2).astype(np.float32)
    xt, xr = rounded(x, torch.float16)
    xt.requires_grad_()
    loss = pl.FocalSigmoidLossFuncV3.apply(xt, dev(y), 0.25, 2)      # fp16 logits, fp32 labels
    assert loss.dtype == torch.float16
    want = oracle.focal_forward(xr, y, 0.25, 2)
    assert np.abs(loss.detach().float().cpu().numpy() - want).max() <= 2.0 ** -10 * np.abs(want).max() + 1e-7
    loss.sum().backward()
    close_grad_stored(xt.grad, oracle.focal_backward(xr, y, 0.25, 2, np.float32(1.0)), torch.float16, "mixed")


@pytest.mark.parametrize("dt", DTYPES, ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape,ignore,frac", LOVASZ_CASES)
def test_lovasz_native_16bit(pl, shape, ignore, frac, dt):
    x, y = seg_inputs(73, shape, ignore, frac)
    xt, xr = rounded(x, dt)
    xt.requires_grad_()
    with torch.autocast("cuda", dtype=dt):
        losses = pl.LovaszSoftmaxFunctionV3.apply(xt, dev(y), ignore)
    assert losses.dtype == torch.float32 and losses.shape == (shape[1],)
    want, want_jacc = oracle.lovasz_forward(xr.astype(np.float64), y, ignore)
    got = losses.detach().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-5 * max(1e-30, np.abs(want).max()), np.abs(got - want).max()
    w = synth.normal(8, 3, (shape[1],), 0.5, 1.0)
    losses.backward(dev(w))
    assert xt.grad.dtype == dt
    g = xt.grad.float().cpu().numpy()
    want_g = oracle.lovasz_backward(w.astype(np.float64), xr.astype(np.float64), y, want_jacc, ignore)
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()
    # 16-bit logits give many exactly tied errors; ties may be ordered differently in fp32 and
    # fp64, which moves single Jaccard differences between pixels of equal error: bounded by the
    # largest difference of the class, as in the fp32 test, plus the storage rounding
    err = np.abs(g - want_g)
    assert np.median(err) <= ULP_REL[dt] * np.abs(want_g).max() + 1e-6
    assert err.max() <= max(1e-5, 2.0 * np.abs(want_jacc).max() * np.abs(w).max() * 1e-3) \
        + ULP_REL[dt] * np.abs(want_g).max(), err.max()


def test_full_resolution_bf16_step_matches_fp32_step_on_the_same_values(pl):
    """At a size the oracle would take long on, use the fp32 kernels (held to the oracle by the
    other tests) as the checker: bf16 storage must not change anything but the final rounding."""
    x, y = seg_inputs(74, (2, 19, 512, 512), 255, 0.05)
    xt, xr = rounded(x, torch.bfloat16)
    yt = dev(y)
    a = xt.clone().requires_grad_()
    b = dev(xr).requires_grad_()
    for make in (lambda: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="sum", ignore_index=255),
                 lambda: pl.LargeMarginSoftmaxV3(lam=0.3, reduction="sum", ignore_index=255)):
        a.grad = b.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            la = make()(a, yt)
        lb = make()(b, yt)
        assert abs(la.item() - lb.item()) <= 1e-6 * abs(lb.item())
        la.backward()
        lb.backward()
        close_grad_stored(a.grad, b.grad.cpu().numpy(), torch.bfloat16, "full resolution")
        assert (a.grad == b.grad.to(torch.bfloat16)).float().mean().item() > 0.999
