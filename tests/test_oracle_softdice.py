"""Pins the oracle's soft dice loss WITHOUT the reference: the defining expression evaluated with
torch fp64 ops, its gradient by fp64 autograd and finite differences, and closed-form special cases
(perfect prediction, p = 1 reducing to 1 - (2|A.B| + s) / (|A| + |B| + s))."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth


def _inputs(seed, n, length, soft=False):
    x = synth.normal(seed, 1, (n, length), 0.0, 2.0, dtype=np.float64)
    if soft:
        y = synth.uniform01(seed, 2, n * length).reshape(n, length)
    else:
        y = synth.bernoulli(seed, 2, (n, length), 0.3).astype(np.float64)
    return x, y


def _defining(xt, yt, p, smooth):
    q = torch.sigmoid(xt)
    numer = 2 * (q * yt).sum(dim=1) + smooth
    denor = (q.pow(p) + yt).sum(dim=1) + smooth      # the label as it is (csrc/soft_dice_kernel_v2.cu:90)
    return 1.0 - numer / denor


def test_binary_labels_agree_with_the_power_form():
    """For labels in {0, 1} the fused kernel's q^p + y and the pure-torch classes' q^p + y^p
    (pytorch_loss/soft_dice_loss.py:35) are the same number; for soft labels with p != 1 they are not,
    and the oracle follows the kernel."""
    x, y = _inputs(74, 2, 300)
    q = 1 / (1 + np.exp(-x))
    for p in (1, 2, 2.5):
        want = 1 - (2 * (q * y).sum(1) + 1.0) / ((q ** p + y ** p).sum(1) + 1.0)
        np.testing.assert_allclose(oracle.soft_dice_forward(x, y, p, 1.0)[0], want, rtol=1e-12)
    xs, ys = _inputs(74, 2, 300, soft=True)
    qs = 1 / (1 + np.exp(-xs))
    kernel_form = 1 - (2 * (qs * ys).sum(1) + 1.0) / ((qs ** 2 + ys).sum(1) + 1.0)
    power_form = 1 - (2 * (qs * ys).sum(1) + 1.0) / ((qs ** 2 + ys ** 2).sum(1) + 1.0)
    got = oracle.soft_dice_forward(xs, ys, 2, 1.0)[0]
    np.testing.assert_allclose(got, kernel_form, rtol=1e-12)
    assert np.abs(got - power_form).min() > 1e-3


@pytest.mark.parametrize("n,length", [(1, 1000), (4, 37), (3, 4096)])
@pytest.mark.parametrize("p,smooth", [(1, 1.0), (2, 1.0), (1.5, 0.1), (3, 5.0)])
@pytest.mark.parametrize("soft", [False, True])
def test_forward_and_backward_against_autograd(n, length, p, smooth, soft):
    x, y = _inputs(71, n, length, soft)
    xt = torch.from_numpy(x).requires_grad_()
    want = _defining(xt, torch.from_numpy(y), p, smooth)
    losses, stats = oracle.soft_dice_forward(x, y, p, smooth)
    np.testing.assert_allclose(losses, want.detach().numpy(), rtol=1e-12, atol=1e-14)
    go = synth.normal(71, 3, (n,), 0.5, 1.0, dtype=np.float64)
    want.backward(torch.from_numpy(go))
    got = oracle.soft_dice_backward(go, x, y, stats, p)
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-9, atol=1e-14)
    l32, s32 = oracle.soft_dice_forward(x.astype(np.float32), y.astype(np.float32), p, smooth)
    np.testing.assert_allclose(l32, want.detach().numpy(), rtol=1e-5, atol=1e-6)


def test_finite_differences():
    x, y = _inputs(72, 2, 50)
    _, stats = oracle.soft_dice_forward(x, y, 2, 1.0)
    g = oracle.soft_dice_backward(np.ones(2), x, y, stats, 2)
    h = 1e-6
    for idx in [(0, 3), (1, 49)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        fd = (oracle.soft_dice_forward(xp, y, 2, 1.0)[0] - oracle.soft_dice_forward(xm, y, 2, 1.0)[0])[idx[0]] / (2 * h)
        assert abs(fd - g[idx]) < 1e-8


def test_closed_form_cases():
    y = synth.bernoulli(73, 2, (1, 500), 0.4).astype(np.float64)
    # saturated, correct prediction: q == y, so with p = 1 the loss is 1 - (2k + s) / (2k + s) = 0
    x = np.where(y > 0, 40.0, -40.0)
    losses, stats = oracle.soft_dice_forward(x, y, 1, 1.0)
    assert abs(losses[0]) < 1e-12 and abs(stats[0, 0] - (2 * y.sum() + 1)) < 1e-9
    # saturated, everything wrong: no overlap, loss = 1 - s / (N + s)
    losses, _ = oracle.soft_dice_forward(-x, y, 1, 1.0)
    assert abs(losses[0] - (1 - 1.0 / (500 + 1.0))) < 1e-12
    # p = 1: set sizes
    x2 = synth.normal(73, 1, (1, 500), 0.0, 2.0, dtype=np.float64)
    q = 1 / (1 + np.exp(-x2))
    losses, _ = oracle.soft_dice_forward(x2, y, 1, 0.5)
    assert abs(losses[0] - (1 - (2 * (q * y).sum() + 0.5) / (q.sum() + y.sum() + 0.5))) < 1e-12
