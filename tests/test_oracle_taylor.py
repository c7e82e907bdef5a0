"""Pins the oracle's Taylor softmax WITHOUT the reference: the series against exact rational
arithmetic, outputs against the defining expression evaluated in torch fp64, the log form against
the plain one, convergence to the library softmax as the order grows, gradients against fp64
autograd of that expression and finite differences, and the cross entropy against F.nll_loss."""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import synth

SHAPES_DIMS = [((2, 5, 3, 4), 1), ((3, 7), 1), ((4, 6, 5), 0), ((2, 3, 4, 5), 3), ((2, 3, 4, 5), -2), ((6,), 0)]


def _series(x, order):
    return sum(x ** i / math.factorial(i) for i in range(order + 1))


def _defining(xt, dim, order, use_log):
    f = _series(xt, order)
    y = f / f.sum(dim=dim, keepdim=True)
    return y.log() if use_log else y


def test_series_against_exact_rationals():
    for order in (2, 4, 8):
        for num in (-7, -1, 0, 3, 11):
            x = Fraction(num, 4)
            exact = sum(x ** i / math.factorial(i) for i in range(order + 1))
            # one "row" holding x and 0: f(0) = 1, so out[0] = f(x) / (f(x) + 1)
            out = oracle.taylor_forward(np.array([[float(x), 0.0]]), 1, order, False)[0, 0]
            assert abs(out - float(exact / (exact + 1))) < 1e-14


@pytest.mark.parametrize("shape,dim", SHAPES_DIMS)
@pytest.mark.parametrize("order", [2, 4, 6])
@pytest.mark.parametrize("use_log", [False, True])
def test_forward_is_the_defining_expression(shape, dim, order, use_log):
    x = synth.normal(61, 1, shape, 0.0, 1.5, dtype=np.float64)
    got = oracle.taylor_forward(x, dim, order, use_log)
    want = _defining(torch.from_numpy(x), dim, order, use_log).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-13)
    plain = oracle.taylor_forward(x, dim, order, False)
    np.testing.assert_allclose(plain.sum(axis=dim), 1.0, rtol=1e-12)
    assert (plain > 0).all()                                   # even order: the polynomial is positive
    got32 = oracle.taylor_forward(x.astype(np.float32), dim, order, use_log)
    np.testing.assert_allclose(got32, want, rtol=2e-5, atol=2e-6)


def test_high_order_converges_to_the_library_softmax():
    x = synth.normal(62, 1, (3, 9, 4), 0.0, 1.0, dtype=np.float64)
    got = oracle.taylor_forward(x, 1, 30, False)
    np.testing.assert_allclose(got, torch.softmax(torch.from_numpy(x), 1).numpy(), rtol=1e-10)
    np.testing.assert_allclose(oracle.taylor_forward(x, 1, 30, True), torch.log_softmax(torch.from_numpy(x), 1).numpy(),
                               rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("shape,dim", SHAPES_DIMS)
@pytest.mark.parametrize("order", [2, 4])
@pytest.mark.parametrize("use_log", [False, True])
def test_backward_against_autograd_and_finite_differences(shape, dim, order, use_log):
    x = synth.normal(63, 1, shape, 0.0, 1.5, dtype=np.float64)
    g = synth.normal(63, 2, shape, 0.0, 1.0, dtype=np.float64)
    xt = torch.from_numpy(x).requires_grad_()
    _defining(xt, dim, order, use_log).backward(torch.from_numpy(g))
    got = oracle.taylor_backward(g, x, dim, order, use_log)
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-10, atol=1e-12)
    # central difference of sum(g * y) in one coordinate
    idx = tuple(s // 2 for s in shape)
    h = 1e-6
    xp, xm = x.copy(), x.copy()
    xp[idx] += h
    xm[idx] -= h
    fd = ((oracle.taylor_forward(xp, dim, order, use_log) - oracle.taylor_forward(xm, dim, order, use_log)) * g).sum() / (2 * h)
    assert abs(fd - got[idx]) < 1e-6 * max(1.0, abs(fd))


@pytest.mark.parametrize("order", [2, 4])
def test_cross_entropy_is_nll_of_the_log_form(order):
    shape = (2, 7, 5, 6)
    x = synth.normal(64, 1, shape, 0.0, 1.5, dtype=np.float64)
    y = synth.seg_labels(64, (2, 5, 6), 7, 255, 0.2)
    logp = _defining(torch.from_numpy(x).requires_grad_(), 1, order, True)
    per = F.nll_loss(logp, torch.from_numpy(y), ignore_index=255, reduction="none")
    np.testing.assert_allclose(oracle.taylor_ce(x, y, order, 255), per.detach().numpy(), rtol=1e-12, atol=1e-13)
    go = synth.normal(64, 3, y.shape, 0.0, 1.0, dtype=np.float64)
    xt = torch.from_numpy(x).requires_grad_()
    F.nll_loss(_defining(xt, 1, order, True), torch.from_numpy(y), ignore_index=255, reduction="none").backward(
        torch.from_numpy(go))
    np.testing.assert_allclose(oracle.taylor_ce_backward(x, y, order, 255, go), xt.grad.numpy(), rtol=1e-10, atol=1e-12)
