"""Pins the oracle's layer norm WITHOUT the reference.

Forward: torch's own layer_norm over the channel dimension (a library routine) and closed-form
properties (zero mean, unit variance up to eps, shift invariance, scaling law).
Backward: the reference's kernel does not return the derivative of the forward, so autograd and
finite differences do not apply. It is held by known answers worked by hand from
csrc/layer_norm.cu:214, by the closed forms that line collapses to on special inputs, and by
agreement, up to the sign, with the second place the reference states the same expression
(pytorch_loss/layer_norm.py:104, written there with sum(x) and a trailing 1/C), evaluated with
torch ops; the sign follows csrc/layer_norm.cu:214.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import synth


def _x(seed, shape, mean=0.5, std=2.0):
    return synth.normal(seed, 1, shape, mean, std, dtype=np.float64)


@pytest.mark.parametrize("shape", [(2, 19, 7), (1, 64, 33), (3, 5, 1), (2, 300, 4)])
@pytest.mark.parametrize("eps", [1e-6, 1e-2])
def test_forward_is_torch_layer_norm_over_channels(shape, eps):
    x = _x(81, shape)
    got = oracle.layer_norm_forward(x, eps)
    want = F.layer_norm(torch.from_numpy(x).permute(0, 2, 1), (shape[1],), eps=eps).permute(0, 2, 1).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-11, atol=1e-12)
    got32 = oracle.layer_norm_forward(x.astype(np.float32), eps)
    np.testing.assert_allclose(got32, want, rtol=0, atol=2e-6)


def test_forward_properties():
    x = _x(82, (2, 40, 9), mean=100.0, std=0.5)
    y = oracle.layer_norm_forward(x, 1e-6)
    assert np.abs(y.mean(axis=1)).max() < 1e-9
    var = x.var(axis=1, keepdims=True)
    np.testing.assert_allclose((y * y).mean(axis=1, keepdims=True), var / (var + 1e-6), rtol=1e-9)
    # adding a constant to every channel changes nothing; scaling by a turns eps into eps / a^2
    np.testing.assert_allclose(oracle.layer_norm_forward(x - 100.0, 1e-6), y, atol=1e-9)
    np.testing.assert_allclose(oracle.layer_norm_forward(3.0 * x, 9e-6), y, atol=1e-9)
    # fp32 with a large common offset: the centred form keeps its accuracy
    y32 = oracle.layer_norm_forward(x.astype(np.float32), 1e-6)
    assert np.abs(y32 - oracle.layer_norm_forward(x.astype(np.float32).astype(np.float64), 1e-6)).max() < 1e-4


@pytest.mark.parametrize("shape", [(2, 19, 7), (1, 64, 33), (2, 300, 4)])
def test_backward_agrees_with_the_second_statement_up_to_sign(shape):
    x = _x(83, shape)
    g = synth.normal(83, 2, shape, 0.0, 1.0, dtype=np.float64)
    eps = 1e-6
    xt, gt = torch.from_numpy(x), torch.from_numpy(g)
    C = shape[1]
    mean = xt.mean(dim=1, keepdim=True)
    var_plus_eps = xt.var(dim=1, keepdim=True, unbiased=False) + eps
    second = ((xt - mean) * (xt - 1 / C) * xt.sum(dim=1, keepdim=True) * var_plus_eps + 1) \
        * var_plus_eps.rsqrt() * (1. / C) * gt
    got = oracle.layer_norm_backward(g, x, eps)
    np.testing.assert_allclose(got, -second.numpy(), rtol=1e-10, atol=1e-12)
    # linear in the upstream gradient, and pixels do not interact
    np.testing.assert_allclose(oracle.layer_norm_backward(2.0 * g, x, eps), 2.0 * got, rtol=1e-12)
    x2 = x.copy()
    x2[:, :, 0] += 1.0
    got2 = oracle.layer_norm_backward(g, x2, eps)
    assert np.array_equal(got2[:, :, 1:], got[:, :, 1:]) and not np.array_equal(got2[:, :, 0], got[:, :, 0])


def test_backward_known_answers_worked_by_hand():
    """csrc/layer_norm.cu:212-216 gives, per pixel with m = mean(x), v = var(x) + eps, r = v^-1/2:
    res_j = -r * (1/C + (x_j - m) * (x_j - 1/C) * m * v) * g_j.
    The numbers below were worked out by hand from that line for inputs where every factor of it shows:
    a dropped term, a wrong sign, v where 1/v belongs, sum(x) for the mean, C for 1/C or a transposed
    index changes at least one of them."""
    bw = oracle.layer_norm_backward
    # C = 2, x = (1, 3): m = 2, var = 1.
    #   eps = 0: v = 1, r = 1:   res_0 = -(1/2 + (-1)(1/2)(2)(1)) g = +1/2 g,  res_1 = -(1/2 + (1)(5/2)(2)(1)) g = -11/2 g
    #   eps = 3: v = 4, r = 1/2: res_0 = -(1/2)(1/2 - 4) g = +7/4 g,           res_1 = -(1/2)(1/2 + 20) g = -41/4 g
    x = np.array([[[1.0], [3.0]]])
    g = np.array([[[2.0], [-1.0]]])
    np.testing.assert_allclose(bw(g, x, 0.0), np.array([[[0.5 * 2.0], [-5.5 * -1.0]]]), rtol=1e-15)
    np.testing.assert_allclose(bw(g, x, 3.0), np.array([[[1.75 * 2.0], [-10.25 * -1.0]]]), rtol=1e-15)
    # two pixels and two samples with different values: (N, C, M) = (2, 2, 2); pixel (n, m) holds channels (a, b)
    #   (0,0) = (1, 3) as above; (0,1) = (0, 2): m = 1, v = 1: res = -(1/2 + (-1)(-1/2)(1)) g = -g, -(1/2 + (1)(3/2)) g = -2 g
    #   (1,0) = (3, 1): the first pixel with its channels swapped: -11/2 g, +1/2 g
    #   (1,1) = (2, 2): constant, eps = 0 would divide by zero; with eps = 1/4: v = 1/4, r = 2: res = -2 (1/2) g = -g
    x = np.array([[[1.0, 0.0], [3.0, 2.0]], [[3.0, 2.0], [1.0, 2.0]]])
    g = np.ones_like(x)
    got = bw(g, x, 0.0)
    np.testing.assert_allclose(got[0], np.array([[0.5, -1.0], [-5.5, -2.0]]), rtol=1e-15)
    np.testing.assert_allclose(got[1, :, 0], np.array([-5.5, 0.5]), rtol=1e-15)
    np.testing.assert_allclose(bw(g, x, 0.25)[1, :, 1], np.array([-1.0, -1.0]), rtol=1e-15)


@pytest.mark.parametrize("C", [3, 19, 64])
def test_backward_closed_forms(C):
    """Special inputs on which the expression of csrc/layer_norm.cu:214 collapses to a closed form."""
    bw = oracle.layer_norm_backward
    eps = 1e-3
    g = synth.normal(84, 2, (2, C, 5), 0.0, 1.0, dtype=np.float64)
    # every channel equal to a: var = 0, v = eps, the second term vanishes: res = -g / (C sqrt(eps)) whatever a is
    for a in (0.0, 1.7, -40.0):
        np.testing.assert_allclose(bw(g, np.full((2, C, 5), a), eps), -g / (C * np.sqrt(eps)), rtol=1e-12)
    # a pixel whose channels add up to 0: the second term carries the mean as a factor, so res = -g / (C sqrt(var + eps))
    x = _x(85, (2, C, 5))
    x -= x.mean(axis=1, keepdims=True)
    want = -g / (C * np.sqrt(x.var(axis=1, keepdims=True) + eps))
    np.testing.assert_allclose(bw(g, x, eps), want, rtol=1e-9, atol=1e-12)
    # a channel that holds exactly 1/C, and one that holds exactly the pixel's mean, keep only the first term
    x = _x(86, (2, C, 5), mean=1.0)
    x[:, 0, :] = 1.0 / C
    x[:, 1, :] = (x[:, 0, :] + x[:, 2:, :].sum(axis=1)) / (C - 1)        # makes channel 1 the mean of all C channels
    r = 1.0 / np.sqrt(x.var(axis=1) + eps)
    got = bw(g, x, eps)
    np.testing.assert_allclose(got[:, 0, :], -r / C * g[:, 0, :], rtol=1e-9)
    np.testing.assert_allclose(got[:, 1, :], -r / C * g[:, 1, :], rtol=1e-7, atol=1e-9)
    assert np.abs(got[:, 2:, :] + (r / C)[:, None, :] * g[:, 2:, :]).max() > 1e-3      # the others do not
    # fp32 build of the oracle agrees with the fp64 one
    np.testing.assert_allclose(bw(g.astype(np.float32), x.astype(np.float32), eps), got, rtol=2e-4, atol=1e-5)
