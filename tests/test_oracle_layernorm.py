"""Pins the oracle's layer norm WITHOUT the reference.

Forward: torch's own layer_norm over the channel dimension (a library routine) and closed-form
properties (zero mean, unit variance up to eps, shift invariance, scaling law).
Backward: the reference's kernel does not return the derivative of the forward, so autograd and
finite differences do not apply. What can be checked is agreement, up to the sign, with the second
place the reference states the same expression (pytorch_loss/layer_norm.py:104, written there with
sum(x) and a trailing 1/C), evaluated with torch ops; the sign follows csrc/layer_norm.cu:214.
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
