"""The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from
the fp64 oracle) against (a) the fp32 oracle, on CPU, and (b) the HIP path, on the GPU."""
import os
import sys

import numpy as np
import pytest
import torch

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

KINDS = ("lsr", "lmargin", "focal", "lovasz")


def load(kind):
    return np.load(os.path.join(HERE, "golden", kind + ".npz"), allow_pickle=False)


@pytest.mark.parametrize("kind", KINDS)
def test_inputs_regenerate_bit_identically(kind):
    g = load(kind)
    for tag, shape in (("small", make_golden.SMALL), ("cfg1", make_golden.CFG1)):
        x, y = make_golden.inputs(shape, kind)
        assert x.astype(np.float64).sum() == g[tag + "_input_checksum"]
        assert np.asarray(y, dtype=np.float64).sum() == g[tag + "_label_checksum"]


@pytest.mark.parametrize("kind", KINDS)
def test_fp32_oracle_against_golden(kind):
    g = load(kind)
    x, y = make_golden.inputs(make_golden.SMALL, kind)
    if kind == "lsr":
        per, grad = oracle.lsr_forward(x, y, 255, 0.1), oracle.lsr_backward(x, y, 255, 0.1)
    elif kind == "lmargin":
        per, grad = oracle.lmargin_forward(x, y, 0.3, 255), oracle.lmargin_backward(x, y, 0.3, 255)
    elif kind == "focal":
        per, grad = oracle.focal_forward(x, y, 0.25, 2.0), oracle.focal_backward(x, y, 0.25, 2.0)
    else:
        per, jacc = oracle.lovasz_forward(x, y, 255)
        grad = oracle.lovasz_backward(np.ones(19, dtype=np.float32), x, y, jacc, 255)
    np.testing.assert_allclose(per.sum(dtype=np.float64), g["small_sum"], rtol=1e-5)
    np.testing.assert_allclose(per, g["small_per"], rtol=2e-5, atol=1e-6 * np.abs(g["small_per"]).mean())
    if kind == "lovasz":   # near-ties order differently in fp32 and fp64
        assert np.median(np.abs(grad - g["small_grad"])) < 1e-7 and np.abs(grad - g["small_grad"]).max() < 5e-3
    else:
        assert np.abs(grad - g["small_grad"]).max() <= 1e-5


def _crit(pl, kind, reduction):
    if kind == "lsr":
        return pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=reduction, ignore_index=255)
    if kind == "lmargin":
        return pl.LargeMarginSoftmaxV3(lam=0.3, reduction=reduction, ignore_index=255)
    if kind == "focal":
        return pl.FocalLossV3(alpha=0.25, gamma=2, reduction=reduction)
    return pl.LovaszSoftmaxV3(reduction=reduction, ignore_index=255)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", KINDS)
def test_hip_path_against_golden(kind):
    import pytorch_loss as pl
    g = load(kind)
    # per-element outputs and gradients at the small shape
    x, y = make_golden.inputs(make_golden.SMALL, kind)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    per = _crit(pl, kind, "none")(xt, yt)
    got = per.detach().cpu().numpy()
    want = g["small_per"]
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6 * np.abs(want).mean())
    per.sum().backward()
    err = np.abs(xt.grad.cpu().numpy() - g["small_grad"])
    if kind == "lovasz":
        assert np.median(err) < 1e-7 and err.max() < 5e-3
    else:
        assert err.max() <= 1e-5
    # reduced losses at the CPU-runnable benchmark configuration
    x, y = make_golden.inputs(make_golden.CFG1, kind)
    xt = torch.from_numpy(x).cuda()
    yt = torch.from_numpy(y).cuda()
    for reduction in ("mean", "sum"):
        out = _crit(pl, kind, reduction)(xt, yt).item()
        want = float(g["cfg1_" + reduction])
        assert abs(out - want) <= 1e-5 * abs(want), (kind, reduction, out, want)
    if kind == "lovasz":
        per = _crit(pl, kind, "none")(xt, yt).cpu().numpy()
        np.testing.assert_allclose(per, g["cfg1_per"], rtol=1e-5)
