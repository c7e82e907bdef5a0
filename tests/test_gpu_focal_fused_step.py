"""FocalLossV3(fb=True) with 'mean' / 'sum': loss and gradient from one pass over logits and labels
(plh_focal_forward_backward_reduced), the backward a multiplication that is skipped for an upstream gradient of 1
(plh_scale_unless_one) - against the oracle and against the module that recomputes in backward."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

# element counts that are and are not multiples of four (the vector kernel and the scalar tail)
SHAPES = [(2, 19, 32, 40), (3, 7, 13, 11), (1, 1, 5, 1), (16, 80, 32, 32), (4099,)]
DTYPES = [(torch.float32, 2e-6), (torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)]


@pytest.fixture(scope="module")
def mod():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def inputs(seed, shape, dtype, soft=False):
    x = synth.normal(seed, 1, shape, 0.0, 3.0)
    y = synth.uniform01(seed, 2, int(np.prod(shape))).reshape(shape) if soft else synth.bernoulli(seed, 2, shape, 0.1).astype(np.float32)
    xt = torch.from_numpy(x).cuda().to(dtype)
    yt = torch.from_numpy(np.ascontiguousarray(y, dtype=np.float32)).cuda().to(dtype)
    return xt.float().cpu().numpy(), yt.float().cpu().numpy(), xt, yt


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("gamma", [2, 1, 1.5])
@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_one_pass_step_matches_the_oracle_and_the_recomputing_module(mod, shape, dtype, tol, gamma, reduction):
    x, y, xt, yt = inputs(311, shape, dtype, soft=(gamma == 1.5))
    losses = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, gamma)
    div = x.size if reduction == "mean" else 1
    want_loss = losses.sum() / div
    want_grad = oracle.focal_backward(x.astype(np.float64), y.astype(np.float64), 0.25, gamma, np.float64(1.0 / div))

    a = xt.clone().requires_grad_(True)
    loss = mod.FocalLossV3(alpha=0.25, gamma=gamma, reduction=reduction, fb=True)(a, yt)
    loss.backward()
    b = xt.clone().requires_grad_(True)
    loss_b = mod.FocalLossV3(alpha=0.25, gamma=gamma, reduction=reduction, fb=False)(b, yt)
    loss_b.backward()

    la, lb = float(loss.detach()), float(loss_b.detach())
    assert loss.dtype == loss_b.dtype and a.grad.dtype == dtype
    if dtype == torch.float16 and abs(want_loss) > 6e4:      # the sum does not fit the fp16 the loss is returned in
        assert la == lb == float("inf")
    else:
        assert abs(la - want_loss) <= max(4 * tol, 4e-6) * abs(want_loss)
        assert abs(la - lb) <= 1e-6 * abs(lb) + (0 if dtype == torch.float32 else tol * abs(lb))
    scale = np.abs(want_grad).max()
    tiny = 6e-8 if dtype == torch.float16 else 0.0      # fp16 gradients of a mean over many elements are subnormal
    assert np.abs(a.grad.float().cpu().numpy() - want_grad).max() <= max(tol, 4e-6) * scale + tiny
    assert (a.grad.float() - b.grad.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * scale + tiny


@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("factor", [0.4, 1024.0, -1.0, 1.0])
def test_an_upstream_gradient_other_than_one_scales_the_kept_gradient(mod, dtype, tol, factor):
    x, y, xt, yt = inputs(312, (2, 19, 33, 31), dtype)
    a = xt.clone().requires_grad_(True)
    (mod.FocalLossV3(fb=True)(a, yt) * factor).backward()
    b = xt.clone().requires_grad_(True)
    (mod.FocalLossV3(fb=False)(b, yt) * factor).backward()
    ref = b.grad.float()
    assert (a.grad.float() - ref).abs().max().item() <= max(tol, 1e-6) * 2 * ref.abs().max().item()


def test_per_element_losses_and_other_dtypes(mod):
    x = torch.randn(2, 6, 4, 4, device="cuda", dtype=torch.float64, requires_grad=True)
    y = (torch.rand(2, 6, 4, 4, device="cuda") < 0.2).double()
    (mod.FocalLossV3(fb=True)(x, y) * 2.0).backward()
    z = x.detach().clone().requires_grad_(True)
    (mod.FocalLossV3(fb=False)(z, y) * 2.0).backward()
    assert x.grad.dtype == torch.float64 and (x.grad - z.grad).abs().max().item() <= 1e-6 * z.grad.abs().max().item()
    a = torch.randn(3, 5, 7, device="cuda", requires_grad=True)
    t = (torch.rand(3, 5, 7, device="cuda") < 0.2).float()
    w = torch.rand(3, 5, 7, device="cuda")
    la = mod.FocalLossV3(fb=True, reduction="none")(a, t)
    (la * w).sum().backward()
    b = a.detach().clone().requires_grad_(True)
    lb = mod.FocalLossV3(fb=False, reduction="none")(b, t)
    (lb * w).sum().backward()
    assert la.shape == a.shape and torch.equal(la, lb)
    assert (a.grad - b.grad).abs().max().item() <= 2e-6 * b.grad.abs().max().item()
    e = torch.zeros(0, 5, device="cuda", requires_grad=True)
    assert float(mod.FocalLossV3(fb=True, reduction="sum")(e, torch.zeros(0, 5, device="cuda")).detach()) == 0


def test_full_size_step(mod):
    """(16,80,128,128) and (8,19,1024,1024): loss and gradient against the recomputing module's."""
    for shape in [(16, 80, 128, 128), (8, 19, 1024, 1024)]:
        g = torch.Generator(device="cuda").manual_seed(6)
        x = torch.randn(shape, device="cuda", generator=g) * 3
        y = (torch.rand(shape, device="cuda", generator=g) < 0.02).float()
        a = x.clone().requires_grad_(True)
        la = mod.FocalLossV3(fb=True)(a, y)
        la.backward()
        b = x.clone().requires_grad_(True)
        lb = mod.FocalLossV3(fb=False)(b, y)
        lb.backward()
        assert abs(float(la.detach()) - float(lb.detach())) <= 1e-6 * abs(float(lb.detach()))
        assert (a.grad - b.grad).abs().max().item() <= 2e-6 * b.grad.abs().max().item()


def test_the_entry_point_on_fp16_logits(mod):
    """The module keeps fp16 logits on the two passes; the entry point itself takes them ('sum': nothing underflows)."""
    from pytorch_loss import _native
    x, y, xt, yt = inputs(313, (3, 7, 13, 11), torch.float16)
    loss, grad, tag = _native.focal_forward_backward_reduced(xt, yt, 2, 0.25, False)
    want_grad = oracle.focal_backward(x.astype(np.float64), y.astype(np.float64), 0.25, 2, np.float64(1.0))
    want_loss = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, 2).sum()
    assert tag == 1 and grad.dtype == torch.float16
    assert abs(float(loss) - want_loss) <= 4e-3 * abs(want_loss)
    assert np.abs(grad.float().cpu().numpy() - want_grad).max() <= 2e-3 * np.abs(want_grad).max()
