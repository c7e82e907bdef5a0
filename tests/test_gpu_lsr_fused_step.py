"""LabelSmoothSoftmaxCEV3(fb=True) with 'mean' / 'sum': loss and gradient from one pass over the logits
(plh_lsr_forward_backward_reduced), the backward a multiplication that is skipped for an upstream gradient of 1
(plh_scale_unless_one) - against the oracle and against the module that recomputes in backward."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

# register-resident shapes (two pixels per lane, one pixel per lane on odd planes, the per-image form on long odd
# planes, rows of up to 32 classes) run the one pass; the others (33 channels and more, long rows) run the forward and
# the backward one after the other behind the same entry point
SHAPES = [(2, 19, 32, 40), (3, 7, 13, 11), (1, 12, 65, 67), (300, 10), (1, 32, 16, 16), (5, 1, 4, 4),
          (70, 200), (9, 3000), (2, 40, 16, 24), (2, 150, 16, 24), (1, 300, 9, 7)]
DTYPES = [(torch.float32, 2e-6), (torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)]


@pytest.fixture(scope="module")
def mod():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def inputs(seed, shape, dtype, ignore_frac=0.1):
    x = synth.normal(seed, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(seed, shape[:1] + shape[2:], shape[1], 255, ignore_frac)
    xt = torch.from_numpy(x).cuda().to(dtype)
    return xt.float().cpu().numpy(), y, xt, torch.from_numpy(y).cuda()


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_one_pass_step_matches_the_oracle_and_the_recomputing_module(mod, shape, dtype, tol, reduction):
    x, y, xt, yt = inputs(321, shape, dtype)
    y.reshape(-1)[::53] = shape[1] + 2                        # labels without a target channel, not ignored
    yt = torch.from_numpy(y).cuda()
    n_valid = int((y != 255).sum())
    losses = oracle.lsr_forward(x.astype(np.float64), y, 255, 0.1)
    want_loss = losses.sum() / (n_valid if reduction == "mean" else 1)
    up = np.full(y.shape, 1.0 / n_valid if reduction == "mean" else 1.0)
    want_grad = oracle.lsr_backward(x.astype(np.float64), y, 255, 0.1, up)

    a = xt.clone().requires_grad_(True)
    loss = mod.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=reduction, ignore_index=255, fb=True)(a, yt)
    loss.backward()
    b = xt.clone().requires_grad_(True)
    loss_b = mod.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=reduction, ignore_index=255, fb=False)(b, yt)
    loss_b.backward()

    la, lb = float(loss.detach()), float(loss_b.detach())
    assert loss.dtype == loss_b.dtype and a.grad.dtype == dtype
    assert abs(la - want_loss) <= max(4 * tol, 2e-6) * abs(want_loss) + 1e-6         # one channel: the loss is an exact 0
    scale = np.abs(want_grad).max()
    assert np.abs(a.grad.float().cpu().numpy() - want_grad).max() <= tol * scale
    assert abs(la - lb) <= 1e-6 * abs(lb) + (0 if dtype == torch.float32 else tol * abs(lb))
    assert (a.grad.float() - b.grad.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * scale
    ign = torch.from_numpy(y == 255).cuda().unsqueeze(1).expand_as(a.grad)
    if ign.any():
        assert a.grad[ign].abs().max().item() == 0            # ignored pixels: exact zeros


def test_the_one_pass_loss_is_the_forward_kernels_loss_bit_for_bit(mod):
    from pytorch_loss import _native
    x, y, xt, yt = inputs(322, (2, 19, 64, 64), torch.float32)
    for mean in (True, False):
        loss, grad, tag = _native.lsr_forward_backward_reduced(xt, yt, 255, 0.1, mean)
        loss2, n_valid = _native.lsr_forward_reduced(xt, yt, 255, 0.1, mean)
        assert loss.cpu().numpy().tobytes() == loss2.cpu().numpy().tobytes() and tag == 0
        want = _native.lsr_backward_scaled(xt, yt, 255, 0.1, torch.ones((), device="cuda"), n_valid if mean else None)
        assert torch.equal(grad, want)


@pytest.mark.parametrize("dtype,tol", [DTYPES[0], DTYPES[2]], ids=["f32", "bf16"])
@pytest.mark.parametrize("factor", [0.4, 1024.0, -1.0, 1.0])
def test_an_upstream_gradient_other_than_one_scales_the_kept_gradient(mod, dtype, tol, factor):
    x, y, xt, yt = inputs(323, (2, 19, 33, 31), dtype)
    a = xt.clone().requires_grad_(True)
    (mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(a, yt) * factor).backward()
    b = xt.clone().requires_grad_(True)
    (mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=False)(b, yt) * factor).backward()
    ref = b.grad.float()
    assert (a.grad.float() - ref).abs().max().item() <= max(tol, 1e-6) * 2 * ref.abs().max().item()


def test_nothing_valid_no_gradient_wanted_and_a_second_backward(mod):
    x = torch.randn(2, 5, 8, 8, device="cuda", requires_grad=True)
    y = torch.full((2, 8, 8), 255, device="cuda", dtype=torch.int64)
    loss = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(x, y)
    loss.backward()
    assert torch.isnan(loss) and x.grad.abs().max().item() == 0
    y = torch.randint(0, 5, (2, 8, 8), device="cuda")
    with torch.no_grad():
        plain = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(x, y)
    assert not plain.requires_grad
    assert torch.equal(plain, mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=False)(x.detach(), y))
    loss = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(x, y)
    loss.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="went to an earlier backward"):
        loss.backward()


def test_full_size_step(mod):
    """(8,19,1024,1024): loss and gradient against the recomputing module's."""
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn((8, 19, 1024, 1024), device="cuda", generator=g) * 2
    y = torch.randint(0, 19, (8, 1024, 1024), device="cuda", generator=g)
    y[torch.rand((8, 1024, 1024), device="cuda", generator=g) < 0.05] = 255
    a = x.clone().requires_grad_(True)
    la = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(a, y)
    la.backward()
    b = x.clone().requires_grad_(True)
    lb = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=False)(b, y)
    lb.backward()
    assert float(la.detach()) == float(lb.detach())
    assert torch.equal(a.grad, b.grad)


@pytest.mark.parametrize("shape", [(3, 7, 13, 11), (2, 19, 32, 40)], ids=str)
def test_labels_that_start_on_an_8_byte_boundary_only(mod, shape):
    """The count of valid labels reads 16-byte pairs where it can: a label view one element into its storage cannot."""
    x, y, xt, yt = inputs(324, shape, torch.float32)
    store = torch.empty(y.size + 1, dtype=torch.int64, device="cuda")
    lab = store[1:].view(y.shape)
    lab.copy_(yt)
    assert lab.data_ptr() % 16 == 8
    a = xt.clone().requires_grad_(True)
    la = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=True)(a, lab)
    la.backward()
    b = xt.clone().requires_grad_(True)
    lb = mod.LabelSmoothSoftmaxCEV3(ignore_index=255, fb=False)(b, yt)
    lb.backward()
    assert float(la.detach()) == float(lb.detach()) and torch.equal(a.grad, b.grad)
