"""Taylor cross entropy on long (N, C) rows: the reduced forward leaves each row's sum of f
(plh_taylor_ce_forward_reduced_sums) and the backward forms the gradient from it elementwise over the flattened tensor
(plh_taylor_ce_backward_scaled_sums) - against the oracle and against the pair that recomputes the sum in backward."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

# rows whose lengths leave the 16-byte chunks of the flattened tensor straddling rows (2049, 3001, 4099), rows that do not
# (4096), a single row, and a tensor that ends in a partial chunk (3 x 2051 elements)
SHAPES = [(7, 2049), (5, 3001), (33, 4096), (3, 4099), (1, 5000), (3, 2051), (130, 2304),
          (300, 40), (130, 48), (40, 64), (90, 88), (6, 2040), (9, 1100), (5, 2048)]           # the last ones: rows that a wavefront holds in registers
SHAPES_FP32_ONLY = [(70, 200), (260, 300), (17, 1000), (1, 77), (9, 1024), (300, 33)]
DTYPES = [(torch.float32, 2e-6), (torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)]


@pytest.fixture(scope="module")
def mod():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def inputs(seed, shape, dtype, ignore_frac=0.2):
    x = synth.normal(seed, 1, shape, 0.0, 0.75)
    y = synth.seg_labels(seed, shape[:1], shape[1], 255, ignore_frac)
    xt = torch.from_numpy(x).cuda().to(dtype)
    return xt.float().cpu().numpy().astype(np.float64), y, xt, torch.from_numpy(y).cuda()


def test_the_predicate_names_long_rows_only(mod):
    from pytorch_loss import _native
    lib = _native.load()
    for tag in (0, 1, 2):
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 2049, 1) == 1
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 2048, 1) == 1 and lib.plh_taylor_ce_saves_sums(tag, 8, 1100, 1) == 1
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 1000, 1) == (1 if tag == 0 else 0)
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 512, 1) == 0 and lib.plh_taylor_ce_saves_sums(tag, 8, 32, 1) == 0
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 64, 1) == 1
        assert lib.plh_taylor_ce_saves_sums(tag, 8, 4000, 2) == 0 and lib.plh_taylor_ce_saves_sums(tag, 8, 19, 1024 * 1024) == 0
    assert lib.plh_taylor_ce_saves_sums(7, 8, 4000, 1) == 0


@pytest.mark.parametrize("order", [2, 4, 6])
@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_step_from_row_sums_matches_the_oracle(mod, shape, dtype, tol, reduction, order):
    check_step_from_row_sums(mod, shape, dtype, tol, reduction, order)


@pytest.mark.parametrize("order", [2, 4, 6])
@pytest.mark.parametrize("shape", SHAPES_FP32_ONLY, ids=str)
def test_rows_that_qualify_with_fp32_logits_only(mod, shape, order):
    check_step_from_row_sums(mod, shape, torch.float32, 2e-6, "mean", order)


def check_step_from_row_sums(mod, shape, dtype, tol, reduction, order):
    from pytorch_loss import _native
    x, y, xt, yt = inputs(401, shape, dtype)
    n_valid = int((y != 255).sum())
    want_loss = oracle.taylor_ce(x, y, order, 255).sum() / (n_valid if reduction == "mean" else 1)
    factor = 3.0
    want_grad = oracle.taylor_ce_backward(x, y, order, 255, factor / (n_valid if reduction == "mean" else 1))

    # the module takes this path for a scalar loss
    a = xt.clone().requires_grad_(True)
    loss = mod.TaylorCrossEntropyLossV3(n=order, ignore_index=255, reduction=reduction)(a, yt)
    (loss * factor).backward()
    assert abs(float(loss.detach()) - want_loss) <= max(tol, 1e-5) * abs(want_loss)
    scale = np.abs(want_grad).max()
    assert np.abs(a.grad.float().cpu().numpy() - want_grad).max() <= tol * scale
    ign = torch.from_numpy(y == 255).cuda().unsqueeze(1).expand_as(a.grad)
    assert a.grad[ign].abs().max().item() == 0 if ign.any() else True

    # the entry points themselves: sums are the rows' S, and the gradient equals the recomputing backward's
    args = _native.taylor_args(xt, yt)
    loss2, nv, sums = _native.taylor_ce_forward_reduced_sums(xt, yt, order, 255, reduction == "mean", args=args)
    assert sums is not None and sums.shape == (shape[0],)
    f = sum(x ** i / float(math.factorial(i)) for i in range(order + 1))
    assert np.abs(sums.cpu().numpy() - f.sum(1)).max() <= 1e-5 * np.abs(f.sum(1)).max()
    assert int(nv) == n_valid and torch.equal(loss2, loss.detach())
    up = torch.full((), factor, device="cuda")
    divide = nv if reduction == "mean" else None
    g_sums = _native.taylor_ce_backward_scaled_sums(sums, order, 255, up, divide, args)
    g_again = _native.taylor_ce_backward(None, None, order, 255, up, divide, args=args)
    assert g_sums.dtype == dtype
    assert (g_sums.float() - g_again.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * scale


def test_views_off_the_16_byte_grid_take_the_recomputing_backward(mod):
    """Logits that start 4 bytes into a 16-byte chunk: the sums are written but the backward sweeps its rows again."""
    shape = (6, 2500)
    x, y, xt, yt = inputs(402, shape, torch.float32)
    base = torch.zeros(shape[0] * shape[1] + 1, device="cuda")
    view = base[1:].view(shape)
    view.copy_(xt)
    a = view.detach().requires_grad_(True)
    assert a.data_ptr() % 16 == 4
    loss = mod.TaylorCrossEntropyLossV3(n=4, ignore_index=255)(a, yt)
    loss.backward()
    n_valid = int((y != 255).sum())
    want = oracle.taylor_ce_backward(x, y, 4, 255, 1.0 / n_valid)
    assert np.abs(a.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()


def test_rows_without_any_valid_label(mod):
    shape = (4, 3000)
    x, y, xt, yt = inputs(403, shape, torch.float32, ignore_frac=1.0)
    a = xt.clone().requires_grad_(True)
    loss = mod.TaylorCrossEntropyLossV3(n=2, ignore_index=255, reduction="sum")(a, yt)
    loss.backward()
    assert float(loss.detach()) == 0.0 and a.grad.abs().max().item() == 0.0


# Channel planes of odd length (crops), fp32, up to 24 channels: the per-image forward leaves S per pixel and the
# backward walks every plane in its own cache lines (taylor_ce_bwd_planes). The last shape has planes that end inside a
# tile's first line; (1, 24, 67, 67) the most channels the form takes.
CROPS = [(2, 19, 65, 67), (1, 24, 67, 67), (3, 5, 63, 66), (1, 1, 4097, 1), (2, 7, 1, 5001),
         (1, 33, 65, 67), (2, 150, 65, 65), (1, 256, 63, 67), (1, 40, 1, 9001),      # 33 .. 256 channels: the forward in tiles per image
         (1, 300, 65, 65), (1, 512, 63, 67)]                                       # 257 .. 512


@pytest.mark.parametrize("order", [2, 4, 6])
@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("shape", CROPS, ids=str)
def test_odd_crops_backward_from_the_pixels_sums(mod, shape, reduction, order):
    from pytorch_loss import _native
    lib = _native.load()
    n, c, m = shape[0], shape[1], shape[2] * shape[3]
    assert lib.plh_taylor_ce_saves_sums(0, n, c, m) == 1 and lib.plh_taylor_ce_saves_sums(2, n, c, m) == 0
    assert lib.plh_taylor_ce_saves_sums(0, n, c, (m + 31) // 32 * 32) == (1 if c > 256 else 0) and lib.plh_taylor_ce_saves_sums(0, n, 25, m) == 0
    assert lib.plh_taylor_ce_saves_sums(0, n, 32, m) == 0 and lib.plh_taylor_ce_saves_sums(0, n, 33, m) == 1 and lib.plh_taylor_ce_saves_sums(0, n, 513, m) == 0
    x = synth.normal(411, 1, shape, 0.0, 0.75).astype(np.float32)
    y = synth.seg_labels(411, shape[:1] + shape[2:], c, 255, 0.15)
    y[0, 0, :3] = c + 3                                  # labels out of range: no target, zero loss and gradient
    xt, yt = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    n_valid = int((y != 255).sum())
    x64 = x.astype(np.float64)
    factor = 0.5
    a = xt.clone().requires_grad_(True)
    loss = mod.TaylorCrossEntropyLossV3(n=order, ignore_index=255, reduction=reduction)(a, yt)
    (loss * factor).backward()
    b = xt.clone().requires_grad_(True)
    per = mod.TaylorCrossEntropyLossV3(n=order, ignore_index=255, reduction="none")(b, yt)
    want = per.sum() / (n_valid if reduction == "mean" else 1)
    (want * factor).backward()                          # the per-pixel path: the recomputing backward kernel
    assert abs(float(loss.detach()) - float(want.detach())) <= 1e-5 * abs(float(want.detach()))
    scale = b.grad.abs().max().item()
    up = factor / (n_valid if reduction == "mean" else 1)
    assert (a.grad - b.grad).abs().max().item() <= 2e-6 * scale + 1e-6 * up   # (one channel: the exact gradient is 0)
    ign = torch.from_numpy(y == 255).cuda().unsqueeze(1).expand_as(a.grad)
    assert a.grad[ign].abs().max().item() == 0
    # and against the oracle where every label is a class or ignored
    y2 = np.where(y >= c, 255, y)
    y2t = torch.from_numpy(y2).cuda()
    a2 = xt.clone().requires_grad_(True)
    loss2 = mod.TaylorCrossEntropyLossV3(n=order, ignore_index=255, reduction="sum")(a2, y2t)
    loss2.backward()
    want_g = oracle.taylor_ce_backward(x64, y2, order, 255, 1.0)
    assert abs(float(loss2.detach()) - oracle.taylor_ce(x64, y2, order, 255).sum()) <= 1e-5 * abs(float(loss2.detach()))
    assert np.abs(a2.grad.cpu().numpy() - want_g).max() <= 2e-6 * np.abs(want_g).max() + 1e-6


def test_odd_crops_on_views_at_another_offset_into_their_lines(mod):
    """Logits one element into their storage: logits and gradient sit at different offsets into a 128-byte line, and the
    recomputing backward runs (the forward's sums are not read)."""
    shape = (2, 19, 65, 67)
    x = synth.normal(412, 1, shape, 0.0, 0.75).astype(np.float32)
    y = synth.seg_labels(412, shape[:1] + shape[2:], shape[1], 255, 0.1)
    store = torch.empty(x.size + 1, device="cuda")
    xt = store[1:].view(shape)
    xt.copy_(torch.from_numpy(x))
    a = xt.requires_grad_(True)
    mod.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="sum")(a, torch.from_numpy(y).cuda()).backward()
    want = oracle.taylor_ce_backward(x.astype(np.float64), y, 4, 255, 1.0)
    assert np.abs(a.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()


def test_more_than_256_channels_on_aligned_planes(mod):
    """257 .. 512 channels take the pair whatever the planes' alignment (here 64 x 64: whole lines)."""
    from pytorch_loss import _native
    shape = (1, 300, 64, 64)
    assert _native.load().plh_taylor_ce_saves_sums(0, 1, 300, 4096) == 1
    x = synth.normal(413, 1, shape, 0.0, 0.75).astype(np.float32)
    y = synth.seg_labels(413, shape[:1] + shape[2:], shape[1], 255, 0.1)
    a = torch.from_numpy(x).cuda().requires_grad_(True)
    loss = mod.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="sum")(a, torch.from_numpy(y).cuda())
    loss.backward()
    x64 = x.astype(np.float64)
    assert abs(float(loss.detach()) - oracle.taylor_ce(x64, y, 4, 255).sum()) <= 1e-5 * abs(float(loss.detach()))
    want = oracle.taylor_ce_backward(x64, y, 4, 255, 1.0)
    assert np.abs(a.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
