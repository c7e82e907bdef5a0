"""LargeMarginSoftmaxV3(fb=True) with 'mean' / 'sum': loss and gradient from one pass over the logits
(plh_lmargin_forward_backward_reduced), the backward a multiplication that is skipped for an upstream gradient of 1
(plh_scale_unless_one) - against the oracle and against the module that recomputes in backward."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

# one shape per launch form of the fused kernel: register-resident (two pixels per lane, one pixel per lane on odd
# planes, the per-image form on long odd planes), rows (a wavefront per 64 rows, a wavefront per row, a block per row),
# and 33 channels and more in NCHW, where the entry point runs the forward and the backward one after the other (a lane
# per pixel on the short planes of 63 pixels)
SHAPES = [(2, 19, 32, 40), (3, 7, 13, 11), (1, 12, 65, 67), (300, 10), (70, 200), (9, 3000), (2, 40, 16, 24), (1, 2, 8, 8),
          (2, 150, 16, 24), (1, 300, 9, 7)]
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
    x, y, xt, yt = inputs(301, shape, dtype)
    n_valid = int((y != 255).sum())
    losses = oracle.lmargin_forward(x.astype(np.float64), y, 0.3, 255)
    want_loss = losses.sum() / (n_valid if reduction == "mean" else 1)
    up = np.full(y.shape, 1.0 / n_valid if reduction == "mean" else 1.0)
    want_grad = oracle.lmargin_backward(x.astype(np.float64), y, 0.3, 255, up)

    a = xt.clone().requires_grad_(True)
    loss = mod.LargeMarginSoftmaxV3(lam=0.3, reduction=reduction, ignore_index=255, fb=True)(a, yt)
    loss.backward()
    b = xt.clone().requires_grad_(True)
    loss_b = mod.LargeMarginSoftmaxV3(lam=0.3, reduction=reduction, ignore_index=255, fb=False)(b, yt)
    loss_b.backward()

    assert loss.dtype == loss_b.dtype and a.grad.dtype == dtype
    assert abs(float(loss.detach()) - want_loss) <= max(tol, 2e-6) * abs(want_loss) * (4 if dtype != torch.float32 else 1)
    scale = np.abs(want_grad).max()
    assert np.abs(a.grad.float().cpu().numpy() - want_grad).max() <= tol * scale
    # same arithmetic as the recomputing pair: equal to the last bits of fp32, to one rounding of the 16-bit types
    la, lb = float(loss.detach()), float(loss_b.detach())
    assert abs(la - lb) <= 1e-6 * abs(lb) + (0 if dtype == torch.float32 else tol * abs(lb))
    assert (a.grad.float() - b.grad.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * scale
    # ignored pixels: exact zeros
    ign = torch.from_numpy(y == 255).cuda().unsqueeze(1).expand_as(a.grad)
    assert a.grad[ign].abs().max().item() == 0 if ign.any() else True


@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("factor", [0.4, 1024.0, -1.0, 1.0])
def test_an_upstream_gradient_other_than_one_scales_the_kept_gradient(mod, dtype, tol, factor):
    shape = (2, 19, 33, 31)                     # 19 * 1023 elements per image: the scaling kernel's ragged end
    x, y, xt, yt = inputs(302, shape, dtype)
    a = xt.clone().requires_grad_(True)
    (mod.LargeMarginSoftmaxV3(fb=True)(a, yt) * factor).backward()
    b = xt.clone().requires_grad_(True)
    (mod.LargeMarginSoftmaxV3(fb=False)(b, yt) * factor).backward()
    ref = b.grad.float()
    assert (a.grad.float() - ref).abs().max().item() <= max(tol, 1e-6) * 2 * ref.abs().max().item()


def test_scale_unless_one_leaves_the_data_alone_for_one(mod):
    from pytorch_loss import _native
    for dtype, tag in [(torch.float32, 0), (torch.float16, 1), (torch.bfloat16, 2)]:
        for numel in [1, 7, 4096, 100003]:
            data = torch.randn(numel, device="cuda").to(dtype)
            data[0] = float("nan")                      # NaN * 1 would stay NaN anyway; -0.0 and denormals must not change either
            if numel > 1:
                data[1] = -0.0
            before = data.clone()
            _native.scale_unless_one(data, tag, torch.ones((), device="cuda"))
            assert data.view(torch.int16 if dtype != torch.float32 else torch.int32).equal(
                before.view(torch.int16 if dtype != torch.float32 else torch.int32))
            data = torch.randn(numel, device="cuda").to(dtype)
            want = (data.float() * 3.0).to(dtype)
            _native.scale_unless_one(data, tag, torch.full((), 3.0, device="cuda", dtype=torch.float64))
            assert data.equal(want)


def test_nothing_valid(mod):
    x = torch.randn(2, 5, 8, 8, device="cuda", requires_grad=True)
    y = torch.full((2, 8, 8), 255, device="cuda", dtype=torch.int64)
    loss = mod.LargeMarginSoftmaxV3(fb=True)(x, y)
    loss.backward()
    assert torch.isnan(loss) and x.grad.abs().max().item() == 0
    x.grad = None
    loss = mod.LargeMarginSoftmaxV3(fb=True, reduction="sum")(x, y)
    loss.backward()
    assert float(loss) == 0 and x.grad.abs().max().item() == 0


def test_other_dtypes_and_empty_input(mod):
    x = torch.randn(2, 6, 4, 4, device="cuda", dtype=torch.float64, requires_grad=True)
    y = torch.randint(0, 6, (2, 4, 4), device="cuda")
    (mod.LargeMarginSoftmaxV3(fb=True)(x, y) * 2.0).backward()
    z = x.detach().clone().requires_grad_(True)
    (mod.LargeMarginSoftmaxV3(fb=False)(z, y) * 2.0).backward()
    assert x.grad.dtype == torch.float64 and (x.grad - z.grad).abs().max().item() <= 1e-6 * z.grad.abs().max().item()
    e = torch.zeros(0, 5, 4, 4, device="cuda", requires_grad=True)
    out = mod.LargeMarginSoftmaxV3(fb=True, reduction="sum")(e, torch.zeros(0, 4, 4, device="cuda", dtype=torch.int64))
    assert float(out.detach()) == 0


def test_full_size_step(mod):
    """(8,19,1024,1024): loss against the recomputing module's, gradient against it on a strided sample."""
    shape = (8, 19, 1024, 1024)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(shape, device="cuda", generator=g) * 2
    y = torch.randint(0, 19, (8, 1024, 1024), device="cuda", generator=g)
    y[torch.rand((8, 1024, 1024), device="cuda", generator=g) < 0.05] = 255
    a = x.clone().requires_grad_(True)
    la = mod.LargeMarginSoftmaxV3(fb=True)(a, y)
    la.backward()
    b = x.clone().requires_grad_(True)
    lb = mod.LargeMarginSoftmaxV3(fb=False)(b, y)
    lb.backward()
    assert abs(float(la.detach()) - float(lb.detach())) <= 1e-6 * abs(float(lb.detach()))
    assert (a.grad - b.grad).abs().max().item() <= 2e-6 * b.grad.abs().max().item()


@pytest.mark.parametrize("shape", [(2, 19, 32, 40), (70, 200)], ids=str)
def test_the_entry_point_on_fp16_logits(mod, shape):
    """The module keeps fp16 logits on the two passes; the entry point itself takes them ('sum': nothing underflows)."""
    from pytorch_loss import _native
    x, y, xt, yt = inputs(303, shape, torch.float16)
    loss, grad, tag = _native.lmargin_forward_backward_reduced(xt, yt, 0.3, 255, False)
    want_grad = oracle.lmargin_backward(x.astype(np.float64), y, 0.3, 255, np.ones(y.shape))
    want_loss = oracle.lmargin_forward(x.astype(np.float64), y, 0.3, 255).sum()
    assert tag == 1 and grad.dtype == torch.float16
    assert abs(float(loss) - want_loss) <= 4e-3 * abs(want_loss)
    assert np.abs(grad.float().cpu().numpy() - want_grad).max() <= 2e-3 * np.abs(want_grad).max()


# (N, C) rows: the forward leaves eight floats of statistics per row and the backward is elementwise over the flattened
# tensor (row ends inside 16-byte chunks, a last chunk that is not whole, one row only); the rows of up to 2048 classes are
# the ones that a wavefront holds in registers in the forward (several rows per wavefront up to 512 classes)
LONG_ROWS = [(5, 5000), (3, 4099), (7, 6001), (1, 4097), (2, 8192), (33, 4100),
             (300, 33), (130, 48), (40, 64), (70, 200), (260, 300), (17, 1000), (9, 1100), (6, 2040), (1, 77)]
ROWS_16BIT_ONLY = [(20, 256), (9, 1024), (5, 2048)]


@pytest.mark.parametrize("dtype,tol", DTYPES, ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", LONG_ROWS, ids=str)
def test_long_rows_backward_from_the_forwards_statistics(mod, shape, dtype, tol):
    check_backward_from_statistics(shape, dtype, tol)


@pytest.mark.parametrize("dtype,tol", DTYPES[1:], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", ROWS_16BIT_ONLY, ids=str)
def test_16_bit_rows_of_a_power_of_two_take_the_statistics_too(mod, shape, dtype, tol):
    check_backward_from_statistics(shape, dtype, tol)


def check_backward_from_statistics(shape, dtype, tol):
    from pytorch_loss import _native
    lib = _native.load()
    tag = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    assert lib.plh_lmargin_saves_stats(tag, shape[0], shape[1], 1) == 1
    assert lib.plh_lmargin_saves_stats(tag, shape[0], 512, 1) == (0 if tag == 0 else 1) and lib.plh_lmargin_saves_stats(tag, 2, 5000, 4) == 0
    assert lib.plh_lmargin_saves_stats(tag, shape[0], 32, 1) == 0
    x = synth.normal(331, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(331, shape[:1], shape[1], 255, 0.2)
    if shape[0] > 2:
        y[::3] = shape[1] + 7                           # rows without a target class, not ignored
    xt = torch.from_numpy(x).cuda().to(dtype)
    x = xt.float().cpu().numpy()
    yt = torch.from_numpy(y).cuda()
    args = _native.lmargin_args(xt, yt)
    loss, n_valid, stats = _native.lmargin_forward_reduced_stats(xt, yt, 0.3, 255, True, args=args)
    loss2, n_valid2 = _native.lmargin_forward_reduced(xt, yt, 0.3, 255, True)
    assert stats is not None and stats.shape == (shape[0], 8)
    assert torch.equal(loss, loss2) and int(n_valid) == int(n_valid2) == int((y != 255).sum())
    nv = max(int((y != 255).sum()), 1)
    scalar = torch.full((), 0.7, device="cuda")
    want = oracle.lmargin_backward(x.astype(np.float64), y, 0.3, 255, np.full(shape[:1], 0.7 / nv))
    got = _native.lmargin_backward_scaled_stats(stats, 0.3, 255, scalar, n_valid, args)
    recomputed = _native.lmargin_backward_scaled(xt, yt, 0.3, 255, scalar, n_valid)
    scale = np.abs(want).max()
    assert got.dtype == dtype
    assert np.abs(got.float().cpu().numpy() - want).max() <= tol * scale
    assert (got.float() - recomputed.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * scale
    ign = torch.from_numpy(y == 255).cuda()
    if ign.any():
        assert got[ign].abs().max().item() == 0
    kept = torch.ones(shape[0], dtype=torch.uint8, device="cuda")
    kept[1::2] = 0
    got_kept = _native.lmargin_backward_scaled_stats(stats, 0.3, 255, scalar, n_valid, args, kept=kept)
    want_kept = want.copy()
    want_kept[1::2] = 0
    assert np.abs(got_kept.float().cpu().numpy() - want_kept).max() <= tol * scale
    if shape[0] > 1:
        assert got_kept[1::2].abs().max().item() == 0


def test_long_rows_module_step_and_views_off_the_16_byte_boundaries(mod):
    shape = (3, 4099)
    x = synth.normal(332, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(332, shape[:1], shape[1], 255, 0.0)
    yt = torch.from_numpy(y).cuda()
    want = oracle.lmargin_backward(x.astype(np.float64), y, 0.3, 255, np.full(shape[:1], 1.0 / shape[0]))
    a = torch.from_numpy(x).cuda().requires_grad_(True)
    mod.LargeMarginSoftmaxV3(ignore_index=255)(a, yt).backward()
    assert np.abs(a.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
    store = torch.empty(x.size + 1, device="cuda")       # logits one element into their storage: the recomputing kernel
    b = store[1:].view(shape)
    b.copy_(torch.from_numpy(x))
    b.requires_grad_(True)
    mod.LargeMarginSoftmaxV3(ignore_index=255)(b, yt).backward()
    assert np.abs(b.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()


def test_rows_between_the_two_capacities_of_a_wavefront(mod):
    """2049 .. 4096 classes: the forward that keeps the statistics is the block-per-row kernel for every element type (also
    where a wavefront could hold a 16-bit row in pieces of 8)."""
    from pytorch_loss import _native
    lib = _native.load()
    assert lib.plh_lmargin_saves_stats(0, 4, 2049, 1) == 1 and lib.plh_lmargin_saves_stats(0, 4, 4096, 1) == 1
    assert lib.plh_lmargin_saves_stats(2, 4, 3000, 1) == 1 and lib.plh_lmargin_saves_stats(2, 4, 2048, 1) == 1
    for shape, dtype, tol in [((3, 2049), torch.float32, 2e-6), ((4, 3000), torch.float32, 2e-6), ((2, 4096), torch.float32, 2e-6),
                              ((4, 3001), torch.bfloat16, 1.6e-2), ((5, 2051), torch.float16, 2e-3), ((4, 3000), torch.bfloat16, 1.6e-2),
                              ((3, 4096), torch.float16, 2e-3)]:
        x = synth.normal(341, 1, shape, 0.0, 2.0)
        y = synth.seg_labels(341, shape[:1], shape[1], 255, 0.2)
        xt = torch.from_numpy(x).cuda().to(dtype)
        x = xt.float().cpu().numpy()
        yt = torch.from_numpy(y).cuda()
        args = _native.lmargin_args(xt, yt)
        loss, n_valid, stats = _native.lmargin_forward_reduced_stats(xt, yt, 0.3, 255, True, args=args)
        assert stats is not None
        nv = max(int((y != 255).sum()), 1)
        one = torch.ones((), device="cuda")
        got = _native.lmargin_backward_scaled_stats(stats, 0.3, 255, one, n_valid, args)
        want = oracle.lmargin_backward(x.astype(np.float64), y, 0.3, 255, np.full(shape[:1], 1.0 / nv))
        assert np.abs(got.float().cpu().numpy() - want).max() <= tol * np.abs(want).max()
        recomputed = _native.lmargin_backward_scaled(xt, yt, 0.3, 255, one, n_valid)      # other block size, other summation order
        assert (got.float() - recomputed.float()).abs().max().item() <= (2e-6 if dtype == torch.float32 else tol) * np.abs(want).max()
