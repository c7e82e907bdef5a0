"""LabelSmoothSoftmaxCEV3 on channel planes of odd length: the forward that keeps every pixel's log-sum-exp
(plh_lsr_forward_reduced_lse) and the backward that forms the gradient from it plane by plane
(plh_lsr_backward_scaled_lse), against the oracle and against the kernels that recompute the softmax."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

# (shape, logit scale): planes of 4225 .. 6499 pixels, so a plane spans several 1024-pixel tiles and has both a
# partly filled first and last cache line; channel counts either side of a group of four planes; one image and several
SHAPES = [((2, 19, 65, 67), 2.0), ((1, 24, 65, 65), 3.0), ((3, 5, 71, 73), 1.0), ((2, 1, 67, 97), 1.0), ((5, 7, 65, 65), 8.0)]


@pytest.fixture(scope="module")
def native():
    from pytorch_loss import _native
    _native.load()
    return _native


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def inputs(seed, shape, scale, ignore_frac=0.1):
    x = synth.normal(seed, 1, shape, 0.0, scale)
    y = synth.seg_labels(seed, shape[:1] + shape[2:], shape[1], 255, ignore_frac)
    return x, y


@pytest.mark.parametrize("shape,scale", SHAPES)
def test_the_library_says_where_it_applies(native, shape, scale):
    lib = native.load()
    n, c = shape[0], shape[1]
    m = shape[2] * shape[3]
    assert lib.plh_lsr_saves_lse(0, n, c, m) == 1 and lib.plh_lsr_saves_lse(2, n, c, m) == 0      # fp32 logits only
    assert lib.plh_lsr_saves_lse(0, n, c, (m + 31) // 32 * 32) == 0     # planes that start on 128-byte lines
    assert lib.plh_lsr_saves_lse(0, n, 25, m) == 0 and lib.plh_lsr_saves_lse(0, n, 32, m) == 0   # the forward is not the per-image form there
    assert lib.plh_lsr_saves_lse(0, n, 33, m) == 1 and lib.plh_lsr_saves_lse(0, n, 256, 4096) == 0   # 33 and more: planes off the lines
    assert lib.plh_lsr_saves_lse(0, n, 257, 4096) == 1                                               # beyond 256: any plane
    assert lib.plh_lsr_saves_lse(2, n, 150, m) == 0
    assert lib.plh_lsr_saves_lse(0, n, c, 4095) == 0        # short planes
    assert lib.plh_lsr_saves_lse(0, n, 4097, 1) == 1 and lib.plh_lsr_saves_lse(2, n, 4097, 1) == 1      # long rows: any element type


@pytest.mark.parametrize("mean", [True, False], ids=["mean", "sum"])
@pytest.mark.parametrize("shape,scale", SHAPES)
def test_forward_keeps_the_log_sum_exp_and_backward_uses_it(native, shape, scale, mean):
    x, y = inputs(141, shape, scale)
    y.reshape(-1)[::97] = shape[1] + 3                       # labels without a target channel, not ignored
    xt, yt = dev(x), dev(y)
    loss, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, mean)
    assert lse is not None and lse.shape == (y.size,)
    want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).reshape(-1).numpy()
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-6 * np.abs(want_lse).max()
    loss2, n_valid2 = native.lsr_forward_reduced(xt, yt, 255, 0.1, mean)
    assert loss.cpu().numpy().tobytes() == loss2.cpu().numpy().tobytes() and int(n_valid.item()) == int(n_valid2.item())
    up = torch.full((), 0.7, device=xt.device)
    div = n_valid if mean else None
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, up, div, native.lsr_args(xt, yt))
    want = native.lsr_backward_scaled(xt, yt, 255, 0.1, up, div)
    ref = want.abs().max().item()
    assert (got - want).abs().max().item() <= 2e-6 * ref
    flat = y.reshape(shape[0], -1)
    g = got.cpu().numpy().reshape(shape[0], shape[1], -1)
    assert not g.transpose(0, 2, 1)[flat == 255].any()      # exact zeros where ignored
    # the oracle, under a unit upstream gradient
    one = torch.ones((), device=xt.device)
    got1 = native.lsr_backward_scaled_lse(lse, 255, 0.1, one, None, native.lsr_args(xt, yt)).cpu().numpy()
    want1 = oracle.lsr_backward(x, y, 255, 0.1, np.float32(1.0))
    assert np.abs(got1 - want1).max() <= 2e-5 * np.abs(want1).max()


def test_byte_mask_of_a_selection(native):
    shape = (2, 19, 65, 67)
    x, y = inputs(142, shape, 2.0)
    xt, yt = dev(x), dev(y)
    kept = (torch.rand(y.size, device=xt.device) < 0.6).to(torch.uint8)
    _, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.0, True)
    one = torch.ones((), device=xt.device)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.0, one, n_valid, native.lsr_args(xt, yt), kept=kept)
    relabelled = yt.clone().reshape(-1)
    relabelled[kept == 0] = 255
    want = native.lsr_backward_scaled(xt, relabelled.reshape(yt.shape), 255, 0.0, one, n_valid)
    assert (got - want).abs().max().item() <= 2e-6 * want.abs().max().item()


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("shape,scale", SHAPES[:3])
def test_module_step_against_the_oracle(native, shape, scale, reduction):
    import pytorch_loss as pl
    x, y = inputs(143, shape, scale)
    xt = dev(x).requires_grad_()
    crit = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=reduction, ignore_index=255)
    loss = crit(xt, dev(y))
    per = oracle.lsr_forward(x.astype(np.float64), y, 255, 0.1)
    n_valid = int((y != 255).sum())
    want = per.sum() / n_valid if reduction == "mean" else per.sum()
    assert abs(loss.item() - want) <= 1e-5 * abs(want)
    loss.backward()
    want_g = oracle.lsr_backward(x, y, 255, 0.1, np.float32(1.0 / n_valid if reduction == "mean" else 1.0))
    err = np.abs(xt.grad.cpu().numpy() - want_g).max()
    assert err <= 2e-5 * np.abs(want_g).max()
    # without a gradient asked for, nothing extra is kept
    with torch.no_grad():
        assert abs(crit(xt, dev(y)).item() - want) <= 1e-5 * abs(want)


def test_views_whose_gradient_sits_elsewhere_in_a_line_take_the_recomputing_kernel(native):
    """Logits that start one element into their storage: the fresh gradient tensor is 256-byte aligned, the logits are
    not, so whole lines of the one are not whole lines of the other and the entry point recomputes."""
    shape = (2, 19, 65, 67)
    x, y = inputs(144, shape, 2.0)
    store = torch.empty(x.size + 1, device="cuda")
    xt = store[1:].view(shape)
    xt.copy_(dev(x))
    yt = dev(y)
    _, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
    want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).reshape(-1).numpy()
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-6 * np.abs(want_lse).max()
    one = torch.ones((), device=xt.device)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, one, n_valid, native.lsr_args(xt, yt))
    want = native.lsr_backward_scaled(xt, yt, 255, 0.1, one, n_valid)
    assert torch.equal(got, want)


def test_sizes_outside_are_refused(native):
    lib = native.load()
    x = torch.zeros((2, 19, 64, 64), device="cuda")
    y = torch.zeros((2, 64, 64), dtype=torch.int64, device="cuda")
    lse = torch.zeros(2 * 64 * 64, device="cuda")
    loss = torch.zeros((), device="cuda")
    ws = torch.empty(int(lib.plh_reduce_workspace_bytes(2 * 64 * 64)), dtype=torch.uint8, device="cuda")
    P = native._ptr
    rc = lib.plh_lsr_forward_reduced_lse(P(x), 0, P(y), P(lse), P(loss), None, 1, P(ws), ws.numel(), 2, 19, 4096, 255, 0.1,
                                         native._stream())
    assert rc == -2                      # PLH_ERR_BAD_SIZE: planes of even length


def test_even_planes_off_the_lines(native):
    """Planes of even length that do not start on 128-byte lines (1022 x 1022 style) take the same pair."""
    shape = (2, 19, 66, 70)            # 4620 pixels: 18480 bytes, not a multiple of 128
    x, y = inputs(146, shape, 2.0)
    xt, yt = dev(x), dev(y)
    _, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
    assert lse is not None
    one = torch.ones((), device=xt.device)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, one, n_valid, native.lsr_args(xt, yt))
    want = native.lsr_backward_scaled(xt, yt, 255, 0.1, one, n_valid)
    assert (got - want).abs().max().item() <= 2e-6 * want.abs().max().item()


# 33 channels and more, every forward shape that can take them: channels shared among wavefronts (aligned planes; planes
# of odd length in tiles per image), the deep form (257..512), a lane per pixel (beyond 512, and planes whose tensors sit
# on element boundaries only)
WIDE = [((2, 40, 65, 65), 2.0), ((2, 150, 66, 70), 2.0), ((1, 60, 65, 67), 1.0), ((1, 300, 65, 65), 2.0),
        ((1, 384, 65, 66), 3.0), ((1, 600, 64, 64), 1.0), ((2, 171, 65, 65), 2.0), ((1, 520, 65, 67), 1.0),
        ((2, 300, 64, 64), 2.0), ((420, 33, 65, 65), 2.0), ((1, 36, 513, 513), 2.0)]     # the last two: 8 and 16 planes per block


@pytest.mark.parametrize("shape,scale", WIDE)
def test_many_channels(native, shape, scale):
    x, y = inputs(147, shape, scale)
    y.reshape(-1)[::101] = shape[1] + 1                      # labels without a target channel, not ignored
    xt, yt = dev(x), dev(y)
    loss, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
    assert lse is not None
    want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).reshape(-1).numpy()
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-6 * np.abs(want_lse).max()
    loss2, n_valid2 = native.lsr_forward_reduced(xt, yt, 255, 0.1, True)
    assert loss.cpu().numpy().tobytes() == loss2.cpu().numpy().tobytes() and int(n_valid.item()) == int(n_valid2.item())
    one = torch.ones((), device=xt.device)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, one, None, native.lsr_args(xt, yt))
    want = native.lsr_backward_scaled(xt, yt, 255, 0.1, one, None)
    assert (got - want).abs().max().item() <= 2e-6 * want.abs().max().item()
    if x.size <= 20_000_000:
        want64 = oracle.lsr_backward(x, y, 255, 0.1, np.float32(1.0))
        assert np.abs(got.cpu().numpy() - want64).max() <= 2e-5 * np.abs(want64).max()


def test_many_channels_on_a_view_one_element_in(native):
    """The forward then runs a lane per pixel, the backward recomputes (logits and gradient sit differently in
    their lines): the pair still gives the module's results."""
    shape = (1, 150, 65, 67)
    x, y = inputs(148, shape, 2.0)
    store = torch.empty(x.size + 1, device="cuda")
    xt = store[1:].view(shape)
    xt.copy_(dev(x))
    yt = dev(y)
    _, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
    want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).reshape(-1).numpy()
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-6 * np.abs(want_lse).max()
    one = torch.ones((), device=xt.device)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, one, n_valid, native.lsr_args(xt, yt))
    want = native.lsr_backward_scaled(xt, yt, 255, 0.1, one, n_valid)
    assert torch.equal(got, want)


# more than 512 channels in NCHW: the forward whose wavefronts stream the channels (planes of 256 pixels and more; tiles
# that end inside a plane; channel counts that leave some wavefronts one channel short, and short last batches)
STREAM = [((1, 600, 16, 16), 2.0), ((2, 513, 17, 19), 1.0), ((1, 1000, 20, 20), 3.0), ((3, 519, 16, 17), 2.0), ((1, 545, 65, 65), 2.0)]


@pytest.mark.parametrize("shape,scale", STREAM)
def test_forward_beyond_512_channels(native, shape, scale):
    x, y = inputs(151, shape, scale)
    y.reshape(-1)[::37] = shape[1] + 5                       # labels without a target channel, not ignored
    x[0, 3, 0, :5] = -np.inf                                 # exp(-inf) = 0 inside a batch
    x[0, ::8, 1, 2] = -np.inf                                # a wavefront whose channels are all -inf at one pixel
    xt, yt = dev(x), dev(y)
    want = oracle.lsr_forward(x.astype(np.float64), y, 255, 0.1)
    got = native.lsr_forward(xt, yt, 255, 0.1).cpu().numpy()
    finite = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), finite)
    assert np.abs(got[finite] - want[finite]).max() <= 2e-6 * np.abs(want[finite]).max()
    for mean in (True, False):
        loss, n_valid = native.lsr_forward_reduced(xt, yt, 255, 0.1, mean)
        assert int(n_valid.item()) == int((y != 255).sum())
    y2 = y.copy()
    y2[0, 0, :5] = 255
    y2[0, 1, 2] = 255                                        # the pixels with infinite losses out of the sum
    want2 = oracle.lsr_forward(x.astype(np.float64), y2, 255, 0.1)
    loss, n_valid = native.lsr_forward_reduced(xt, dev(y2), 255, 0.1, True)
    assert abs(float(loss) - want2.sum() / (y2 != 255).sum()) <= 2e-6 * abs(want2.sum() / (y2 != 255).sum())
    if lib_saves(native, shape):
        _, _, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
        want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).reshape(-1).numpy()
        assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-6 * np.abs(want_lse).max()


def lib_saves(native, shape):
    return native.load().plh_lsr_saves_lse(0, shape[0], shape[1], shape[2] * shape[3]) == 1


# (N, C) rows: the forward leaves one log-sum-exp per row and the backward is elementwise over the flattened tensor (row
# ends inside 16-byte chunks, a last chunk that is not whole, one row only); the first six are the block-per-row forward's,
# the next ones rows that a wavefront holds in registers (several rows per wavefront among them), the last ones those of
# them that qualify only with fp32 logits
ROWS = [(5, 5000), (3, 4099), (7, 6001), (1, 4097), (2, 8192), (33, 4100),
        (300, 40), (130, 48), (40, 64), (9, 1100), (6, 2040), (5, 2048), (17, 1032)]
ROWS_16BIT_ONLY = [(4, 3000), (3, 4096), (5, 2051)]
ROWS_FP32_ONLY = [(70, 200), (260, 300), (17, 1000), (1, 77), (9, 1024), (300, 33), (50, 100)]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", ROWS, ids=str)
def test_long_rows(native, shape, dtype, tol):
    check_rows_from_lse(native, shape, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", ROWS_16BIT_ONLY, ids=str)
def test_rows_that_qualify_with_16_bit_logits_only(native, shape, dtype, tol):
    assert native.load().plh_lsr_saves_lse(0, shape[0], shape[1], 1) == 0
    check_rows_from_lse(native, shape, dtype, tol)


@pytest.mark.parametrize("shape", ROWS_FP32_ONLY, ids=str)
def test_rows_that_qualify_with_fp32_logits_only(native, shape):
    lib = native.load()
    assert lib.plh_lsr_saves_lse(1, shape[0], shape[1], 1) == 0 and lib.plh_lsr_saves_lse(2, shape[0], shape[1], 1) == 0
    check_rows_from_lse(native, shape, torch.float32, 2e-6)


def check_rows_from_lse(native, shape, dtype, tol):
    lib = native.load()
    tag = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    assert lib.plh_lsr_saves_lse(tag, shape[0], shape[1], 1) == 1 and lib.plh_lsr_saves_lse(tag, shape[0], 512, 1) == 0
    assert lib.plh_lsr_saves_lse(tag, shape[0], 32, 1) == 0
    x = synth.normal(161, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(161, shape[:1], shape[1], 255, 0.2)
    y[::3] = shape[1] + 7 if shape[0] > 2 else y[::3]           # rows without a target class, not ignored
    xt = torch.from_numpy(x).cuda().to(dtype)
    x = xt.float().cpu().numpy()
    yt = dev(y)
    loss, n_valid, lse = native.lsr_forward_reduced_lse(xt, yt, 255, 0.1, True)
    assert lse is not None and lse.shape == (shape[0],)
    want_lse = torch.logsumexp(torch.from_numpy(x).double(), 1).numpy()
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 4e-6 * np.abs(want_lse).max()
    nv = int((y != 255).sum())
    assert int(n_valid.item()) == nv
    scalar = torch.full((), 0.7, device="cuda")
    kept = torch.ones(shape[0], dtype=torch.uint8, device="cuda")
    kept[1::2] = 0
    up = np.full(shape[:1], 0.7 / max(nv, 1))
    want = oracle.lsr_backward(x.astype(np.float64), y, 255, 0.1, up)
    got = native.lsr_backward_scaled_lse(lse, 255, 0.1, scalar, n_valid, native.lsr_args(xt, yt))
    assert got.dtype == dtype
    assert np.abs(got.float().cpu().numpy() - want).max() <= tol * np.abs(want).max()
    ign = torch.from_numpy(y == 255).cuda()
    if ign.any():
        assert got[ign].abs().max().item() == 0
    got_kept = native.lsr_backward_scaled_lse(lse, 255, 0.1, scalar, n_valid, native.lsr_args(xt, yt), kept=kept)
    want_kept = want.copy()
    want_kept[1::2] = 0
    assert np.abs(got_kept.float().cpu().numpy() - want_kept).max() <= tol * np.abs(want).max()
    assert got_kept[1::2].abs().max().item() == 0 if shape[0] > 1 else True


def test_long_rows_on_views_off_the_16_byte_boundaries(native):
    """Logits one element into their storage: the backward goes row by row, element by element."""
    shape = (3, 4099)
    x = synth.normal(162, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(162, shape[:1], shape[1], 255, 0.0)
    store = torch.empty(x.size + 1, device="cuda")
    xt = store[1:].view(shape)
    xt.copy_(torch.from_numpy(x))
    yt = dev(y)
    a = xt.requires_grad_(True)
    from pytorch_loss import LabelSmoothSoftmaxCEV3
    loss = LabelSmoothSoftmaxCEV3(ignore_index=255)(a, yt)
    loss.backward()
    want = oracle.lsr_backward(x.astype(np.float64), y, 255, 0.1, np.full(shape[:1], 1.0 / shape[0]))
    assert np.abs(a.grad.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()

