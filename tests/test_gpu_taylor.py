"""GPU parity of the Taylor softmax Function, modules and cross entropy (through the C ABI) against
the CPU oracle: 1e-5 relative on outputs and losses, 1e-5 max-abs on gradients for fp32; one rounding
step of the storage type for 16-bit tensors."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth
from .test_gpu_parity import SEG_CASES, close_loss, dev, seg_inputs

pytestmark = pytest.mark.gpu

CASES = [
    # (shape, dim)                               execution shape
    ((2, 19, 64, 64), 1),                        # uniform tiles, slice in registers
    ((2, 19, 7, 9), 1),                          # one pixel per thread
    ((3, 2, 5, 8), 1),
    ((37, 10), 1),                               # (N, C), C <= 32
    ((33, 100), 1),                              # wavefront per row, the row in registers
    ((9, 77), 1),                                #   odd length: element by element
    ((2, 33, 6, 7), 1),                          # lane per slice
    ((24, 6, 5), 0),                             # dim 0: 24 channels 30 apart
    ((2, 3, 4, 40), 3),                          # last dim of a 4-D tensor: rows of 40
    ((2, 3, 16, 5), -2),
    ((64, 8, 8, 8), 0),                          # dim 0 with 64 channels: lane per slice
    ((6, 1000), 1),                              # longer register rows: 8 and 32 steps per wavefront
    ((3, 2047), -1),
    ((7, 201), 1),
    ((70, 33), 1),
    ((21, 136), 1),
    ((5, 260), 1),
    ((9, 264), 1),                               #   16-bit rows of 257..512 elements in whole chunks: 16 lanes, 4 steps
    ((6, 512), 1),
    ((5, 200), 1),                               #   short rows in whole chunks that end inside a 128-byte line
    ((7, 301), 1),                               #   257..512 elements in short pieces: 16 lanes, 32 single elements
    ((5, 258), 1),                               #   ... 16 pieces of two
    ((4, 1001), 1),
    ((5, 1544), 1),
    ((2, 2056), 1),                              # beyond the register rows: a block per row
    ((3, 4099), 1),                              #   odd length: element by element
    ((2, 30000), -1),                            #   1024-thread blocks
    ((2, 19, 65, 65), 1),                        # planes of odd length, 4096 pixels or more: tiles per image, four
    ((2, 11, 67, 63), 1),                        #   pixels per lane where the slices fit (the backward holds two:
    ((1, 24, 4097, 1), 1),                       #   12 channels fp32, 24 for 16-bit elements; the forward one: 24 / 32)
    ((2, 25, 65, 65), 1),
    ((2, 40, 16, 16), 1),                        # 33..256 channels, 64 pixels or more per image: the channels of a
    ((1, 150, 12, 16), 1),                       #   pixel shared out over the wavefronts of a block
    ((2, 256, 8, 8), 1),
    ((2, 60, 65, 65), 1),                        #   the same on planes of odd length: tiles per image
    ((1, 33, 67, 63), 1),
]


def close_rel(got, want, what=""):
    """Gradients through log f can be large where the polynomial comes close to 0 (f(-2.5) is 0.2 for
    order 8): hold them to 1e-5 of the tensor's largest magnitude, and to 1e-5 absolute when that is
    below 1."""
    err = np.abs(got.astype(np.float64) - want).max() if got.size else 0.0
    assert err <= 1e-5 * max(1.0, np.abs(want).max()), "%s grad err %.3e vs max %.3e" % (what, err, np.abs(want).max())


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


@pytest.mark.parametrize("shape,dim", CASES)
@pytest.mark.parametrize("order", [2, 4, 8])
@pytest.mark.parametrize("use_log", [False, True])
def test_function_matches_oracle(pl, shape, dim, order, use_log):
    x = synth.normal(101, 1, shape, 0.0, 1.5)
    g = synth.normal(101, 2, shape, 0.0, 1.0)
    xt = dev(x).requires_grad_()
    out = pl.TaylorSoftmaxFunc.apply(xt, dim, order, use_log)
    want = oracle.taylor_forward(x.astype(np.float64), dim, order, use_log)
    assert out.shape == xt.shape and out.dtype == torch.float32
    assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
    out.backward(dev(g))
    want_g = oracle.taylor_backward(g.astype(np.float64), x.astype(np.float64), dim, order, use_log)
    close_rel(xt.grad.cpu().numpy(), want_g, "taylor")
    if not use_log:
        assert torch.allclose(out.sum(dim=dim), torch.ones_like(out.sum(dim=dim)), atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape,dim", CASES[:7] + CASES[-25:])
def test_function_16bit(pl, shape, dim, dt):
    x = synth.normal(102, 1, shape, 0.0, 1.0)
    g = synth.normal(102, 2, shape, 0.0, 1.0)
    xt = dev(x).to(dt).requires_grad_()
    gt = dev(g).to(dt)
    xr, gr = xt.detach().float().cpu().numpy().astype(np.float64), gt.float().cpu().numpy().astype(np.float64)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dt]
    for use_log in (False, True):
        xt.grad = None
        out = pl.TaylorSoftmaxFunc.apply(xt, dim, 4, use_log)
        assert out.dtype == dt
        want = oracle.taylor_forward(xr, dim, 4, use_log)
        assert (np.abs(out.detach().float().cpu().numpy() - want) <= ulp * np.abs(want) + 1e-6).all()
        out.backward(gt)
        want_g = oracle.taylor_backward(gr, xr, dim, 4, use_log)
        assert xt.grad.dtype == dt
        assert (np.abs(xt.grad.float().cpu().numpy() - want_g) <= ulp * np.abs(want_g) + 1e-5).all()


def test_modules_and_defaults(pl):
    x = synth.normal(103, 1, (2, 19, 16, 16), 0.0, 1.5)
    xt = dev(x)
    a = pl.TaylorSoftmaxV3(dim=1, n=4)(xt)
    b = pl.LogTaylorSoftmaxV3(dim=1, n=4)(xt)
    assert torch.allclose(a.log(), b, atol=1e-5)
    assert torch.equal(pl.taylor_softmax_v3(xt, 1, 4, False), a)
    m = pl.TaylorSoftmaxV3()
    assert (m.dim, m.n) == (1, 2)
    c = pl.TaylorCrossEntropyLossV3()
    assert (c.n, c.ignore_index, c.reduction) == (2, -1, "mean")
    with pytest.raises(AssertionError):
        pl.TaylorSoftmaxV3(n=3)
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.TaylorSoftmaxV3()(torch.zeros(2, 3))
    assert pl.TaylorSoftmaxV3()(torch.zeros(0, 5, device="cuda")).shape == (0, 5)


@pytest.mark.parametrize("shape,ignore,frac", SEG_CASES)
@pytest.mark.parametrize("order", [2, 4])
def test_cross_entropy_matches_oracle(pl, shape, ignore, frac, order):
    x, y = seg_inputs(104, shape, ignore, frac)
    x = (x * 0.75).astype(np.float32)
    yt = dev(y)
    per = oracle.taylor_ce(x.astype(np.float64), y, order, ignore)
    n_valid = int((y != ignore).sum())
    # per pixel
    xt = dev(x).requires_grad_()
    out = pl.TaylorCrossEntropyLossV3(n=order, ignore_index=ignore, reduction="none")(xt, yt)
    assert out.shape == yt.shape
    close_loss(out.detach().cpu().numpy(), per, "taylor ce")
    assert (out.detach().cpu().numpy()[y == ignore] == 0).all()
    go = synth.normal(7, 3, y.shape, 0.0, 1.0)
    out.backward(dev(go))
    close_rel(xt.grad.cpu().numpy(), oracle.taylor_ce_backward(x.astype(np.float64), y, order, ignore, go), "taylor ce")
    g = xt.grad.cpu().numpy()
    assert (g[np.broadcast_to(np.expand_dims(y == ignore, 1), g.shape)] == 0).all()
    if frac >= 1.0:
        return
    for red in ("sum", "mean"):
        xt = dev(x).requires_grad_()
        out = pl.TaylorCrossEntropyLossV3(n=order, ignore_index=ignore, reduction=red)(xt, yt)
        want = per.sum() / (n_valid if red == "mean" else 1)
        assert out.dim() == 0 and abs(out.item() - want) <= 1e-5 * abs(want)
        (out * 2.0).backward()
        scale = 2.0 / (n_valid if red == "mean" else 1)
        close_rel(xt.grad.cpu().numpy(), oracle.taylor_ce_backward(x.astype(np.float64), y, order, ignore, scale),
                  "taylor ce " + red)


def test_cross_entropy_equals_the_reference_composition(pl):
    """TaylorCrossEntropyLossV3 in the reference is LogTaylorSoftmaxV3 followed by F.nll_loss."""
    x, y = seg_inputs(105, (2, 19, 32, 32), 255, 0.1)
    xt1, xt2, yt = dev(x).requires_grad_(), dev(x).requires_grad_(), dev(y)
    fused = pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255)(xt1, yt)
    composed = torch.nn.functional.nll_loss(pl.LogTaylorSoftmaxV3(dim=1, n=4)(xt2), yt, ignore_index=255)
    assert abs(fused.item() - composed.item()) <= 1e-6 * abs(composed.item())
    fused.backward()
    composed.backward()
    assert (xt1.grad - xt2.grad).abs().max().item() <= 1e-9 + 1e-5 * xt2.grad.abs().max().item()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 19, 32, 32), (2, 19, 65, 65), (2, 32, 63, 65), (1, 33, 65, 65)])
def test_cross_entropy_16bit(pl, dt, shape):
    x, y = seg_inputs(106, shape, 255, 0.1)
    xt = dev(x * 0.5).to(dt).requires_grad_()
    xr = xt.detach().float().cpu().numpy().astype(np.float64)
    with torch.autocast("cuda", dtype=dt):
        out = pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="sum")(xt, dev(y))
    want = oracle.taylor_ce(xr, y, 4, 255).sum()
    assert out.dtype == torch.float32 and abs(out.item() - want) <= 1e-5 * abs(want)
    out.backward()
    want_g = oracle.taylor_ce_backward(xr, y, 4, 255, 1.0)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dt]
    assert xt.grad.dtype == dt
    assert (np.abs(xt.grad.float().cpu().numpy() - want_g) <= ulp * np.abs(want_g) + 1e-7).all()
