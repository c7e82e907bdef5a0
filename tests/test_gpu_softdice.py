"""GPU parity of the soft dice loss (through the C ABI) against the CPU oracle: losses 1e-5 relative,
gradients 1e-5 of the largest gradient magnitude (a row's gradient scales with 1/denor, so an
absolute bound would be vacuous for long rows), 16-bit tensors within one storage rounding."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _inputs(seed, n, length, soft=False):
    x = synth.normal(seed, 1, (n, length), 0.0, 2.0)
    if soft:
        y = synth.uniform01(seed, 2, n * length).reshape(n, length).astype(np.float32)
    else:
        y = synth.bernoulli(seed, 2, (n, length), 0.3).astype(np.float32)
    return x, y


CASES = [(1, 1), (1, 1000), (4, 37), (3, 4096), (7, 1023), (2, 100_003), (64, 512), (1, 2_000_000), (3, 513 * 513), (5, 4099), (6, 2)]


@pytest.mark.parametrize("n,length", CASES)
@pytest.mark.parametrize("p,smooth", [(1, 1.0), (2, 1.0), (1.5, 0.1)])
@pytest.mark.parametrize("soft", [False, True])
def test_function_matches_oracle(pl, n, length, p, smooth, soft):
    x, y = _inputs(111, n, length, soft)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    loss = pl.SoftDiceLossV3Func.apply(xt, yt, p, smooth)
    want, stats = oracle.soft_dice_forward(x.astype(np.float64), y.astype(np.float64), p, smooth)
    assert loss.shape == (n,) and loss.dtype == torch.float32
    assert np.abs(loss.detach().cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max() + 1e-7
    go = synth.normal(111, 3, (n,), 0.5, 1.0)
    loss.backward(torch.from_numpy(go).cuda())
    want_g = oracle.soft_dice_backward(go.astype(np.float64), x.astype(np.float64), y.astype(np.float64), stats, p)
    err = np.abs(xt.grad.cpu().numpy() - want_g).max()
    assert err <= 1e-5 * np.abs(want_g).max() + 1e-12, (err, np.abs(want_g).max())


def test_module_flattens_everything_into_one_row(pl):
    shape = (4, 1, 96, 96)
    x = synth.normal(112, 1, shape, 0.0, 2.0)
    y = synth.bernoulli(112, 2, shape, 0.3).astype(np.float32)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    crit = pl.SoftDiceLossV3()
    assert (crit.p, crit.smooth) == (1, 1.0)
    loss = crit(xt, torch.from_numpy(y).cuda())
    want, stats = oracle.soft_dice_forward(x.reshape(1, -1).astype(np.float64), y.reshape(1, -1).astype(np.float64), 1, 1.0)
    assert loss.shape == (1,) and abs(loss.item() - want[0]) <= 1e-5 * abs(want[0])
    loss.backward()
    want_g = oracle.soft_dice_backward(np.ones(1), x.reshape(1, -1).astype(np.float64), y.reshape(1, -1).astype(np.float64),
                                       stats, 1).reshape(shape)
    assert np.abs(xt.grad.cpu().numpy() - want_g).max() <= 1e-5 * np.abs(want_g).max()
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        crit(torch.zeros(2, 3), torch.zeros(2, 3))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_16bit(pl, dt):
    x, y = _inputs(113, 3, 4096)
    xt = torch.from_numpy(x).cuda().to(dt).requires_grad_()
    yt = torch.from_numpy(y).cuda().to(dt)
    xr = xt.detach().float().cpu().numpy().astype(np.float64)
    with torch.autocast("cuda", dtype=dt):
        loss = pl.SoftDiceLossV3Func.apply(xt, yt, 2, 1.0)
    want, stats = oracle.soft_dice_forward(xr, y.astype(np.float64), 2, 1.0)
    assert loss.dtype == torch.float32 and np.abs(loss.detach().cpu().numpy() - want).max() <= 1e-5
    loss.sum().backward()
    want_g = oracle.soft_dice_backward(np.ones(3), xr, y.astype(np.float64), stats, 2)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dt]
    assert xt.grad.dtype == dt
    assert (np.abs(xt.grad.float().cpu().numpy() - want_g) <= ulp * np.abs(want_g) + 1e-7).all()


def test_results_do_not_depend_on_scheduling(pl):
    x, y = _inputs(114, 2, 300_000)
    xt, yt = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    a = pl.SoftDiceLossV3Func.apply(xt, yt, 1, 1.0)
    for _ in range(3):
        assert torch.equal(pl.SoftDiceLossV3Func.apply(xt, yt, 1, 1.0), a)
