"""Short classifier rows in numbers that take a wavefront through several rounds.

The wavefront-per-row kernels give a wavefront four rows of up to 256 elements at a time (one row above
that) and the grid is capped, so beyond 262144 rows (65536 of the longer ones) every wavefront walks through
several rounds and reuses its LDS tile (the gradients of a round leave as one run) -- the small shapes of the
parity tests never get there. Rows are independent of each other, so the check is size-independent: per-row
losses and gradient rows of the big call must equal, bit for bit, those of calls on slices of it (first rows,
rows around a round's boundary, the ragged last rows), which are single-round launches of the same kernels
that the parity tests hold
against the oracle.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

ROWS = 262144 * 2 + 4 * 3 + 3          # two full rounds of the capped grid, three more blocks' worth, a ragged end


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _slices(rows):
    return [slice(0, 70), slice(262144 - 37, 262144 + 41), slice(2 * 262144 - 5, 2 * 262144 + 9), slice(rows - 7, rows)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("classes", [150, 151, 130, 34, 200, 256, 264, 300, 301, 512, 1000, 1001])
@pytest.mark.parametrize("loss", ["lsr", "lmargin", "taylor"])
def test_many_short_rows_equal_their_slices(pl, loss, classes, dtype):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(classes * 7 + 1)
    x = (torch.randn((ROWS, classes), device="cuda", generator=gen) * 3).to(dtype)
    y = torch.randint(0, classes, (ROWS,), device="cuda", generator=gen)
    ignore = {"lsr": -100, "lmargin": 255, "taylor": -1}[loss]
    y[torch.rand((ROWS,), device="cuda", generator=gen) < 0.1] = ignore
    if loss == "lsr":
        crit = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="none", ignore_index=ignore)
    elif loss == "lmargin":
        crit = pl.LargeMarginSoftmaxV3(lam=0.3, reduction="none", ignore_index=ignore)
    else:
        crit = pl.TaylorCrossEntropyLossV3(n=4, ignore_index=ignore, reduction="none")

    def run(xs, ys):
        xs = xs.clone().requires_grad_()
        per = crit(xs, ys)
        per.sum().backward()
        return per.detach(), xs.grad

    per_all, grad_all = run(x, y)
    assert torch.isfinite(per_all.float()).all() and torch.isfinite(grad_all.float()).all()
    assert (grad_all[y == ignore] == 0).all()
    for sl in _slices(ROWS):
        per, grad = run(x[sl], y[sl])
        assert torch.equal(per, per_all[sl]), (loss, classes, dtype, sl)
        assert torch.equal(grad, grad_all[sl]), (loss, classes, dtype, sl)
