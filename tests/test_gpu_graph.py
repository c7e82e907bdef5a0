"""A training step of each loss captured in a HIP graph and replayed: the entry points launch only
kernels on the caller's stream (no memset nodes, no host synchronisation, no allocation of their
own), so a captured step must give the eager step's loss and gradient bit for bit on every replay,
also after the inputs were overwritten in place."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _seg(seed, shape=(2, 19, 64, 96)):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, device="cuda", generator=g) * 2.0
    y = torch.randint(0, shape[1], shape[:1] + shape[2:], device="cuda", generator=g)
    y[torch.rand(y.shape, device="cuda", generator=g) < 0.05] = 255
    return x, y


def _binary(seed, shape=(2, 8, 32, 32)):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(shape, device="cuda", generator=g) * 1.5
    return x, (torch.rand(shape, device="cuda", generator=g) < 0.2).float()


CASES = {
    "lsr": (lambda pl: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="mean", ignore_index=255), _seg),
    "lmargin": (lambda pl: pl.LargeMarginSoftmaxV3(lam=0.3, reduction="mean", ignore_index=255), _seg),
    "lovasz": (lambda pl: pl.LovaszSoftmaxV3(reduction="mean", ignore_index=255), _seg),
    "taylor": (lambda pl: pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="mean"), _seg),
    "ohem": (lambda pl: pl.OhemCELoss(score_thresh=0.7, n_min=500, ignore_index=255), _seg),
    "ohem_lmargin": (lambda pl: pl.OhemLargeMarginLoss(score_thresh=0.7, n_min=500, ignore_index=255), _seg),
    "focal": (lambda pl: pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean"), _binary),
    "dice": (lambda pl: pl.SoftDiceLossV3(p=1, smooth=1.0), _binary),
    # loss and gradient from one pass, the backward a multiplication that returns at once (count of the labels,
    # finishing kernels and the scalar test are all kernels on the stream)
    "lsr_fb": (lambda pl: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="mean", ignore_index=255, fb=True), _seg),
    "lmargin_fb": (lambda pl: pl.LargeMarginSoftmaxV3(lam=0.3, reduction="mean", ignore_index=255, fb=True), _seg),
    "focal_fb": (lambda pl: pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean", fb=True), _binary),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_captured_step_replays_like_eager(pl, name):
    make, inputs = CASES[name]
    crit = make(pl)
    x0, y0 = inputs(1)
    x = x0.clone().requires_grad_()
    y = y0.clone()

    def step():
        x.grad = None
        loss = crit(x, y)
        loss.backward()
        return loss

    side = torch.cuda.Stream()                      # warm-up off the default stream, as capture requires
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    x.grad = None
    with torch.cuda.graph(graph):
        loss_g = crit(x, y)
        loss_g.backward()
    grad_g = x.grad

    for seed in (1, 2, 3, 2):
        xs, ys = inputs(seed)
        with torch.no_grad():
            x.copy_(xs)
            y.copy_(ys)
        graph.replay()
        torch.cuda.synchronize()
        got_loss, got_grad = loss_g.detach().clone(), grad_g.clone()
        xe = xs.clone().requires_grad_()
        want = crit(xe, ys)
        want.backward()
        torch.cuda.synchronize()
        assert torch.equal(got_loss, want.detach()), (name, seed, got_loss, want)
        assert torch.equal(got_grad, xe.grad), (name, seed)
