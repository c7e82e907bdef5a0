"""The reference's own way of testing (the __main__ harness of every module, e.g.
pytorch_loss/label_smooth.py:174-253): two identical networks, one trained with criterion A and one
with criterion B on the same batches, and the difference of losses and weights watched over the
iterations. Here A is the HIP module and B the pure-torch restatement of the reference's V1/V2
flow running under torch autograd on the same GPU; a small conv net stands in for resnet18
(torchvision is not part of this image)."""
import copy

import pytest
import torch
import torch.nn as nn

from oracle import torch_ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


def _net(n_out):
    torch.manual_seed(15)
    return nn.Sequential(nn.Conv2d(3, 16, 3, padding=1), nn.ReLU(), nn.Conv2d(16, 16, 3, padding=1), nn.ReLU(),
                         nn.Conv2d(16, n_out, 1)).cuda()


def _train_pair(crit_a, crit_b, n_out, make_labels, steps=30, lr=0.05):
    net_a = _net(n_out)
    net_b = copy.deepcopy(net_a)
    opt_a = torch.optim.SGD(net_a.parameters(), lr=lr, momentum=0.9)
    opt_b = torch.optim.SGD(net_b.parameters(), lr=lr, momentum=0.9)
    g = torch.Generator(device="cuda").manual_seed(16)
    first = last = None
    for it in range(steps):
        x = torch.randn(4, 3, 24, 24, device="cuda", generator=g)
        y = make_labels(g, x)
        la = crit_a(net_a(x), y)
        lb = crit_b(net_b(x), y)
        assert abs(la.item() - lb.item()) <= 2e-5 * abs(lb.item()) + 1e-7, (it, la.item(), lb.item())
        for opt, loss in ((opt_a, la), (opt_b, lb)):
            opt.zero_grad()
            loss.backward()
            opt.step()
        first = la.item() if first is None else first
        last = la.item()
    drift = max((pa - pb).abs().max().item() for pa, pb in zip(net_a.parameters(), net_b.parameters()))
    assert drift <= 1e-4, drift      # fp32 rounding differences between the two flows, amplified by 30 momentum steps
    assert last < first              # and it trains


def _seg_labels(n_cls):
    def make(g, x):
        # a class the net can learn: the first input plane cut into n_cls bands
        y = ((x[:, 0] * 0.5 + 0.5).clamp(0, 0.999) * n_cls).long()
        y[0, :3, :] = 255            # a stripe of ignored pixels, as in the reference's harness
        y[3, 5, 7] = 255
        return y
    return make


def test_label_smooth_ce_trains_like_the_torch_flow(pl):
    _train_pair(pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, ignore_index=255),
                lambda lg, y: torch_ref.lsr(lg, y, 0.1, "mean", 255), 19, _seg_labels(19))


def test_large_margin_trains_like_the_torch_flow(pl):
    _train_pair(pl.LargeMarginSoftmaxV3(lam=0.3, ignore_index=255),
                lambda lg, y: torch_ref.lmargin(lg, y, 0.3, "mean", 255), 19, _seg_labels(19))


def test_lovasz_trains_like_the_torch_flow(pl):
    _train_pair(pl.LovaszSoftmaxV3(ignore_index=255),
                lambda lg, y: torch_ref.lovasz(lg, y, "mean", 255), 8, _seg_labels(8), lr=0.02)


def test_focal_trains_like_the_torch_flow(pl):
    def soft_labels(g, x):           # soft labels, like the root focal harness (focal_loss.py:262)
        return torch.sigmoid(3.0 * x[:, :1] + torch.randn(4, 6, 24, 24, device="cuda", generator=g))
    _train_pair(pl.FocalLossV3(alpha=0.25, gamma=2), lambda lg, y: torch_ref.focal(lg, y, 0.25, 2, "mean"), 6,
                soft_labels)


def test_taylor_ce_trains_like_the_torch_flow(pl):
    _train_pair(pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255),
                lambda lg, y: torch_ref.taylor_ce(lg, y, 4, "mean", 255), 19, _seg_labels(19))
