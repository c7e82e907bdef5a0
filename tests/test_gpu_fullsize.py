"""The benchmark configurations at full size on the GPU.

The oracle checks one image of each batch (what a CPU finishes in seconds); the rest of the batch
is held to size-independent properties: gradient rows of valid pixels sum to zero, ignored pixels
give exact zeros, the valid count is an exact integer, 'mean' equals 'sum' / count, results do
not depend on where in the batch an image sits, Lovasz Jaccard differences telescope to one and
the loss does not change under a permutation of the pixels.
"""
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


def _seg_full(name):
    w = synth.workload(name)            # portable generator: identical bits on every box
    return w["logits"], w["labels"]


@pytest.mark.parametrize("name", ["cfg2", "cfg4"])
def test_channel_softmax_losses_full_size(pl, name):
    x, y = _seg_full(name)
    assert x.shape == (8, 19, 1024, 1024)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    if name == "cfg2":
        make = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=255)
        o_fwd = lambda a, b: oracle.lsr_forward(a, b, 255, 0.1)
        o_bwd = lambda a, b, g: oracle.lsr_backward(a, b, 255, 0.1, g)
    else:
        make = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=255)
        o_fwd = lambda a, b: oracle.lmargin_forward(a, b, 0.3, 255)
        o_bwd = lambda a, b, g: oracle.lmargin_backward(a, b, 0.3, 255, g)

    n_valid = int((y != 255).sum())
    mean = make("mean")(xt, yt)
    mean.backward()
    g_mean = xt.grad.clone()
    xt.grad = None
    total = make("sum")(xt, yt)
    total.backward()
    g_sum = xt.grad.clone()
    xt.grad = None
    per = make("none")(xt, yt)

    # reductions agree with each other and with the exact integer count
    assert abs(mean.item() - total.item() / n_valid) <= 1e-6 * abs(mean.item())
    assert abs(per.double().sum().item() - total.item()) <= 1e-5 * abs(total.item())
    # masks: exact zeros at ignored pixels, nowhere else
    ign = yt == 255
    assert (per[ign] == 0).all() and (per[~ign] > 0).all()
    assert (g_sum.permute(0, 2, 3, 1)[ign] == 0).all()
    # softmax-type gradients: rows of valid pixels sum to zero
    assert g_sum.sum(dim=1).abs().max().item() < 1e-5
    # mean gradient = sum gradient / n_valid (linearity in the upstream scalar)
    assert (g_mean * n_valid - g_sum).abs().max().item() < 1e-5
    # oracle on one image; position in the batch must not matter
    k = 5
    want = o_fwd(x[k:k + 1], y[k:k + 1])
    got = per[k:k + 1].detach().cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
    want_g = o_bwd(x[k:k + 1], y[k:k + 1], None)
    err = np.abs(g_sum[k:k + 1].cpu().numpy() - want_g).max()
    assert err <= 1e-5, err
    alone = make("none")(xt[k:k + 1].detach().contiguous(), yt[k:k + 1].contiguous())
    assert torch.equal(alone, per[k:k + 1].detach())
    # whole-batch loss against the oracle's per-image sums
    ref_total = sum(o_fwd(x[i:i + 1], y[i:i + 1]).sum(dtype=np.float64) for i in range(x.shape[0]))
    assert abs(total.item() - ref_total) <= 1e-5 * abs(ref_total)


@pytest.mark.parametrize("kind,shape", [("lsr", (6, 19, 769, 769)), ("lmargin", (9, 19, 513, 513)), ("lsr", (3, 21, 1023, 1025))])
def test_odd_crops_full_size(pl, kind, shape):
    """fp32 channel planes of odd length take tiles per image with four pixels per lane (every image ends in a
    partly filled lane, every plane starts at another offset into a cache line): the same properties as above at
    crop sizes segmentation trains on, the oracle on the last image, and no dependence on the batch position."""
    x = synth.normal(31, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(31, shape[:1] + shape[2:], shape[1], 255, 0.05)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    if kind == "lsr":
        make = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=255)
        o_fwd = lambda a, b: oracle.lsr_forward(a, b, 255, 0.1)
        o_bwd = lambda a, b, g: oracle.lsr_backward(a, b, 255, 0.1, g)
    else:
        make = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=255)
        o_fwd = lambda a, b: oracle.lmargin_forward(a, b, 0.3, 255)
        o_bwd = lambda a, b, g: oracle.lmargin_backward(a, b, 0.3, 255, g)
    n_valid = int((y != 255).sum())
    mean = make("mean")(xt, yt)
    mean.backward()
    g_mean = xt.grad.clone()
    xt.grad = None
    per = make("none")(xt, yt)
    per.sum().backward()
    g_sum = xt.grad.clone()
    assert abs(mean.item() - per.double().sum().item() / n_valid) <= 1e-6 * abs(mean.item())
    ign = yt == 255
    assert (per[ign] == 0).all() and (per[~ign] > 0).all()
    assert (g_sum.permute(0, 2, 3, 1)[ign] == 0).all()
    assert g_sum.sum(dim=1).abs().max().item() < 1e-5
    assert (g_mean * n_valid - g_sum).abs().max().item() < 1e-5
    k = shape[0] - 1                                # the last image: its last lane is the last of the tensor
    want = o_fwd(x[k:k + 1], y[k:k + 1])
    got = per[k:k + 1].detach().cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
    err = np.abs(g_sum[k:k + 1].cpu().numpy() - o_bwd(x[k:k + 1], y[k:k + 1], None)).max()
    assert err <= 1e-5, err
    alone = make("none")(xt[k:k + 1].detach().contiguous(), yt[k:k + 1].contiguous())
    assert torch.equal(alone, per[k:k + 1].detach())


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("kind,shape", [("lsr", (6, 19, 769, 769)), ("lmargin", (9, 19, 513, 513))])
def test_odd_crops_full_size_16bit(pl, kind, shape, dt):
    """The same crops with 16-bit logits (tiles per image, four pixels per lane, 8-byte accesses that start on
    2-byte boundaries): exact zeros at ignored pixels, 'mean' against the per-pixel losses, the oracle on the
    stored values of the last image to one step of the storage type, no dependence on the batch position."""
    x = synth.normal(33, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(33, shape[:1] + shape[2:], shape[1], 255, 0.05)
    xt = torch.from_numpy(x).cuda().to(dt).requires_grad_()
    yt = torch.from_numpy(y).cuda()
    k = shape[0] - 1
    xr = xt[k:k + 1].detach().float().cpu().numpy()
    if kind == "lsr":
        make = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=255)
        want = oracle.lsr_forward(xr, y[k:k + 1], 255, 0.1)
        want_g = oracle.lsr_backward(xr, y[k:k + 1], 255, 0.1, None)
    else:
        make = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=255)
        want = oracle.lmargin_forward(xr, y[k:k + 1], 0.3, 255)
        want_g = oracle.lmargin_backward(xr, y[k:k + 1], 0.3, 255, None)
    n_valid = int((y != 255).sum())
    with torch.autocast("cuda", dtype=dt):
        mean = make("mean")(xt, yt)
        per = make("none")(xt, yt)
    assert per.dtype == torch.float32 and mean.dtype == torch.float32
    per.sum().backward()
    g_sum = xt.grad
    assert g_sum.dtype == dt
    assert abs(mean.item() - per.double().sum().item() / n_valid) <= 1e-6 * abs(mean.item())
    ign = yt == 255
    assert (per[ign] == 0).all() and (per[~ign] > 0).all()
    assert (g_sum.permute(0, 2, 3, 1)[ign] == 0).all()
    got = per[k:k + 1].detach().cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
    ulp = 2.0 ** -10 if dt == torch.float16 else 2.0 ** -7      # one step of the storage type
    got_g = g_sum[k:k + 1].float().cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got_g - want_g) <= ulp * np.abs(want_g) + 1e-6)    # + fp32 arithmetic on values of order one
    with torch.autocast("cuda", dtype=dt):
        alone = make("none")(xt[k:k + 1].detach().contiguous(), yt[k:k + 1].contiguous())
    assert torch.equal(alone, per[k:k + 1].detach())


def test_focal_full_size(pl):
    w = synth.workload("cfg3")
    x, y = w["logits"], w["labels"]
    assert x.shape == (16, 80, 128, 128)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    mean = pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean")(xt, yt)
    mean.backward()
    per = pl.FocalLossV3(alpha=0.25, gamma=2, reduction="none")(xt.detach(), yt)
    want = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, 2.0)
    assert abs(mean.item() - want.mean()) <= 1e-5 * want.mean()
    got = per.cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6 * want.mean())
    want_g = oracle.focal_backward(x, y, 0.25, 2.0, np.float32(1.0 / x.size))
    g = xt.grad.cpu().numpy()
    assert np.abs(g - want_g).max() <= 1e-5
    assert np.abs(g - want_g).max() <= 2e-5 * np.abs(want_g).max()      # relative: 'mean' makes 1e-5 absolute vacuous
    # symmetry loss(x, y; a) == loss(-x, 1-y; 1-a)
    flipped = pl.FocalLossV3(alpha=0.75, gamma=2, reduction="none")(-xt.detach(), 1.0 - yt)
    assert (flipped - per).abs().max().item() <= 1e-6


def test_lovasz_full_size(pl):
    from pytorch_loss import _native
    w = synth.workload("cfg5")
    x, y = w["logits"], w["labels"]
    assert x.shape == (4, 19, 512, 1024)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    yt = torch.from_numpy(y).cuda()
    losses = pl.LovaszSoftmaxV3(reduction="none", ignore_index=255)(xt, yt)
    losses.sum().backward()
    want, want_jacc = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(losses.detach().cpu().numpy(), want, rtol=1e-5)
    # gradient against the fp64 oracle: identical up to re-ordering of near-ties
    want_g = oracle.lovasz_backward(np.ones(19), x.astype(np.float64), y, want_jacc, 255)
    err = np.abs(xt.grad.cpu().numpy() - want_g)
    assert np.median(err) < 1e-9 and err.max() <= 1e-5, (np.median(err), err.max())
    g = xt.grad
    assert (g.permute(0, 2, 3, 1)[yt == 255] == 0).all()
    assert g.sum(dim=1).abs().max().item() < 1e-6            # softmax Jacobian: rows sum to zero
    # saved Jaccard differences: zero at ignored pixels, each class telescopes to J(all) = 1
    _, jacc = _native.lovasz_forward(xt.detach(), yt, 255)
    assert (jacc[:, (yt == 255).reshape(-1)] == 0).all()
    assert (jacc.double().sum(dim=1) - 1.0).abs().max().item() < 1e-6
    assert (jacc >= 0).all()        # J is monotone along the sorted order
    # the loss is a function of the multiset of (error, label) pairs: permuting pixels changes nothing
    perm = torch.randperm(512 * 1024, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
    xp = xt.detach().reshape(4, 19, -1)[:, :, perm].reshape(4, 19, 512, 1024).contiguous()
    yp = yt.reshape(4, -1)[:, perm].reshape(4, 512, 1024).contiguous()
    lp = pl.LovaszSoftmaxV3(reduction="none", ignore_index=255)(xp, yp)
    assert (lp - losses.detach()).abs().max().item() <= 2e-6


@pytest.mark.parametrize("n_pix", [2 ** 21 + 4096 + 3, 8192 * 1024 + 4096 + 3], ids=["regions_of_16k", "regions_of_32k"])
def test_lovasz_long_rows_use_larger_staging_regions(pl, n_pix):
    """Class rows of more than 256 regions of 8192 pixels: the staging regions double in size (up to
    32768 pixels) so that a tile still sends runs of values to each of them."""
    from pytorch_loss import _native
    x = synth.normal(91, 1, (n_pix, 2), 0.0, 2.0)
    y = synth.randint(91, 2, (n_pix,), 0, 2).astype(np.int64)
    y[synth.bernoulli(91, 3, (n_pix,), 0.05)] = 255
    losses, jacc = _native.lovasz_forward(torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda(), 255)
    l64, j64 = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(losses.cpu().numpy(), l64, rtol=1e-5)
    jacc = jacc.cpu().numpy()
    assert (jacc[:, y == 255] == 0).all()
    np.testing.assert_allclose(jacc.sum(axis=1, dtype=np.float64), 1.0, rtol=1e-4)
    assert np.abs(jacc - j64).max() <= 2.0 ** -23         # J is near 1 here: one fp32 ulp of it, as in the reference
    # bit pattern against the fp32 restatement (at this length fp32 differences of J round to 0 for
    # many keys that are not left out, so the zero pattern is only comparable in fp32)
    _, j32 = oracle.lovasz_forward(x, y, 255)
    assert (jacc.view(np.uint32) == j32.view(np.uint32)).mean() > 0.99


def test_lovasz_rows_longer_than_the_staging_regions(pl):
    """More than 1024 regions of 32768 pixels per class row: the Jaccard differences are scattered
    straight to pixel order, and the pixels left out of the sort are cleared beforehand. The CPU
    oracle needs a minute at this length; the check is the torch restatement of the V1 flow
    (stable sort, cumulative sums) in fp64 on the same device, plus the size-independent properties."""
    from oracle import torch_ref
    n_pix = 32768 * 1024 + 4096 + 3
    g = torch.Generator(device="cuda").manual_seed(91)
    x = 2 * torch.randn(n_pix, 2, device="cuda", generator=g)
    y = torch.randint(0, 2, (n_pix,), device="cuda", generator=g)
    y[torch.rand(n_pix, device="cuda", generator=g) < 0.05] = 255
    xt = x.clone().requires_grad_()
    losses = pl.LovaszSoftmaxV3(reduction="none", ignore_index=255)(xt, y)
    losses.sum().backward()
    xr = x.double().requires_grad_()
    want, _ = torch_ref.lovasz_per_class(xr, y, 255)
    want.sum().backward()
    np.testing.assert_allclose(losses.detach().cpu().numpy(), want.detach().cpu().numpy(), rtol=1e-5)
    # J is within one fp32 ulp of 1 over most of a row this long, and so are its differences
    # (csrc/lovasz_softmax.cu:124-147 forms them in fp32 as well): that ulp bounds the gradient error
    err = (xt.grad.double() - xr.grad).abs()
    assert err.max().item() <= 2.0 ** -23 and err.median().item() <= 2.0 ** -26, (err.median().item(), err.max().item())
    assert (xt.grad[y == 255] == 0).all()
    from pytorch_loss import _native
    _, jacc = _native.lovasz_forward(x, y, 255)
    assert (jacc[:, y == 255] == 0).all()
    np.testing.assert_allclose(jacc.double().sum(dim=1).cpu().numpy(), 1.0, rtol=1e-4)


def test_neighbouring_ops_full_size(pl):
    """Taylor cross entropy, the OHEM cross entropy, the target encoder and soft dice at the benchmark
    shapes, against fp64 torch library routines evaluated on the same GPU tensors, and the first
    image against the oracle."""
    import torch.nn.functional as F
    x, y = _seg_full("cfg2")
    xt = torch.from_numpy(x).cuda()
    yt = torch.from_numpy(y).cuda()
    n_valid = int((y != 255).sum())

    # target encoder: exact values everywhere
    enc = pl.OnehotEncoder(19, lb_smooth=0.1, ignore_idx=255)(yt)
    assert enc.shape == xt.shape
    valid = (yt != 255)
    assert torch.equal(enc.argmax(dim=1)[valid], yt[valid])
    assert (enc.sum(dim=1)[~valid] == 0).all()
    hot, cold = np.float32(1.0 - 0.1), np.float32(0.1 / 19)
    assert int((enc == float(hot)).sum()) == n_valid and int((enc == float(cold)).sum()) == 18 * n_valid
    assert np.array_equal(enc[:1].cpu().numpy(), oracle.onehot(y[:1], 19, 0.1, 255))
    del enc

    # Taylor cross entropy: -log of the order-4 series ratio, with torch ops in fp64 on one image at a time
    leaf = xt.clone().requires_grad_()
    loss = pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="sum")(leaf, yt)
    want = 0.0
    for i in range(xt.shape[0]):
        xd = xt[i:i + 1].double()
        f = 1 + xd + xd ** 2 / 2 + xd ** 3 / 6 + xd ** 4 / 24
        want += F.nll_loss((f / f.sum(dim=1, keepdim=True)).log(), yt[i:i + 1], ignore_index=255, reduction="sum").item()
    assert abs(loss.item() - want) <= 1e-5 * abs(want)
    loss.backward()
    g = leaf.grad
    assert (g.permute(0, 2, 3, 1)[~valid] == 0).all()
    want_g = oracle.taylor_ce_backward(x[:1], y[:1], 4, 255, np.float32(1.0))
    assert np.abs(g[:1].cpu().numpy() - want_g).max() <= 1e-5 * np.abs(want_g).max()
    del leaf, g, loss

    # OHEM cross entropy: the fused forward against torch's cross entropy on the relabelled batch
    n_min = y.size // 16
    leaf = xt.clone().requires_grad_()
    loss = pl.OhemCELoss(score_thresh=0.7, n_min=n_min, ignore_index=255)(leaf, yt)
    new_labels = pl.score_ohem_label(xt, yt, 255, 0.7, n_min)
    kept = int((new_labels != 255).sum())
    assert n_min <= kept < n_valid
    want = sum(F.cross_entropy(xt[i:i + 1].double(), new_labels[i:i + 1], ignore_index=255, reduction="sum").item()
               for i in range(xt.shape[0])) / kept
    assert abs(loss.item() - want) <= 1e-5 * abs(want)
    loss.backward()
    gone = (new_labels == 255)
    assert (leaf.grad.permute(0, 2, 3, 1)[gone] == 0).all()
    rows = leaf.grad.permute(0, 2, 3, 1)[~gone].double().sum(dim=1)
    assert rows.abs().max().item() <= 1e-6 / kept * 19
    del leaf, rows

    # soft dice at (64, 1, 1024, 1024) as one row
    g = torch.Generator(device="cuda").manual_seed(3)
    dx = (torch.randn((64, 1, 1024, 1024), device="cuda", generator=g) * 2.0).requires_grad_()
    dy = (torch.rand(dx.shape, device="cuda", generator=g) < 0.3).float()
    for p in (1, 2):
        dx.grad = None
        loss = pl.SoftDiceLossV3(p=p, smooth=1.0)(dx, dy)
        loss.backward()
        q = torch.sigmoid(dx.detach().double())
        numer = 2 * (q * dy).sum() + 1.0
        denor = (q.pow(p) + dy.double().pow(p)).sum() + 1.0
        want = (1 - numer / denor).item()
        assert abs(loss.item() - want) <= 1e-5 * abs(want)
        want_g = p * q.pow(p) * (1 - q) * numer / denor ** 2 - 2 * dy * q * (1 - q) / denor
        assert (dx.grad.double() - want_g).abs().max().item() <= 1e-5 * want_g.abs().max().item()
        del q, want_g
