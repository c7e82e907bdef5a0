"""Tensors of more than 2^31 (and, for 16-bit logits, 2^32) elements.

The kernels index with 64-bit offsets; nothing at benchmark size would notice a 32-bit wrap. A CPU
oracle cannot cover such tensors in seconds, so each test gathers a few thousand pixels (the first
and last ones, the ones whose elements sit on either side of every multiple of 2^31 elements, and
random ones), hands exactly those to the oracle as a small problem and compares; an address that
wrapped would read or write another pixel's values. Whole-tensor properties (exact counts, sums
against torch in fp64, exact zeros at ignored pixels) cover what sampling cannot.
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

IGN = 255


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    if torch.cuda.get_device_properties(0).total_memory < 100 * 2 ** 30:
        pytest.skip("needs ~50 GB of device memory")
    return pytorch_loss


@pytest.fixture(autouse=True)
def _release():
    yield
    torch.cuda.empty_cache()


def _sample(n_size, c, m_size, count=2048, seed=3):
    """(image index, pixel index) pairs worth checking in an (n_size, c, m_size) tensor."""
    rng = np.random.default_rng(seed)
    total = n_size * m_size
    flat = [np.arange(0, min(total, 600)), np.arange(max(0, total - 600), total), rng.integers(0, total, count)]
    n_idx = [f // m_size for f in flat]
    m_idx = [f % m_size for f in flat]
    elems = n_size * c * m_size
    for boundary in range(2 ** 31, elems, 2 ** 31):
        plane, m0 = divmod(boundary, m_size)          # the (image, channel) plane the boundary falls in
        around = np.arange(max(0, m0 - 300), min(m_size, m0 + 300))
        n_idx.append(np.full(around.shape, plane // c))
        m_idx.append(around)
    return np.concatenate(n_idx), np.concatenate(m_idx)


def _gather(t, n_idx, m_idx):
    """t (N, C, M) or (N, M) on the device -> numpy (1, C, S) or (1, S) of the sampled pixels."""
    ni = torch.from_numpy(n_idx).cuda()
    mi = torch.from_numpy(m_idx).cuda()
    if t.dim() == 2:
        return t[ni, mi].unsqueeze(0).cpu().numpy()
    return t[ni, :, mi].t().unsqueeze(0).contiguous().float().cpu().numpy()


def _seg_inputs(shape, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    n, c, m = shape
    x = torch.empty(shape, device="cuda", dtype=dtype)
    for i in range(n):                                 # image by image: bounded temporaries
        x[i] = (2 * torch.randn(c, m, device="cuda", generator=g)).to(dtype)
    y = torch.randint(0, c, (n, m), device="cuda", generator=g)
    y[torch.rand(n, m, device="cuda", generator=g) < 0.05] = IGN
    return x, y


SEG_SHAPES = {
    # block-uniform tiles, several images: element offsets pass 2^31 between images
    "uniform_f32": ((14, 19, 4096 * 2048), torch.float32),
    # one image, odd pixel count: the general addressing form, a plane straddles 2^31
    "ragged_f32": ((1, 19, 113100001), torch.float32),
    # 16-bit logits, 4 pixels per lane: more than 2^32 elements
    "uniform_bf16": ((27, 19, 4096 * 2048), torch.bfloat16),
}


@pytest.mark.parametrize("op", ["lsr", "lmargin", "taylor"])
@pytest.mark.parametrize("case", list(SEG_SHAPES))
def test_per_pixel_losses(pl, op, case):
    shape, dtype = SEG_SHAPES[case]
    n, c, m = shape
    assert n * c * m > 2 ** 31
    x, y = _seg_inputs(shape, dtype, seed=11)
    x.requires_grad_()
    if op == "lsr":
        crit = lambda red: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction=red, ignore_index=IGN)
        o_fwd = lambda a, b: oracle.lsr_forward(a, b, IGN, 0.1)
        o_bwd = lambda a, b, g: oracle.lsr_backward(a, b, IGN, 0.1, g)
    elif op == "lmargin":
        crit = lambda red: pl.LargeMarginSoftmaxV3(lam=0.3, reduction=red, ignore_index=IGN)
        o_fwd = lambda a, b: oracle.lmargin_forward(a, b, 0.3, IGN)
        o_bwd = lambda a, b, g: oracle.lmargin_backward(a, b, 0.3, IGN, g)
    else:
        crit = lambda red: pl.TaylorCrossEntropyLossV3(n=4, reduction=red, ignore_index=IGN)
        o_fwd = lambda a, b: oracle.taylor_ce(a, b, 4, IGN)
        o_bwd = lambda a, b, g: oracle.taylor_ce_backward(a, b, 4, IGN, g)

    per = crit("none")(x, y)
    gout = (torch.rand(n, m, device="cuda") + 0.5).to(dtype)      # autograd hands it over in the loss's type
    per.backward(gout)
    grad = x.grad
    x.grad = None
    assert per.dtype == dtype and grad.dtype == dtype and grad.shape == x.shape

    # whole tensor: exact zeros at ignored pixels and nowhere else, the reduced forms agree
    ign = y == IGN
    assert (per[ign] == 0).all() and (per[~ign] > 0).all()
    for i in range(n):
        assert (grad[i][:, ign[i]] == 0).all()
    n_valid = int((~ign).sum())
    with torch.no_grad():
        total = crit("sum")(x, y)
        mean = crit("mean")(x, y)
    if dtype == torch.float32:
        ref_total = per.detach().double().sum().item()
        assert abs(total.item() - ref_total) <= 1e-5 * ref_total
        assert abs(mean.item() - ref_total / n_valid) <= 1e-5 * ref_total / n_valid

    # sampled pixels against the oracle (fp32 arithmetic on the same stored values)
    n_idx, m_idx = _sample(n, c, m)
    xs, ys = _gather(x.detach(), n_idx, m_idx), _gather(y, n_idx, m_idx)
    gs = _gather(gout.float(), n_idx, m_idx)
    want, want_g = o_fwd(xs, ys), o_bwd(xs, ys, gs)
    got, got_g = _gather(per.detach().float(), n_idx, m_idx), _gather(grad, n_idx, m_idx)
    if dtype == torch.float32:
        assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
        assert np.abs(got_g - want_g).max() <= 1e-5
    else:                                               # results are rounded to bf16 on the way out
        assert np.all(np.abs(got - want) <= 2 ** -8 * np.abs(want) + 1e-6)
        assert np.all(np.abs(got_g - want_g) <= 2 ** -8 * np.abs(want_g) + 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_rows_of_few_channels(pl, dtype):
    """(N, C) logits (flattened channels-last segmentation): wavefronts move their 64 rows through LDS."""
    n, c = 113100001, 19
    assert n * c > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(29)
    x = torch.empty(n, c, device="cuda", dtype=dtype)
    step = 1 << 24
    for i in range(0, n, step):
        x[i:i + step] = (2 * torch.randn(min(step, n - i), c, device="cuda", generator=g)).to(dtype)
    y = torch.randint(0, c, (n,), device="cuda", generator=g)
    y[torch.rand(n, device="cuda", generator=g) < 0.05] = IGN
    x.requires_grad_()
    per = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="none", ignore_index=IGN)(x, y)
    gout = (torch.rand(n, device="cuda") + 0.5).to(dtype)
    per.backward(gout)
    ign = y == IGN
    assert (per[ign] == 0).all() and (per[~ign] > 0).all() and (x.grad[ign] == 0).all()
    rows = np.concatenate([np.arange(0, 600), np.arange(n - 600, n), np.random.default_rng(4).integers(0, n, 2048)]
                          + [np.arange(b // c - 300, b // c + 300) for b in range(2 ** 31, n * c, 2 ** 31)])
    it = torch.from_numpy(rows).cuda()
    xs, ys, gs = x.detach()[it].float().cpu().numpy(), y[it].cpu().numpy(), gout[it].float().cpu().numpy()
    want, want_g = oracle.lsr_forward(xs, ys, IGN, 0.1), oracle.lsr_backward(xs, ys, IGN, 0.1, gs)
    got, got_g = per.detach()[it].float().cpu().numpy(), x.grad[it].float().cpu().numpy()
    if dtype == torch.float32:
        assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
        assert np.abs(got_g - want_g).max() <= 1e-5
    else:
        assert np.all(np.abs(got - want) <= 2 ** -8 * np.abs(want) + 1e-6)
        assert np.all(np.abs(got_g - want_g) <= 2 ** -8 * np.abs(want_g) + 1e-6)


def test_long_rows(pl):
    """Vocabulary-sized rows, more than 2^31 elements in all: a block per row."""
    n, c = 43000, 50257
    assert n * c > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(31)
    x = torch.empty(n, c, device="cuda")
    for i in range(0, n, 4096):
        x[i:i + 4096] = 2 * torch.randn(min(4096, n - i), c, device="cuda", generator=g)
    y = torch.randint(0, c, (n,), device="cuda", generator=g)
    y[torch.rand(n, device="cuda", generator=g) < 0.05] = IGN
    x.requires_grad_()
    per = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="none", ignore_index=IGN)(x, y)
    gout = torch.rand(n, device="cuda") + 0.5
    per.backward(gout)
    rows = np.concatenate([np.arange(0, 8), np.arange(n - 8, n), np.arange(2 ** 31 // c - 4, 2 ** 31 // c + 4)])
    it = torch.from_numpy(rows).cuda()
    xs, ys, gs = x.detach()[it].cpu().numpy(), y[it].cpu().numpy(), gout[it].cpu().numpy()
    want, want_g = oracle.lsr_forward(xs, ys, IGN, 0.1), oracle.lsr_backward(xs, ys, IGN, 0.1, gs)
    assert np.all(np.abs(per.detach()[it].cpu().numpy() - want) <= 1e-5 * np.abs(want) + 1e-6)
    assert np.abs(x.grad[it].cpu().numpy() - want_g).max() <= 1e-5
    # every row's gradient sums to gout * (sumw - sum of the weights) = 0 for valid rows
    assert x.grad.sum(dim=1).abs().max().item() < 1e-4


@pytest.mark.parametrize("op", ["lsr", "lmargin"])
@pytest.mark.parametrize("shape", [(2_200_000, 1000), (14_500_000, 150)], ids=["wavefront_per_row", "16_lanes_per_row"])
def test_register_rows(pl, op, shape):
    """(N, C) rows that sit in a wavefront's registers, more than 2^31 elements in all."""
    n, c = shape
    assert n * c > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(33)
    x = torch.empty(n, c, device="cuda")
    step = 1 << 20
    for i in range(0, n, step):
        x[i:i + step] = 2 * torch.randn(min(step, n - i), c, device="cuda", generator=g)
    y = torch.randint(0, c, (n,), device="cuda", generator=g)
    y[torch.rand(n, device="cuda", generator=g) < 0.05] = IGN
    x.requires_grad_()
    if op == "lsr":
        per = pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="none", ignore_index=IGN)(x, y)
    else:
        per = pl.LargeMarginSoftmaxV3(lam=0.3, reduction="none", ignore_index=IGN)(x, y)
    gout = torch.rand(n, device="cuda") + 0.5
    per.backward(gout)
    mid = 2 ** 31 // c
    rows = np.concatenate([np.arange(0, 70), np.arange(n - 70, n), np.arange(mid - 70, mid + 70),
                           np.random.default_rng(5).integers(0, n, 1024)])
    it = torch.from_numpy(rows).cuda()
    xs, ys, gs = x.detach()[it].cpu().numpy(), y[it].cpu().numpy(), gout[it].cpu().numpy()
    if op == "lsr":
        want, want_g = oracle.lsr_forward(xs, ys, IGN, 0.1), oracle.lsr_backward(xs, ys, IGN, 0.1, gs)
    else:
        want, want_g = oracle.lmargin_forward(xs, ys, 0.3, IGN), oracle.lmargin_backward(xs, ys, 0.3, IGN, gs)
    assert np.all(np.abs(per.detach()[it].cpu().numpy() - want) <= 1e-5 * np.abs(want) + 1e-6)
    assert np.abs(x.grad[it].cpu().numpy() - want_g).max() <= 1e-5
    # the gradient of a valid row sums to 0 for both losses, and ignored rows are exact zeros
    assert x.grad.sum(dim=1).abs().max().item() < 1e-4
    assert (x.grad[y == IGN] == 0).all().item() and (per.detach()[y == IGN] == 0).all().item()


def test_focal(pl):
    numel = 2 ** 31 + 12345
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.empty(numel, device="cuda")
    half = numel // 2
    x[:half] = -2 + 1.5 * torch.randn(half, device="cuda", generator=g)
    x[half:] = -2 + 1.5 * torch.randn(numel - half, device="cuda", generator=g)
    y = (torch.rand(numel, device="cuda", generator=g) < 0.02).float()
    x.requires_grad_()
    per = pl.FocalLossV3(alpha=0.25, gamma=2, reduction="none")(x, y)
    per.sum().backward()
    idx = np.concatenate([np.arange(0, 600), np.arange(numel - 600, numel), np.arange(2 ** 31 - 300, 2 ** 31 + 300),
                          np.random.default_rng(1).integers(0, numel, 4096)])
    it = torch.from_numpy(idx).cuda()
    xs, ys = x.detach()[it].cpu().numpy(), y[it].cpu().numpy()
    want = oracle.focal_forward(xs, ys, 0.25, 2.0)
    want_g = oracle.focal_backward(xs, ys, 0.25, 2.0, None)
    got, got_g = per.detach()[it].cpu().numpy(), x.grad[it].cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-7)
    assert np.abs(got_g - want_g).max() <= 1e-5
    with torch.no_grad():
        mean = pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean")(x, y)
    ref = per.detach().double().mean().item()
    assert abs(mean.item() - ref) <= 1e-5 * ref


def test_one_hot(pl):
    n, c, m = 14, 19, 4096 * 2048
    g = torch.Generator(device="cuda").manual_seed(7)
    y = torch.randint(0, c, (n, m), device="cuda", generator=g)
    y[torch.rand(n, m, device="cuda", generator=g) < 0.05] = IGN
    out = pl.OnehotEncoder(c, lb_smooth=0.1, ignore_idx=IGN)(y)
    assert out.shape == (n, c, m) and out.numel() > 2 ** 31
    n_idx, m_idx = _sample(n, c, m)
    want = oracle.onehot(_gather(y, n_idx, m_idx), c, 0.1, IGN)
    assert np.array_equal(_gather(out, n_idx, m_idx).view(np.uint32), want.view(np.uint32))
    # every pixel's channels add up to the same constant, ignored pixels to zero
    sums = out.sum(dim=1)
    assert (sums[y == IGN] == 0).all()
    assert (sums[y != IGN] - (0.9 + 18 * 0.1 / 19)).abs().max().item() < 1e-6


def test_taylor_softmax(pl):
    n, c, m = 14, 19, 4096 * 2048
    x, _ = _seg_inputs((n, c, m), torch.float32, seed=13)
    x.requires_grad_()
    out = pl.TaylorSoftmaxV3(dim=1, n=4)(x)
    gout = torch.empty_like(out)
    for i in range(n):
        gout[i] = torch.rand(c, m, device="cuda") - 0.5
    out.backward(gout)
    assert (out.detach().sum(dim=1) - 1).abs().max().item() < 1e-5
    n_idx, m_idx = _sample(n, c, m)
    xs, gs = _gather(x.detach(), n_idx, m_idx), _gather(gout, n_idx, m_idx)
    want = oracle.taylor_forward(xs, 1, 4, False)
    want_g = oracle.taylor_backward(gs, xs, 1, 4, False)
    assert np.abs(_gather(out.detach(), n_idx, m_idx) - want).max() <= 1e-6
    assert np.abs(_gather(x.grad, n_idx, m_idx) - want_g).max() <= 1e-5


def test_layer_norm(pl):
    n, c, m = 9, 256, 1024 * 1024
    assert n * c * m > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(17)
    x = torch.empty(n, c, m, device="cuda")
    for i in range(n):
        x[i] = 3 * torch.randn(c, m, device="cuda", generator=g) + 1
    x.requires_grad_()
    out = pl.LayerNormV3Func.apply(x, 1e-6)
    gout = torch.empty_like(out)
    for i in range(n):
        gout[i] = torch.rand(c, m, device="cuda", generator=g) - 0.5
    out.backward(gout)
    assert out.detach().mean(dim=1).abs().max().item() < 1e-5
    n_idx, m_idx = _sample(n, c, m, count=1024)
    xs, gs = _gather(x.detach(), n_idx, m_idx), _gather(gout, n_idx, m_idx)
    want = oracle.layer_norm_forward(xs.astype(np.float64), 1e-6)
    want_g = oracle.layer_norm_backward(gs.astype(np.float64), xs.astype(np.float64), 1e-6)
    assert np.abs(_gather(out.detach(), n_idx, m_idx) - want).max() <= 1e-5
    got_g = _gather(x.grad, n_idx, m_idx)
    assert np.abs(got_g - want_g).max() <= 1e-5 * max(1.0, np.abs(want_g).max())


def test_soft_dice(pl):
    batch, length = 3, 2 ** 30 + 4097              # rows start at odd offsets, the last one beyond 2^31
    g = torch.Generator(device="cuda").manual_seed(19)
    x = torch.empty(batch, length, device="cuda")
    y = torch.empty(batch, length, device="cuda")
    for i in range(batch):
        x[i] = torch.randn(length, device="cuda", generator=g)
        y[i] = (torch.rand(length, device="cuda", generator=g) < 0.3).float()
    x.requires_grad_()
    loss = pl.SoftDiceLossV3Func.apply(x, y, 1, 1.0)
    assert loss.shape == (batch,)
    loss.sum().backward()
    # the defining expression, sums in fp64 row by row
    want_rows, stats = [], []
    for i in range(batch):
        p = torch.sigmoid(x.detach()[i]).double()
        numer = 2 * (p * y[i]).sum() + 1.0
        denor = p.sum() + y[i].double().sum() + 1.0
        want_rows.append((1 - numer / denor).item())
        stats.append((numer.item(), denor.item()))
        del p
    assert np.allclose(loss.detach().cpu().numpy(), np.array(want_rows), rtol=1e-5)
    # gradient of sampled elements: d/dx [1 - numer/denor] = -(2 y denor - numer) / denor^2 * s(1-s)
    idx = np.concatenate([np.arange(0, 300), np.arange(length - 300, length), np.random.default_rng(2).integers(0, length, 2048)])
    it = torch.from_numpy(idx).cuda()
    for i in range(batch):
        xs, ys = x.detach()[i][it].double(), y[i][it].double()
        s = torch.sigmoid(xs)
        numer, denor = stats[i]
        ref = -(2 * ys * denor - numer) / denor ** 2 * s * (1 - s)
        got = x.grad[i][it].double()
        assert (got - ref).abs().max().item() <= 1e-5 * max(ref.abs().max().item(), 1e-12)


def test_ohem(pl):
    n, c, m = 14, 19, 4096 * 2048
    x, y = _seg_inputs((n, c, m), torch.float32, seed=23)
    n_min = n * m // 16
    crit = pl.OhemCELoss(score_thresh=0.7, n_min=n_min, ignore_index=IGN)
    x.requires_grad_()
    loss = crit(x, y)
    loss.backward()
    # the reference's rule on torch's own softmax and sort (pytorch_loss/ohem_loss.py:22-30)
    with torch.no_grad():
        valid = y != IGN
        lse = torch.empty(n, m, device="cuda")
        picked = torch.empty(n, m, device="cuda")
        for i in range(n):
            lse[i] = torch.logsumexp(x[i], dim=0)
            picked[i] = x[i].gather(0, y[i].clamp(0, c - 1).unsqueeze(0))[0]
        ce = (lse - picked)
        scores = torch.exp(-ce)
        sc_valid = scores[valid]
        kth = torch.kthvalue(sc_valid, n_min + 1).values.item() if n_min < sc_valid.numel() else float("inf")
        thresh = max(0.7, kth)
        # pixels strictly above the threshold go; ties at the threshold are resolved by sorted position, so
        # the kept count is only pinned when the threshold is the constant one or untied
        kept = valid & (scores <= thresh)
        ref = (ce[kept].double().sum() / kept.sum()).item()
    assert abs(loss.item() - ref) <= 2e-5 * ref
    # the gradient lives on kept pixels only and its rows sum to zero
    gsum = torch.zeros(n, m, device="cuda")
    for i in range(n):
        gsum[i] = x.grad[i].sum(dim=0)
        assert (x.grad[i][:, ~kept[i] & (scores[i] > thresh * (1 + 1e-5))] == 0).all()
    assert gsum.abs().max().item() < 1e-6
