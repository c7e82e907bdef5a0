"""GPU parity of the online-hard-example-mining step (through the C ABI) against the CPU oracle.

The relabelling is integer work on given scores, so `plh_ohem_select_labels` is held bit-exact to
the oracle on identical fp32 scores, with tie-heavy score sets, every boundary of n_min and tile
sizes around the kernels' 1024-pixel tiles.  The scores are floating point: 1e-6 absolute against
the fp32 oracle.  The fused call is then (a) bit-exact to the oracle's selection applied to the
GPU's own scores and (b) equal to the all-oracle result except at pixels whose score lies within
2e-6 of a decision boundary (the threshold or the n_min-th smallest score), where no two fp32
softmax evaluations need agree.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth
from .test_gpu_parity import close_grad, dev, seg_inputs
from .test_oracle_ohem import _scores

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def native():
    from pytorch_loss import _native
    _native.load()
    return _native


SCORE_CASES = [
    ((2, 19, 64, 64), 255, 0.05),        # uniform tiles, 8 bytes per lane
    ((2, 19, 7, 9), 255, 0.1),           # one pixel per thread
    ((3, 2, 5, 8), -100, 0.2),
    ((37, 10), -100, 0.1),
    ((33, 100), -100, 0.1),              # (N, C) rows of 33..2048 channels: a wavefront per row, in registers
    ((9, 77), -100, 0.1),                #   (odd lengths element by element, others in 16-byte chunks)
    ((6, 1000), 255, 0.2),
    ((7, 201), 255, 0.1),
    ((70, 33), -100, 0.1),
    ((21, 136), 255, 0.1),
    ((5, 260), 255, 0.2),
    ((9, 264), 255, 0.1),                  # rows of 257..512 elements: 16 lanes per row
    ((7, 301), 255, 0.1),
    ((4, 1001), -100, 0.1),
    ((5, 1544), 255, 0.1),
    ((3, 2047), 255, 0.1),
    ((2, 2056), 255, 0.0),               # longer rows: a block per row, 16-byte chunks
    ((3, 4100), 255, 0.3),
    ((2, 4099), -100, 0.0),              #   odd length: element by element
    ((2, 50000), 255, 0.0),
    ((2, 33, 6, 7), 255, 0.2),
    ((2, 40, 16, 16), 255, 0.1),         # 33..256 channels: shared out over the wavefronts of a block
    ((1, 150, 12, 16), 255, 0.05),
    ((2, 256, 8, 8), 255, 0.1),
    ((2, 52, 8, 8), 255, 0.1),
    ((2, 65, 8, 8), 255, 0.1),
    ((1, 133, 8, 8), 255, 0.1),
    ((1, 171, 8, 8), 255, 0.1),
    ((2, 257, 8, 8), 255, 0.1),          # 257..512 channels: up to 64 slots per wavefront, half the pixels per lane
    ((1, 300, 9, 8), 255, 0.1),
    ((1, 449, 8, 8), -100, 0.2),
    ((1, 512, 8, 9), 255, 0.1),
    ((1, 513, 8, 8), 255, 0.1),          # one channel more: a lane per pixel
    ((2, 19, 65, 65), 255, 0.05),        # planes of odd length, 4096 pixels or more: tiles per image, four pixels
    ((3, 5, 71, 61), -100, 0.1),         #   per lane, the last lane of an image with 1 or 3 pixels; the widest
    ((2, 24, 4097, 1), 255, 0.1),        #   slices that take this form (24 channels fp32, 32 for 16-bit logits)
    ((2, 32, 65, 65), 255, 0.1),
    ((1, 25, 63, 65), 255, 0.1),
    ((2, 150, 65, 65), 255, 0.05),       # 33..256 channels on such planes: the split shape in tiles per image
    ((1, 33, 67, 63), -100, 0.1),
    ((1, 256, 4097, 1), 255, 0.1),
    ((2, 19, 16, 16), 255, 1.0),         # everything ignored
]


@pytest.mark.parametrize("shape,ignore,frac", SCORE_CASES)
@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
def test_scores_match_oracle(native, shape, ignore, frac, dt):
    x, y = seg_inputs(81, shape, ignore, frac)
    xt = dev(x).to(dt)
    got = native.ohem_scores(xt, dev(y), ignore).cpu().numpy()
    want = oracle.ohem_scores(xt.float().cpu().numpy(), y, ignore)
    assert got.dtype == np.float32 and got.shape == y.shape
    assert np.abs(got - want).max() <= 1e-6
    assert (got[y == ignore] == 1.0).all() and got.max() <= 1.0 and got.min() >= 0.0


@pytest.mark.parametrize("kind", ["smooth", "coarse", "saturated"])
@pytest.mark.parametrize("n", [1, 5, 1023, 1024, 1025, 4099, 70_001])
def test_select_is_bit_exact_on_given_scores(native, kind, n):
    s = _scores(82, n, kind)
    y = synth.randint(82, 2, (n,), 0, 19).astype(np.int64)
    y[synth.bernoulli(82, 3, (n,), 0.1)] = 255
    st, yt = dev(s), dev(y)
    for n_min in sorted({0, 1, 2, n // 16, n // 2, n - 1, n, n + 3, -1}):
        for thresh in (0.0, 0.5, 0.7, 0.875, 1.0):
            got = native.ohem_select_labels(st, yt, 255, thresh, n_min).cpu().numpy()
            want = oracle.ohem_select(s, y, 255, thresh, max(n_min, 0))
            assert np.array_equal(got, want), (kind, n, n_min, thresh, int((got != want).sum()))
    assert np.array_equal(yt.cpu().numpy(), y)          # the input labels are not touched


def test_select_all_equal_scores(native):
    n = 5000
    y = synth.randint(83, 2, (n,), 0, 19).astype(np.int64)
    for value in (1.0, 0.25):
        s = np.full((n,), value, dtype=np.float32)
        for n_min in (1, 1024, 1025, 4999):
            got = native.ohem_select_labels(dev(s), dev(y), 255, 0.1, n_min).cpu().numpy()
            assert np.array_equal(got, oracle.ohem_select(s, y, 255, 0.1, n_min))
            assert (got[:n_min] == y[:n_min]).all() and (got[n_min:] == 255).all()


def _near_boundary(scores, thresh, n_min, tol=2e-6):
    flat = np.sort(scores.ravel())
    near = np.abs(scores - np.float32(thresh)) <= tol
    if 0 < n_min < flat.size:
        near |= np.abs(scores - flat[n_min - 1]) <= tol
    return near


@pytest.mark.parametrize("shape,ignore,frac", SCORE_CASES)
@pytest.mark.parametrize("thresh,div", [(0.7, 16), (0.05, 16), (0.3, 2), (0.0, 4)])
def test_score_label_matches_oracle(native, shape, ignore, frac, thresh, div):
    x, y = seg_inputs(84, shape, ignore, frac)
    xt, yt = dev(x), dev(y)
    n_min = y.size // div
    got = native.ohem_score_label(xt, yt, ignore, thresh, n_min).cpu().numpy()
    own = native.ohem_scores(xt, yt, ignore).cpu().numpy()
    assert np.array_equal(got, oracle.ohem_select(own, y, ignore, thresh, n_min))
    s = oracle.ohem_scores(x, y, ignore)
    want = oracle.ohem_select(s, y, ignore, thresh, n_min)
    differ = got != want
    assert not (differ & ~_near_boundary(s, thresh, n_min)).any(), int(differ.sum())
    assert differ.mean() < 1e-3


def test_score_label_full_resolution(native):
    shape = (2, 19, 1024, 1024)
    x, y = seg_inputs(85, shape, 255, 0.05)
    x *= 2.0                                            # a sharper softmax: scores on both sides of 0.7
    xt, yt = dev(x), dev(y)
    n_min = y.size // 16
    got = native.ohem_score_label(xt, yt, 255, 0.7, n_min).cpu().numpy()
    own = native.ohem_scores(xt, yt, 255).cpu().numpy()
    assert np.array_equal(got, oracle.ohem_select(own, y, 255, 0.7, n_min))
    kept = got != 255
    assert np.array_equal(got[kept], y[kept]) and (own[~kept & (y != 255)] > 0.7).all()
    assert kept.sum() >= n_min and kept[(own <= 0.7) & (y != 255)].all()
    # a threshold that nothing reaches below n_min: the tie-ranked branch at full size
    got2 = native.ohem_score_label(xt, yt, 255, 1e-7, y.size // 2).cpu().numpy()
    assert np.array_equal(got2, oracle.ohem_select(own, y, 255, 1e-7, y.size // 2))


@pytest.mark.parametrize("which", ["ce", "lmargin"])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_ohem_modules(native, which, dt):
    import pytorch_loss as pl
    shape = (2, 19, 32, 32)
    x, y = seg_inputs(86, shape, 255, 0.05)
    xt = dev(x).to(dt).requires_grad_()
    xr = xt.detach().float().cpu().numpy()
    yt = dev(y)
    n_min = y.size // 16
    crit = (pl.OhemCELoss if which == "ce" else pl.OhemLargeMarginLoss)(score_thresh=0.3, n_min=n_min, ignore_index=255)
    with torch.autocast("cuda", dtype=dt, enabled=dt != torch.float32):
        loss = crit(xt, yt)
    new_labels = pl.score_ohem_label(xt, yt, 255, 0.3, n_min).cpu().numpy()
    assert (new_labels != y).any() and np.array_equal(yt.cpu().numpy(), y)
    if which == "ce":
        per = oracle.lsr_forward(xr.astype(np.float64), new_labels, 255, 0.0)
        grad_of = lambda g: oracle.lsr_backward(xr, new_labels, 255, 0.0, g)
        # plain cross entropy is what the reference's criterion computes (ohem_loss.py:20)
        ce = torch.nn.functional.cross_entropy(torch.from_numpy(xr).double(), torch.from_numpy(new_labels),
                                               ignore_index=255, reduction="mean").item()
        assert abs(loss.item() - ce) <= 1e-5 * abs(ce)
    else:
        per = oracle.lmargin_forward(xr.astype(np.float64), new_labels, 0.3, 255)
        grad_of = lambda g: oracle.lmargin_backward(xr, new_labels, 0.3, 255, g)
    n_valid = int((new_labels != 255).sum())
    want = per.sum() / n_valid
    assert abs(loss.item() - want) <= 1e-5 * abs(want)
    loss.backward()
    want_g = grad_of(np.float32(1.0 / n_valid))
    if dt == torch.float32:
        close_grad(xt.grad.cpu().numpy(), want_g, which)
    else:
        err = np.abs(xt.grad.float().cpu().numpy() - want_g) - (2.0 ** -7 * np.abs(want_g) + 1e-7)
        assert (err <= 0).all()
    # default n_min = numel // 16 (ohem_loss.py:23)
    crit2 = (pl.OhemCELoss if which == "ce" else pl.OhemLargeMarginLoss)(score_thresh=0.3)
    assert crit2.n_min is None and torch.isfinite(crit2(xt.detach(), yt)).item()


def test_ohem_refuses_cpu_tensors():
    import pytorch_loss as pl
    x = torch.randn(2, 5, 4, 4)
    y = torch.randint(0, 5, (2, 4, 4))
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.OhemCELoss(0.7)(x, y)


@pytest.mark.parametrize("which", ["ce", "lm"])
@pytest.mark.parametrize("case", ["n_min_covers_everything", "all_ignored", "huge_logit_gaps", "ragged", "deep",
                                  "split", "rows", "register_rows", "short_register_rows", "block_rows"])
def test_ohem_ce_fused_forward_edge_cases(native, case, which):
    """The one-pass forwards (scores and per-pixel loss from the same sums) against the oracle's
    relabelling followed by torch's cross entropy or the oracle's large-margin loss."""
    import pytorch_loss as pl
    # deep: more channels than the register-resident form holds; rows: (N, C) inputs
    shape = {"ragged": (2, 7, 9, 11), "deep": (2, 40, 6, 10), "split": (2, 150, 8, 16), "rows": (300, 23),
             "register_rows": (90, 1000), "short_register_rows": (203, 150), "block_rows": (40, 2500)}.get(
        case, (2, 19, 16, 24))
    x, y = seg_inputs(91, shape, 255, 0.05)
    n_min, thresh = y.size // 16, 0.3
    if case == "n_min_covers_everything":
        n_min = y.size + 5
    if case == "all_ignored":
        y[...] = 255
    if case == "huge_logit_gaps":
        x = x * 60.0            # softmax at the label underflows to 0 for many pixels; their loss is ~1e2
    xt = dev(x).requires_grad_()
    crit = (pl.OhemCELoss if which == "ce" else pl.OhemLargeMarginLoss)(score_thresh=thresh, n_min=n_min, ignore_index=255)
    loss = crit(xt, dev(y))
    new_labels = oracle.ohem_score_label(x, y, 255, thresh, n_min)
    if case == "n_min_covers_everything":
        assert np.array_equal(new_labels, y)
    n_valid = int((new_labels != 255).sum())
    if n_valid == 0:
        assert torch.isnan(loss).item()        # the mean over no pixels, as nn.CrossEntropyLoss gives it
        return
    if which == "ce":
        want = torch.nn.functional.cross_entropy(torch.from_numpy(x).double(), torch.from_numpy(new_labels),
                                                 ignore_index=255, reduction="mean").item()
        want_g = oracle.lsr_backward(x, new_labels, 255, 0.0, np.float32(1.0 / n_valid))
    else:
        want = oracle.lmargin_forward(x.astype(np.float64), new_labels, 0.3, 255).sum() / n_valid
        want_g = oracle.lmargin_backward(x, new_labels, 0.3, 255, np.float32(1.0 / n_valid))
    assert np.isfinite(loss.item()) and abs(loss.item() - want) <= 1e-5 * abs(want), (loss.item(), want)
    loss.backward()
    close_grad(xt.grad.cpu().numpy(), want_g, case)
    # the same loss as the two-step composition the reference runs (ohem_loss.py:41-45)
    if which == "lm":
        two_step = pl.LargeMarginSoftmaxV3(ignore_index=255, reduction="mean")(
            xt.detach(), pl.score_ohem_label(xt, dev(y), 255, thresh, n_min))
        assert abs(two_step.item() - loss.item()) <= 1e-6 * abs(loss.item())


@pytest.mark.parametrize("lam", [None, 0.3], ids=["ce", "lmargin"])
@pytest.mark.parametrize("shape,scale,thresh,div", [
    ((2, 19, 40, 52), 2.0, 0.7, 16),         # the n_min-th smallest score is below the threshold: "drop what exceeds it"
    ((2, 19, 40, 52), 2.0, 1e-7, 2),         # ... above it: ranks among the ties decide
    ((2, 5, 33, 31), 40.0, 0.7, 4),          # saturated softmaxes: valid pixels that score exactly 1, next to ignored ones
    ((3, 7, 9, 11), 40.0, 2.0, 8),           # a threshold nothing exceeds: every valid pixel stays
    ((500, 23), 3.0, 0.5, 16),
    ((64, 300), 6.0, 0.5, 8),
])
def test_kept_mask_is_the_relabelling(native, shape, scale, thresh, div, lam):
    """The forwards that hand their selection on as a byte mask: the mask is the relabelling of
    plh_ohem_score_label bit for bit (kept = new label is not ignore_index), loss and count are those of the entry
    points that write new labels, and the masked backward on the old labels is the backward on the new ones."""
    x = synth.normal(131, 1, shape, 0.0, scale)
    y = synth.seg_labels(131, shape[:1] + shape[2:], shape[1], 255, 0.1)
    xt, yt = dev(x), dev(y)
    n_min = y.size // div
    loss, n_valid, args, kept = native.ohem_ce_forward(xt, yt, 255, thresh, n_min, lam)
    new_labels = native.ohem_score_label(xt, yt, 255, thresh, n_min)
    assert torch.equal(kept[:y.size].view(y.shape).bool(), new_labels != 255)
    assert int(n_valid.item()) == int((new_labels != 255).sum().item())
    assert np.array_equal(yt.cpu().numpy(), y)                        # the labels are left alone
    lib = native.load()
    P, st = native._ptr, native._stream
    n, c = shape[0], shape[1]
    m = x.size // (n * c)
    scratch = torch.empty((2, y.size), device=xt.device)
    ws = torch.empty(int(lib.plh_ohem_ce_workspace_bytes(y.size)), dtype=torch.uint8, device=xt.device)
    out_labels = torch.empty_like(yt)
    loss2 = torch.empty((), device=xt.device)
    cnt2 = torch.empty((), dtype=torch.int64, device=xt.device)
    head = (P(xt), 0, P(yt), P(out_labels), P(scratch[0]), P(scratch[1]), P(loss2), P(cnt2), P(ws), ws.numel(), n, c, m, 255)
    rc = (lib.plh_ohem_ce_forward(*head, thresh, n_min, st()) if lam is None
          else lib.plh_ohem_lmargin_forward(*head, lam, thresh, n_min, st()))
    assert rc == 0
    assert torch.equal(out_labels, new_labels) and int(cnt2.item()) == int(n_valid.item())
    if int(n_valid.item()):
        # the same pixels, added up per block by another kernel when the threshold rule decides (the score kernel's
        # own sums): equal to rounding
        assert abs(loss2.item() - loss.float().item()) <= 1e-6 * abs(loss2.item())
    one = torch.ones((), device=xt.device)
    got = native.ohem_backward(args, kept, 255, one, n_valid, lam)
    if lam is None:
        want = native.lsr_backward_scaled(xt, new_labels, 255, 0.0, one, n_valid)
    else:
        want = native.lmargin_backward_scaled(xt, new_labels, lam, 255, one, n_valid)
    assert torch.equal(got, want)               # -0.0 == 0.0: a dropped pixel's products may carry a sign


@pytest.mark.parametrize("lam", [None, 0.3], ids=["ce", "lmargin"])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(2, 19, 32, 32), (2, 19, 40, 52), (2, 19, 65, 67), (3, 7, 9, 11), (500, 23), (2, 40, 24, 24)],
                         ids=["uniform", "general", "per_image", "one_pixel", "rows", "split"])
def test_threshold_rule_from_the_score_kernel_switches_exactly_at_n_min(native, shape, dt, lam):
    """The forwards with the byte mask take mask, sum and count from their score pass when at least n_min pixels
    score within the threshold, and from the selection otherwise: n_min one below, at and one above that number of
    pixels (and 0, and far above) give the relabelling of plh_ohem_score_label and the mean loss over it."""
    x = synth.normal(137, 1, shape, 0.0, 2.5)
    y = synth.seg_labels(137, shape[:1] + shape[2:], shape[1], 255, 0.1)
    xt, yt = dev(x).to(dt), dev(y)
    xw = xt.float().cpu().numpy()
    thresh = 0.6
    scores = native.ohem_scores(xt, yt, 255).cpu().numpy()
    within = int((np.minimum(scores, 1.0) <= thresh).sum())
    assert 2 < within < y.size - 2
    for n_min in (0, within - 1, within, within + 1, within + (y.size - within) // 2, y.size - 1):
        loss, n_valid, args, kept = native.ohem_ce_forward(xt, yt, 255, thresh, n_min, lam)
        new_labels = native.ohem_score_label(xt, yt, 255, thresh, n_min)
        assert torch.equal(kept[:y.size].view(y.shape).bool(), new_labels != 255), n_min
        assert int(n_valid.item()) == int((new_labels != 255).sum().item()), n_min
        if lam is None:
            want = torch.nn.functional.cross_entropy(torch.from_numpy(xw).double(), new_labels.cpu(), ignore_index=255,
                                                     reduction="mean").item()
        else:
            nl = new_labels.cpu().numpy()
            want = oracle.lmargin_forward(xw.astype(np.float64), nl, lam, 255).sum() / max(int((nl != 255).sum()), 1)
        tol = 1e-5 if dt == torch.float32 else 2.0 ** -8          # the loss comes back in the logits' type
        assert abs(loss.float().item() - want) <= tol * abs(want), (n_min, loss.item(), want)
        # with more than `within` positions below n_min, pixels above the threshold stay
        if n_min > within:
            assert int(n_valid.item()) >= min(n_min, int((y != 255).sum())) - int((y == 255).sum())
