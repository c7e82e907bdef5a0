"""Pins the CPU oracle (oracle/plo_oracle.c and oracle/torch_ref.py) WITHOUT the reference.

The reference holds no golden vectors for this path, so each oracle function is
pinned against what the mathematics fixes: library routines it must reduce to
(F.cross_entropy, BCE-with-logits, Categorical entropy), brute force from the
definition (Lovasz by explicit set Jaccard), fp64 autograd of an independently
written formulation, and invariants (gradient rows summing to zero, exact zeros
at ignored pixels).  None of the checks retypes the oracle's own formula.
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import synth, torch_ref

torch.manual_seed(0)


def _seg_inputs(seed, shape, n_cls, ignore=255, frac=0.2, dtype=np.float64, std=2.0):
    logits = synth.normal(seed, 1, shape, 0.0, std, dtype=dtype)
    labels = synth.seg_labels(seed, shape[:1] + shape[2:], n_cls, ignore, frac)
    return logits, labels


SEG_SHAPES = [(2, 19, 8, 8), (3, 2, 5, 7), (4, 3, 1, 9), (5, 64), (2, 227, 3, 3), (1, 33, 4, 4, 2)]


# ------------------------------------------------------------------ LSR ----

@pytest.mark.parametrize("shape", SEG_SHAPES)
@pytest.mark.parametrize("smooth", [0.0, 0.1, 0.35])
def test_lsr_forward_is_library_cross_entropy_identity(shape, smooth):
    x, y = _seg_inputs(3, shape, shape[1])
    xt, yt = torch.from_numpy(x), torch.from_numpy(y)
    n_cls = shape[1]
    # loss = CE_with_label_smoothing(s) - (s/C) * CE_plain   (target weight 1-s, others s/C)
    want = (F.cross_entropy(xt, yt, ignore_index=255, reduction="none", label_smoothing=smooth)
            - smooth / n_cls * F.cross_entropy(xt, yt, ignore_index=255, reduction="none"))
    got = oracle.lsr_forward(x, y, 255, smooth)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-12)
    assert (got[y == 255] == 0).all()
    if smooth == 0.0:
        np.testing.assert_allclose(
            got, F.cross_entropy(xt, yt, ignore_index=255, reduction="none").numpy(), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape", SEG_SHAPES)
def test_lsr_backward_matches_autograd_of_library_identity(shape):
    x, y = _seg_inputs(4, shape, shape[1])
    smooth, n_cls = 0.1, shape[1]
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch.from_numpy(y)
    go = torch.from_numpy(synth.normal(9, 5, y.shape, 0.0, 1.0, dtype=np.float64))
    loss = (F.cross_entropy(xt, yt, ignore_index=255, reduction="none", label_smoothing=smooth)
            - smooth / n_cls * F.cross_entropy(xt, yt, ignore_index=255, reduction="none"))
    (loss * go).sum().backward()
    got = oracle.lsr_backward(x, y, 255, smooth, go.numpy())
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-10, atol=1e-12)
    # invariants: ignored -> exactly 0 ; valid rows sum to 0 under unit upstream gradient
    unit = oracle.lsr_backward(x, y, 255, smooth)
    ign = np.expand_dims(y == 255, 1)
    assert (np.broadcast_to(ign, unit.shape) * unit == 0).all()
    np.testing.assert_allclose(unit.sum(axis=1), 0.0, atol=1e-12)


def test_lsr_f32_tracks_f64_and_torch_flow():
    x, y = _seg_inputs(5, (2, 19, 16, 16), 19, dtype=np.float32)
    l32 = oracle.lsr_forward(x, y, 255, 0.1)
    l64 = oracle.lsr_forward(x.astype(np.float64), y, 255, 0.1)
    np.testing.assert_allclose(l32, l64, rtol=2e-6, atol=2e-6)
    xt = torch.from_numpy(x).requires_grad_()
    lt = torch_ref.lsr(xt, torch.from_numpy(y), 0.1, "none", 255)
    np.testing.assert_allclose(lt.detach().numpy(), l32, rtol=2e-6, atol=2e-6)
    lt.sum().backward()
    np.testing.assert_allclose(xt.grad.numpy(), oracle.lsr_backward(x, y, 255, 0.1), rtol=0, atol=2e-6)


def test_lsr_reductions():
    x, y = _seg_inputs(6, (2, 5, 6, 6), 5)
    per = oracle.lsr_forward(x, y, 255, 0.1)
    assert np.isclose(oracle.reduce_pixels(per, y, "sum", 255), per.sum())
    assert np.isclose(oracle.reduce_pixels(per, y, "mean", 255), per.sum() / (y != 255).sum())
    assert oracle.reduce_pixels(per, y, "none", 255) is per
    for red in ("mean", "sum"):
        want = torch_ref.lsr(torch.from_numpy(x), torch.from_numpy(y), 0.1, red, 255).item()
        assert np.isclose(oracle.reduce_pixels(per, y, red, 255), want, rtol=1e-12)
    # everything ignored: 0/0 -> NaN, as in every version of the reference
    y_all = np.full_like(y, 255)
    assert np.isnan(oracle.reduce_pixels(oracle.lsr_forward(x, y_all, 255, 0.1), y_all, "mean", 255))


# ---------------------------------------------------------------- focal ----

def _focal_inputs(seed, shape, soft, dtype=np.float64):
    x = synth.normal(seed, 1, shape, -1.0, 3.0, dtype=dtype)
    if soft:
        y = synth.uniform01(seed, 2, int(np.prod(shape))).reshape(shape).astype(dtype)
    else:
        y = synth.bernoulli(seed, 2, shape, 0.3).astype(dtype)
    return x, y


def _textbook_focal(x, y, alpha, gamma):
    """Lin et al. with soft labels: -|y-p|^g [a y log p + (1-a)(1-y) log(1-p)], via logsigmoid."""
    p = torch.sigmoid(x)
    return -(y - p).abs().pow(gamma) * (alpha * y * F.logsigmoid(x) + (1 - alpha) * (1 - y) * F.logsigmoid(-x))


@pytest.mark.parametrize("soft", [False, True])
def test_focal_gamma0_is_weighted_bce_with_logits(soft):
    x, y = _focal_inputs(7, (3, 4, 5, 6), soft)
    xt, yt = torch.from_numpy(x), torch.from_numpy(y)
    alpha = 0.25
    ones, zeros = torch.ones_like(xt), torch.zeros_like(xt)
    want = (alpha * yt * F.binary_cross_entropy_with_logits(xt, ones, reduction="none")
            + (1 - alpha) * (1 - yt) * F.binary_cross_entropy_with_logits(xt, zeros, reduction="none"))
    got = oracle.focal_forward(x, y, alpha, 0.0)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("soft", [False, True])
@pytest.mark.parametrize("alpha,gamma", [(0.25, 2.0), (0.5, 1.0), (0.75, 3.0), (0.1, 0.5), (0.25, 2.5)])
def test_focal_forward_backward_vs_textbook_autograd(soft, alpha, gamma):
    x, y = _focal_inputs(8, (2, 3, 7, 5), soft)
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch.from_numpy(y)
    go = torch.from_numpy(synth.normal(2, 5, x.shape, 0.0, 1.0, dtype=np.float64))
    want = _textbook_focal(xt, yt, alpha, gamma)
    np.testing.assert_allclose(oracle.focal_forward(x, y, alpha, gamma), want.detach().numpy(),
                               rtol=1e-10, atol=1e-13)
    (want * go).sum().backward()
    got = oracle.focal_backward(x, y, alpha, gamma, go.numpy())
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-8, atol=1e-11)


def test_focal_symmetry_and_extreme_logits():
    x, y = _focal_inputs(9, (4, 50), True)
    a = oracle.focal_forward(x, y, 0.3, 2.0)
    b = oracle.focal_forward(-x, 1.0 - y, 0.7, 2.0)
    np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-14)
    xe = np.array([-120.0, -60.0, -30.0, 0.0, 30.0, 60.0, 120.0], dtype=np.float32)
    for lab in (0.0, 1.0):
        ye = np.full_like(xe, lab)
        l32 = oracle.focal_forward(xe, ye, 0.25, 2.0)
        g32 = oracle.focal_backward(xe, ye, 0.25, 2.0)
        assert np.isfinite(l32).all() and np.isfinite(g32).all()
        want = _textbook_focal(torch.from_numpy(xe).double(), torch.from_numpy(ye).double(), 0.25, 2.0)
        np.testing.assert_allclose(l32, want.numpy(), rtol=1e-5, atol=1e-6)


def test_focal_f32_tracks_f64_and_torch_flow():
    x, y = _focal_inputs(10, (2, 8, 16, 16), False, dtype=np.float32)
    l32 = oracle.focal_forward(x, y, 0.25, 2.0)
    l64 = oracle.focal_forward(x.astype(np.float64), y.astype(np.float64), 0.25, 2.0)
    np.testing.assert_allclose(l32, l64, rtol=1e-5, atol=1e-6)
    xt = torch.from_numpy(x).requires_grad_()
    lt = torch_ref.focal(xt, torch.from_numpy(y), 0.25, 2, "none")
    np.testing.assert_allclose(lt.detach().numpy(), l32, rtol=1e-5, atol=1e-6)
    lt.sum().backward()
    np.testing.assert_allclose(xt.grad.numpy(), oracle.focal_backward(x, y, 0.25, 2.0), rtol=0, atol=2e-6)


# -------------------------------------------------------------- lmargin ----

def _independent_lmargin(x, y, lam, ignore):
    """Per-pixel loss from library pieces only: the target channel is physically
    removed (no masking constant), the margin term is written as
    (lam/2) * ( CE(uniform, q) - H(q) ) with q = softmax of the remaining C-1 logits."""
    n_cls = x.shape[1]
    xf = x.movedim(1, -1).reshape(-1, n_cls)
    yf = y.reshape(-1)
    valid = yf != ignore
    xv, yv = xf[valid], yf[valid]
    keep = torch.arange(n_cls).unsqueeze(0).expand(len(yv), -1)
    keep = keep[keep != yv.unsqueeze(1)].reshape(len(yv), n_cls - 1)
    rest = torch.gather(xv, 1, keep)
    uniform = torch.full_like(rest, 1.0 / (n_cls - 1))
    ce_uniform = F.cross_entropy(rest, uniform, reduction="none")
    entropy = torch.distributions.Categorical(logits=rest).entropy()
    per_valid = F.cross_entropy(xv, yv, reduction="none") + lam / 2.0 * (ce_uniform - entropy)
    out = torch.zeros(len(yf), dtype=x.dtype)
    out = out.index_put((valid.nonzero().reshape(-1),), per_valid)
    return out.reshape(y.shape)


@pytest.mark.parametrize("shape", SEG_SHAPES)
@pytest.mark.parametrize("lam", [0.0, 0.3, 1.5])
def test_lmargin_vs_independent_formulation(shape, lam):
    x, y = _seg_inputs(11, shape, shape[1])
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch.from_numpy(y)
    want = _independent_lmargin(xt, yt, lam, 255)
    got = oracle.lmargin_forward(x, y, lam, 255)
    np.testing.assert_allclose(got, want.detach().numpy(), rtol=1e-10, atol=1e-11)
    if lam == 0.0:
        np.testing.assert_allclose(
            got, F.cross_entropy(torch.from_numpy(x), yt, ignore_index=255, reduction="none").numpy(),
            rtol=1e-12, atol=1e-12)
    go = torch.from_numpy(synth.normal(3, 5, y.shape, 0.0, 1.0, dtype=np.float64))
    (want * go).sum().backward()
    gg = oracle.lmargin_backward(x, y, lam, 255, go.numpy())
    np.testing.assert_allclose(gg, xt.grad.numpy(), rtol=1e-9, atol=1e-11)
    unit = oracle.lmargin_backward(x, y, lam, 255)
    assert (unit * np.broadcast_to(np.expand_dims(y == 255, 1), unit.shape) == 0).all()
    np.testing.assert_allclose(unit.sum(axis=1), 0.0, atol=1e-11)


def test_lmargin_dominant_target_stays_finite():
    # target logit far above the rest: the non-target softmax must not underflow to 0/0
    x = np.zeros((1, 4, 1, 3), dtype=np.float32)
    x[0, 2] = 200.0
    x[0, 0, 0, 1] = -150.0
    y = np.full((1, 1, 3), 2, dtype=np.int64)
    l = oracle.lmargin_forward(x, y, 0.3, 255)
    g = oracle.lmargin_backward(x, y, 0.3, 255)
    assert np.isfinite(l).all() and np.isfinite(g).all()
    want = _independent_lmargin(torch.from_numpy(x).double(), torch.from_numpy(y), 0.3, 255)
    np.testing.assert_allclose(l, want.numpy(), rtol=1e-5, atol=1e-6)


def test_lmargin_f32_tracks_f64_and_torch_flow():
    x, y = _seg_inputs(12, (2, 19, 16, 16), 19, dtype=np.float32)
    l32 = oracle.lmargin_forward(x, y, 0.3, 255)
    l64 = oracle.lmargin_forward(x.astype(np.float64), y, 0.3, 255)
    np.testing.assert_allclose(l32, l64, rtol=3e-6, atol=3e-6)
    xt = torch.from_numpy(x).requires_grad_()
    lt = torch_ref.lmargin(xt, torch.from_numpy(y), 0.3, "none", 255, per_pixel=True)
    np.testing.assert_allclose(lt.detach().numpy(), l32, rtol=3e-6, atol=3e-6)
    lt.sum().backward()
    np.testing.assert_allclose(xt.grad.numpy(), oracle.lmargin_backward(x, y, 0.3, 255), rtol=0, atol=3e-6)
    for red in ("mean", "sum"):
        want = torch_ref.lmargin(torch.from_numpy(x), torch.from_numpy(y), 0.3, red, 255).item()
        assert np.isclose(oracle.reduce_pixels(l32, y, red, 255), want, rtol=1e-5)


# --------------------------------------------------------------- lovasz ----

def _softmax(x):
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def _lovasz_brute_force(x, y, ignore):
    """Straight from the definition: sort errors descending, and for every prefix S_k of that
    order take the Jaccard loss of the binary problem in which exactly the pixels of S_k are
    mispredicted:  J(S_k) = 1 - |GT \\ S_k| / |GT u S_k|.  loss_c = sum_k e_(k) (J(S_k) - J(S_{k-1}))."""
    n_cls = x.shape[1]
    probs = np.moveaxis(_softmax(x), 1, 0).reshape(n_cls, -1)
    labels = y.reshape(-1)
    valid = [i for i in range(labels.size) if labels[i] != ignore]
    out = np.zeros(n_cls)
    for c in range(n_cls):
        gt = {i for i in valid if labels[i] == c}
        errs = {i: abs((1.0 if i in gt else 0.0) - probs[c, i]) for i in valid}
        order = sorted(valid, key=lambda i: (-errs[i], i))
        seen, prev, total = set(), 0.0, 0.0
        for i in order:
            seen.add(i)
            jac = 1.0 - len(gt - seen) / len(gt | seen)
            total += errs[i] * (jac - prev)
            prev = jac
        out[c] = total
    return out


@pytest.mark.parametrize("shape,frac", [((1, 3, 2, 3), 0.0), ((2, 4, 3, 3), 0.3), ((1, 5, 4, 4), 0.2),
                                         ((3, 2, 2, 2), 0.5)])
def test_lovasz_forward_matches_set_definition(shape, frac):
    x, y = _seg_inputs(13, shape, shape[1], frac=frac)
    got, jacc = oracle.lovasz_forward(x, y, 255)
    np.testing.assert_allclose(got, _lovasz_brute_force(x, y, 255), rtol=1e-12, atol=1e-13)
    assert jacc.shape == (shape[1], y.size)
    assert (jacc[:, y.reshape(-1) == 255] == 0).all()
    # the Jaccard differences of one class telescope to J(all valid pixels) = 1 when any pixel is valid
    if (y != 255).any():
        np.testing.assert_allclose(jacc.sum(axis=1), 1.0, rtol=1e-12)


def test_lovasz_special_cases():
    x, y = _seg_inputs(14, (2, 4, 3, 3), 3, frac=0.2)   # class 3 never appears
    assert not (y == 3).any()
    losses, _ = oracle.lovasz_forward(x, y, 255)
    p3 = np.moveaxis(_softmax(x), 1, 0).reshape(4, -1)[3][y.reshape(-1) != 255]
    assert np.isclose(losses[3], p3.max(), rtol=1e-12)       # absent class: J == 1 => loss = max prob
    y_all = np.full_like(y, 255)
    losses, jacc = oracle.lovasz_forward(x, y_all, 255)
    assert (losses == 0).all() and (jacc == 0).all()
    # perfect prediction -> loss ~ 0 for present classes
    yy = synth.randint(1, 1, (1, 3, 3), 0, 3)
    big = np.full((1, 3, 3, 3), -40.0)
    np.put_along_axis(big, yy[:, None], 40.0, axis=1)
    losses, _ = oracle.lovasz_forward(big, yy, 255)
    assert np.abs(losses).max() < 1e-12


def test_lovasz_loss_is_invariant_to_tie_order():
    # build exact ties: two pixels with identical logits but different labels
    x = synth.normal(15, 1, (1, 3, 1, 6), 0.0, 1.0, dtype=np.float64)
    x[..., 1] = x[..., 0]
    x[..., 3] = x[..., 2]
    y = np.array([[[0, 1, 2, 2, 1, 0]]], dtype=np.int64)
    base, _ = oracle.lovasz_forward(x, y, 255)
    perm = [1, 0, 3, 2, 4, 5]
    swapped, _ = oracle.lovasz_forward(x[..., perm], y[..., perm], 255)
    np.testing.assert_allclose(base, swapped, rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("shape", [(2, 5, 4, 4), (1, 19, 6, 6), (3, 3, 2, 5)])
def test_lovasz_backward_vs_autograd_and_finite_differences(shape):
    x, y = _seg_inputs(16, shape, shape[1], frac=0.2)
    w = synth.normal(4, 5, (shape[1],), 0.5, 1.0, dtype=np.float64)
    xt = torch.from_numpy(x).requires_grad_()
    lt = torch_ref.lovasz(xt, torch.from_numpy(y), "none", 255)
    losses, jacc = oracle.lovasz_forward(x, y, 255)
    np.testing.assert_allclose(losses, lt.detach().numpy(), rtol=1e-12, atol=1e-13)
    (lt * torch.from_numpy(w)).sum().backward()
    got = oracle.lovasz_backward(w, x, y, jacc, 255)
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-9, atol=1e-12)
    ign = np.broadcast_to(np.expand_dims(y == 255, 1), got.shape)
    assert (got[ign] == 0).all()
    # central finite differences on a handful of coordinates (the loss is piecewise linear in p;
    # step small enough not to cross a sort boundary for generic inputs)
    flat = x.reshape(-1)
    eps = 1e-7
    for k in list(range(0, flat.size, max(1, flat.size // 7)))[:7]:
        xp, xm = flat.copy(), flat.copy()
        xp[k] += eps
        xm[k] -= eps
        fp = (oracle.lovasz_forward(xp.reshape(shape), y, 255)[0] * w).sum()
        fm = (oracle.lovasz_forward(xm.reshape(shape), y, 255)[0] * w).sum()
        assert abs((fp - fm) / (2 * eps) - got.reshape(-1)[k]) < 1e-6


def test_lovasz_f32_tracks_f64():
    x, y = _seg_inputs(17, (2, 19, 16, 16), 19, dtype=np.float32)
    l32, j32 = oracle.lovasz_forward(x, y, 255)
    l64, j64 = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(l32, l64, rtol=1e-5, atol=1e-6)
    w = np.ones(19, dtype=np.float32)
    g32 = oracle.lovasz_backward(w, x, y, j32, 255)
    g64 = oracle.lovasz_backward(w.astype(np.float64), x.astype(np.float64), y, j64, 255)
    # fp32 softmax can reorder near-ties relative to fp64, moving single Jaccard differences
    assert np.abs(g32 - g64).max() < 2e-3
    assert np.median(np.abs(g32 - g64)) < 1e-7


# ----------------------------------------------------------- generators ----

def test_synth_is_bit_stable():
    a = synth.normal(15, 1, (4, 5), 0.0, 2.0)
    assert a.dtype == np.float32
    # known-answer values: any change of the generator changes every committed fixture
    assert synth._splitmix64(np.array([0], dtype=np.uint64))[0] == np.uint64(0xE220A8397B1DCDAF)
    b = synth.normal(15, 1, (4, 5), 0.0, 2.0)
    assert (a.view(np.uint32) == b.view(np.uint32)).all()
    big = synth.normal(1, 1, (1 << 16,), 0.0, 1.0, dtype=np.float64)
    assert abs(big.mean()) < 0.02 and abs(big.std() - 1.0) < 0.02
    lb = synth.seg_labels(15, (8, 64, 64), 19)
    frac = (lb == 255).mean()
    assert 0.03 < frac < 0.07 and lb[lb != 255].max() == 18 and lb.min() == 0
    z = synth.workload("cfg5", scale=1 / 16)
    counts = np.bincount(z["labels"][z["labels"] != 255], minlength=19)
    assert counts[0] > counts[5] > counts[18] > 0
