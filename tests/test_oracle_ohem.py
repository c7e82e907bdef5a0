"""Pins the oracle's online-hard-example-mining functions WITHOUT the reference.

scores: the library softmax gathered at the label.  select: (a) the rule evaluated per pixel from
its definition by counting (position of pixel i in the ascending stable order = number of pixels
with a smaller score + number of equal scores at smaller indices), which involves no sort at all;
(b) torch.sort(stable=True) as an independent sort; (c) counting invariants.  Ties are the point:
score sets with a few distinct values and many exact 1.0 are included.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth


def _scores(seed, n, kind):
    u = synth.uniform01(seed, 1, n).astype(np.float32)
    if kind == "smooth":
        return u
    if kind == "coarse":                      # 8 distinct values: long runs of ties
        return (np.floor(u * 8) / 8).astype(np.float32)
    if kind == "saturated":                   # most pixels at exactly 1.0, like a converged model
        return np.where(u < 0.9, np.float32(1.0), u).astype(np.float32)
    raise ValueError(kind)


def _by_counting(scores, labels, ignore, thresh, n_min):
    s = scores.astype(np.float64).ravel()
    out = labels.copy().ravel()
    if n_min >= s.size:
        return out.reshape(labels.shape)
    for i in range(s.size):
        pos = int((s < s[i]).sum() + (s[:i] == s[i]).sum())
        if pos >= n_min and scores.ravel()[i] > np.float32(thresh):
            out[i] = ignore
    return out.reshape(labels.shape)


@pytest.mark.parametrize("shape", [(2, 19, 8, 8), (3, 2, 5, 7), (5, 64), (2, 33, 3, 3)])
def test_ohem_scores_are_library_softmax_at_the_label(shape):
    x = synth.normal(41, 1, shape, 0.0, 2.0, dtype=np.float64)
    y = synth.seg_labels(41, shape[:1] + shape[2:], shape[1], 255, 0.2)
    got = oracle.ohem_scores(x, y, 255)
    p = torch.softmax(torch.from_numpy(x), 1)
    idx = torch.from_numpy(np.where(y == 255, 0, y)).unsqueeze(1)
    want = p.gather(1, idx).squeeze(1).numpy()
    want[y == 255] = 1.0
    assert np.abs(got - want).max() < 1e-14
    got32 = oracle.ohem_scores(x.astype(np.float32), y, 255)
    assert got32.dtype == np.float32 and np.abs(got32 - want).max() < 1e-6
    assert (got32[y == 255] == 1.0).all()


@pytest.mark.parametrize("kind", ["smooth", "coarse", "saturated"])
@pytest.mark.parametrize("n_min", [0, 1, 7, 100, 299, 300, 1000])
@pytest.mark.parametrize("thresh", [0.0, 0.5, 0.7, 1.0])
def test_ohem_select_matches_the_definition_by_counting(kind, n_min, thresh):
    n = 300
    s = _scores(43, n, kind)
    y = synth.randint(43, 2, (n,), 0, 19).astype(np.int64)
    y[synth.bernoulli(43, 3, (n,), 0.1)] = 255
    got = oracle.ohem_select(s, y, 255, thresh, n_min)
    assert np.array_equal(got, _by_counting(s, y, 255, thresh, n_min))


@pytest.mark.parametrize("kind", ["smooth", "coarse", "saturated"])
def test_ohem_select_matches_torch_stable_sort(kind):
    n = 50_000
    s = _scores(44, n, kind)
    y = synth.randint(44, 2, (n,), 0, 19).astype(np.int64)
    for n_min, thresh in [(n // 16, 0.7), (n // 2, 0.3), (n - 1, 0.0), (10, 0.99)]:
        order = torch.sort(torch.from_numpy(s), stable=True).indices.numpy()
        want = y.copy()
        tail = order[n_min:]
        want[tail[s[tail] > np.float32(thresh)]] = 255
        assert np.array_equal(oracle.ohem_select(s, y, 255, thresh, n_min), want)


def test_ohem_select_invariants():
    n = 20_000
    s = _scores(45, n, "saturated")
    y = synth.randint(45, 2, (n,), 0, 19).astype(np.int64)
    for n_min in (0, 500, 5000, 19_000):
        out = oracle.ohem_select(s, y, 255, 0.7, n_min)
        kept = out != 255
        assert np.array_equal(out[kept], y[kept])                      # labels are only ever set to ignore
        assert (s[~kept] > 0.7).all()                                  # only pixels above the threshold go
        # at least min(n_min, n) pixels stay, and everything at or under the threshold stays
        assert kept.sum() >= min(n_min, n) and kept[s <= 0.7].all()
        # exactly max(n_min, #(s <= thresh)) stay
        assert kept.sum() == max(n_min, int((s <= 0.7).sum()))
    assert np.array_equal(oracle.ohem_select(s, y, 255, 0.7, n), y)     # n_min >= P: unchanged
    assert np.array_equal(oracle.ohem_select(s, y, 255, 0.7, n + 5), y)


def test_ohem_score_label_composes():
    shape = (2, 19, 16, 16)
    x = synth.normal(46, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(46, (2, 16, 16), 19, 255, 0.05)
    out = oracle.ohem_score_label(x, y, 255, 0.2, 32)
    assert out.shape == y.shape and out.dtype == np.int64
    s = oracle.ohem_scores(x, y, 255)
    assert np.array_equal(out, _by_counting(s, y, 255, 0.2, 32))
