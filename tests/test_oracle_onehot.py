"""Pins the oracle's one-hot / smoothed-target encoder WITHOUT the reference: the library one_hot
for smooth = 0, the value set and per-pixel sums, zero columns at ignored pixels, and the tie to
the label-smoothed loss (loss = -sum_j target_j * log_softmax_j must equal the LSR oracle, which
is pinned separately against F.cross_entropy)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import synth

SHAPES = [(4, 6, 5), (3, 9), (7,), (2, 3, 4, 5)]


@pytest.mark.parametrize("shape", SHAPES)
def test_plain_one_hot_is_the_library_routine(shape):
    y = synth.randint(7, 1, shape, 0, 11)
    got = oracle.onehot(y, 11, 0.0, -1)
    want = F.one_hot(torch.from_numpy(y), 11).movedim(-1, 1).numpy().astype(np.float32)
    assert got.shape == (shape[0], 11) + tuple(shape[1:]) and got.dtype == np.float32
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("smooth", [0.0, 0.1, 0.35])
def test_smoothed_targets_values_sums_and_ignored_columns(shape, smooth):
    n_cls = 19
    y = synth.randint(8, 1, shape, 0, n_cls)
    y[synth.bernoulli(8, 2, shape, 0.2)] = 255
    got = oracle.onehot(y, n_cls, smooth, 255)
    pos, neg = np.float32(1.0 - smooth), np.float32(np.float32(smooth) / np.float32(n_cls))
    ign = np.expand_dims(y == 255, 1)
    assert (got[np.broadcast_to(ign, got.shape)] == 0).all()
    valid = ~np.broadcast_to(ign, got.shape)
    assert set(np.unique(got[valid]).tolist()) <= {float(pos), float(neg)}
    # the label's channel carries pos, and exactly one channel per valid pixel does
    at_label = np.take_along_axis(got, np.expand_dims(np.where(y == 255, 0, y), 1), 1).squeeze(1)
    assert (at_label[y != 255] == pos).all()
    if smooth < 0.5:
        assert ((got == pos).sum(axis=1)[y != 255] == 1).all()
    np.testing.assert_allclose(got.sum(axis=1)[y != 255], pos + (n_cls - 1) * neg, rtol=1e-6)   # = 1 - smooth/C


def test_targets_reproduce_the_label_smoothed_loss():
    shape = (2, 19, 6, 7)
    x = synth.normal(9, 1, shape, 0.0, 2.0, dtype=np.float64)
    y = synth.seg_labels(9, (2, 6, 7), 19, 255, 0.2)
    t = oracle.onehot(y, 19, 0.1, 255, dtype=np.float64)
    logp = torch.log_softmax(torch.from_numpy(x), 1).numpy()
    np.testing.assert_allclose(-(t * logp).sum(axis=1), oracle.lsr_forward(x, y, 255, 0.1), rtol=1e-6, atol=1e-9)


def test_out_of_range_label_matches_no_channel():
    y = np.array([[0, 5, -3, 2]])
    got = oracle.onehot(y, 3, 0.3, -1)
    assert (got[0, :, 1] == np.float32(0.1)).all() and (got[0, :, 2] == np.float32(0.1)).all()
