"""GPU parity of the one-hot / smoothed-target encoder (through the C ABI) against the CPU oracle:
the outputs are selections between three fp32 constants, so the bar is bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu

CASES = [
    # (label shape, classes)                     execution shape
    ((2, 64, 64), 19),                           # plane after plane, 16-byte stores
    ((2, 7, 9), 19),                             # odd row length: one pixel per thread
    ((3, 5, 8), 2),
    ((2, 3, 6), 19),                             # row length 18: two pixels per thread
    ((37,), 10),                                 # (N,) labels -> (N, C)
    ((33,), 100),                                # more than 32 classes, m_size = 1
    ((2, 6, 8), 33),                             # more than 32 classes, 16-byte row stores
    ((2, 5, 7), 227),
    ((1, 2, 3, 4), 64),
    ((4, 1024, 256), 19),
    ((2, 1028, 1024), 3),                        # planes of more than 2^20 pixels go chunk by chunk, the last one short
    ((1, 2048, 1025), 5),                        #   (2 and 3 chunks)
    ((3, 65, 65), 19),                           # planes of odd length: 16-byte stores from 4-byte boundaries, the last
    ((2, 513, 513), 4),                          #   lane of a plane with 1 .. 3 pixels
    ((5, 257), 40),
    ((2, 1023, 2), 7),
]


@pytest.fixture(scope="module")
def pl():
    import pytorch_loss
    from pytorch_loss import _native
    _native.load()
    return pytorch_loss


@pytest.mark.parametrize("shape,n_cls", CASES)
@pytest.mark.parametrize("smooth,ignore", [(0.0, -1), (0.1, 255), (0.4, 0)])
def test_onehot_is_bit_exact(pl, shape, n_cls, smooth, ignore):
    y = synth.randint(95, 1, shape, 1 if ignore == 0 else 0, n_cls)
    if ignore >= 0:
        y[synth.bernoulli(95, 2, shape, 0.15)] = ignore
    yt = torch.from_numpy(y).cuda()
    got = pl.convert_to_one_hot_cu(yt, n_cls, smooth, ignore)
    want = oracle.onehot(y, n_cls, smooth, ignore)
    assert got.dtype == torch.float32 and tuple(got.shape) == want.shape and not got.requires_grad
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    enc = pl.OnehotEncoder(n_cls, lb_smooth=smooth, ignore_idx=ignore)
    assert torch.equal(enc(yt), got)
    assert torch.equal(pl.OnehotEncoder(n_cls, smooth, ignore, check=False)(yt), got)
    if smooth == 0.0:
        assert torch.equal(pl.convert_to_one_hot(yt, n_cls, ignore), got)


def test_onehot_range_errors_and_surface(pl):
    y = torch.tensor([[0, 2, 5], [1, 1, 0]], device="cuda")
    with pytest.raises(RuntimeError, match="less than min_len"):
        pl.convert_to_one_hot_cu(y, 3)
    with pytest.raises(RuntimeError, match="more than 0"):
        pl.convert_to_one_hot_cu(torch.tensor([[0, -2]], device="cuda"), 3)
    # the same labels pass once the offending value is the ignore index, or with the check off
    ok = pl.convert_to_one_hot_cu(y, 3, 0.0, 5)
    assert (ok[:, :, 2].cpu() == torch.tensor([[0.0, 0.0, 0.0], [1.0, 0.0, 0.0]])).all()
    loose = pl.OnehotEncoder(3, check=False)(y)
    assert (loose[0, :, 2] == 0).all()                 # label 5 of 3 classes matches no channel
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.convert_to_one_hot_cu(torch.zeros(2, 3, dtype=torch.long), 3)
    with pytest.raises(RuntimeError, match="kLong"):
        pl.convert_to_one_hot_cu(torch.zeros(2, 3, dtype=torch.int32, device="cuda"), 3)
    assert pl.convert_to_one_hot_cu(torch.zeros(0, 4, dtype=torch.long, device="cuda"), 3).shape == (0, 3, 4)


def test_onehot_targets_feed_a_soft_label_loss(pl):
    """The encoder's output is what the label-smoothed loss weighs log-probabilities with."""
    shape = (2, 19, 32, 32)
    x = synth.normal(96, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(96, (2, 32, 32), 19, 255, 0.1)
    xt, yt = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    t = pl.OnehotEncoder(19, lb_smooth=0.1, ignore_idx=255)(yt)
    via_targets = -(t * torch.log_softmax(xt.double(), 1)).sum(1)
    direct = pl.LSRCrossEntropyFunctionV3.apply(xt, yt, 0.1, 255)
    assert torch.allclose(via_targets.float(), direct, rtol=1e-5, atol=1e-6)
