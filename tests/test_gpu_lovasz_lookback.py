"""The decoupled look-back variant of the Lovasz sort passes (plh_lovasz_forward_lookback: tile descriptors and
chained waits instead of a histogram kernel and a row scan in front of every pass) must give the results of the
default passes bit for bit: same keys, same stable order, same Jaccard differences, same fixed-order loss sums."""
import numpy as np
import pytest
import torch

import oracle
from oracle import synth

from .test_gpu_parity import dev, seg_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def native():
    from pytorch_loss import _native
    _native.load()
    return _native


CASES = [
    # shape, logits scale, boost of the label's logit            what it exercises
    ((2, 5, 100, 100), 2.0, 0.0),          # several tiles per class, the last one ragged
    ((1, 4, 70, 64), 2.0, 0.0),            # a little over one tile
    ((2, 19, 64, 64), 2.0, 0.0),
    ((3, 7, 200, 300), 2.0, 0.0),          # 44 tiles per class: long chains of descriptors
    ((2, 400, 40, 50), 0.002, 0.0),        # near-uniform predictions: two passes per class
    ((2, 120, 40, 50), 0.3, 0.0),          # three passes
    ((2, 120, 40, 50), 1.0, 12.0),         # confident predictions: all four
    ((1, 3, 1024, 1100), 2.0, 0.0),        # rows of 1.1 M pixels: 275 tiles
]


@pytest.mark.parametrize("shape,scale,boost", CASES)
def test_look_back_variant_is_bit_identical(native, shape, scale, boost):
    n_cls = shape[1]
    y = synth.seg_labels(61, shape[:1] + shape[2:], n_cls, 255, 0.1)
    x = synth.normal(61, 1, shape, 0.0, scale)
    if boost:
        x = x + np.float32(boost) * np.moveaxis(np.eye(n_cls, dtype=np.float32)[np.where(y == 255, 0, y)], -1, 1)
    xt, yt = dev(x), dev(y)
    losses, jacc = native.lovasz_forward(xt, yt, 255)
    for _ in range(2):                                  # twice: tickets and descriptors are cleared per call
        losses_lb, jacc_lb = native.lovasz_forward(xt, yt, 255, look_back=True)
        assert not torch.isnan(losses_lb).any()
        assert torch.equal(losses_lb, losses)
        assert torch.equal(jacc_lb.view(torch.int32), jacc.view(torch.int32))
    l64, _ = oracle.lovasz_forward(x.astype(np.float64), y, 255)
    np.testing.assert_allclose(losses_lb.cpu().numpy(), l64, rtol=3e-4 if boost else 1e-5)
