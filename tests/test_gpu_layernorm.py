"""GPU parity of the channel layer norm (through the C ABI) against the CPU oracle.
Outputs are O(1): 1e-5 absolute. The backward's values grow like |x|^3, so it is held to 1e-5 of
the tensor's largest magnitude. 16-bit tensors: one rounding of the storage type."""
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


# (N, C, M): every kernel shape -- all channels in one wave (C <= 32), channels split over the four
# waves with every slot count, one pixel per lane (ragged M, C > 512), contiguous rows (M == 1),
# and the two-sweep kernel (C > 1024)
SHAPES = [(2, 1, 64), (2, 3, 130), (2, 8, 64), (1, 19, 1000), (2, 32, 66), (2, 33, 64), (1, 64, 300), (2, 65, 128),
          (1, 100, 77), (1, 128, 256), (1, 200, 64), (1, 256, 130), (1, 384, 64), (1, 512, 128), (1, 513, 64),
          (1, 768, 70), (1, 1024, 64), (1, 1025, 40), (5, 96, 1), (3, 2000, 1), (2, 64, 49), (3, 40, 3),
          # planes of odd length, 4096 pixels or more: pixel groups per image, the last lane of an image with 1 .. 3 pixels
          (2, 19, 4225), (3, 64, 4097), (2, 100, 4099), (1, 768, 4098), (2, 40, 4331)]


@pytest.mark.parametrize("shape", SHAPES)
def test_function_matches_oracle(pl, shape):
    x = synth.normal(121, 1, shape, 0.3, 1.5)
    g = synth.normal(121, 2, shape, 0.0, 1.0)
    xt = torch.from_numpy(x).cuda().requires_grad_()
    out = pl.LayerNormV3Func.apply(xt, 1e-6)
    assert out.shape == xt.shape and out.dtype == torch.float32
    want = oracle.layer_norm_forward(x.astype(np.float64), 1e-6)
    if shape[1] > 1:
        assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-5
    else:       # a single channel: var = 0, the output is (x - x) / sqrt(eps) = 0 exactly
        assert (out == 0).all()
    out.backward(torch.from_numpy(g).cuda())
    want_g = oracle.layer_norm_backward(g.astype(np.float64), x.astype(np.float64), 1e-6)
    err = np.abs(xt.grad.cpu().numpy() - want_g).max()
    assert err <= 1e-5 * np.abs(want_g).max(), (err, np.abs(want_g).max())


def test_backward_known_answers(pl):
    """The hand-worked values of csrc/layer_norm.cu:214 that pin the oracle (tests/test_oracle_layernorm.py),
    straight through the HIP path: pixels (1,3), (0,2), (3,1) at eps = 0 and the constant pixel (2,2) at eps = 1/4."""
    x = torch.tensor([[[1.0, 0.0], [3.0, 2.0]], [[3.0, 2.0], [1.0, 2.0]]], device="cuda")
    for eps, want in ((0.0, {(0, 0): (0.5, -5.5), (0, 1): (-1.0, -2.0), (1, 0): (-5.5, 0.5)}),
                      (0.25, {(1, 1): (-1.0, -1.0)}),
                      (3.0, {(0, 0): (1.75, -10.25), (1, 0): (-10.25, 1.75)})):
        xt = x.clone().requires_grad_()
        pl.LayerNormV3Func.apply(xt, eps).backward(torch.ones_like(x))
        got = xt.grad.cpu().numpy()
        for (n, m), chans in want.items():
            np.testing.assert_allclose(got[n, :, m], np.array(chans), rtol=2e-6, err_msg=str((eps, n, m)))


@pytest.mark.parametrize("shape", [(3, 1317, 57), (2, 1500, 1), (4, 3000, 1), (1, 2048, 33)])
def test_long_slices_with_an_outlying_first_channel(pl, shape):
    """More than 1024 channels, and (N, C) rows: one pass over the slice with shifted sums. A first channel far from
    the slice's mean must not cost accuracy (the shift is the mean of the first few channels, not the first one)."""
    x = synth.normal(123, 1, shape, 0.3, 1.5)
    x[:, 0, :] += 12.0
    out = pl.LayerNormV3Func.apply(torch.from_numpy(x).cuda(), 1e-6).cpu().numpy()
    want = oracle.layer_norm_forward(x.astype(np.float64), 1e-6)
    assert np.abs(out - want).max() <= 1e-5, np.abs(out - want).max()


def test_large_common_offset_keeps_accuracy(pl):
    x = synth.normal(122, 1, (2, 64, 256), 1000.0, 0.5)
    out = pl.LayerNormV3Func.apply(torch.from_numpy(x).cuda(), 1e-6).cpu().numpy()
    want = oracle.layer_norm_forward(x.astype(np.float64), 1e-6)
    assert np.abs(out - want).max() <= 5e-4        # input spacing 6e-5 over a spread of 0.5


@pytest.mark.parametrize("affine", [True, False])
def test_module_on_nchw(pl, affine):
    shape = (2, 48, 12, 10)
    x = synth.normal(123, 1, shape, 0.0, 2.0)
    xt = torch.from_numpy(x).cuda()
    mod = pl.LayerNormV3(48, affine=affine, eps=1e-5).cuda()
    if affine:
        assert mod.weight.shape == (1, 48, 1) and mod.bias.shape == (1, 48, 1)
        with torch.no_grad():
            mod.weight.copy_(torch.linspace(0.5, 1.5, 48).view(1, 48, 1))
            mod.bias.copy_(torch.linspace(-1, 1, 48).view(1, 48, 1))
    else:
        assert mod.weight is None and mod.bias is None
    y = mod(xt)
    want = oracle.layer_norm_forward(x.reshape(2, 48, -1).astype(np.float64), 1e-5)
    if affine:
        want = want * np.linspace(0.5, 1.5, 48).reshape(1, 48, 1) + np.linspace(-1, 1, 48).reshape(1, 48, 1)
    assert y.shape == shape and np.abs(y.detach().cpu().numpy().reshape(2, 48, -1) - want).max() <= 1e-5
    with pytest.raises(RuntimeError, match="only supports gpu mode"):
        pl.LayerNormV3Func.apply(torch.zeros(1, 4, 4), 1e-6)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
# (the last four: 385..768 channels in the forms that hold two pixels per lane - planes of 4096 pixels and more that are
# not whole groups of four pixels, in groups per image, and fp16 with more than 512 channels on aligned planes)
@pytest.mark.parametrize("shape", [(2, 19, 64), (1, 96, 260), (1, 256, 128), (1, 600, 66), (4, 80, 1), (2, 30, 7),
                                   (1, 600, 4098), (2, 448, 4102), (1, 768, 4097), (1, 640, 256)])
def test_16bit(pl, dt, shape):
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dt]
    x = synth.normal(124, 1, shape, 0.3, 1.5)
    g = synth.normal(124, 2, shape, 0.0, 1.0)
    xt = torch.from_numpy(x).cuda().to(dt).requires_grad_()
    gt = torch.from_numpy(g).cuda().to(dt)
    xr = xt.detach().float().cpu().numpy().astype(np.float64)
    gr = gt.float().cpu().numpy().astype(np.float64)
    out = pl.LayerNormV3Func.apply(xt, 1e-6)
    assert out.dtype == dt
    want = oracle.layer_norm_forward(xr, 1e-6)
    assert (np.abs(out.detach().float().cpu().numpy() - want) <= ulp * np.abs(want) + 1e-6).all()
    out.backward(gt)
    want_g = oracle.layer_norm_backward(gr, xr, 1e-6)
    assert xt.grad.dtype == dt
    assert (np.abs(xt.grad.float().cpu().numpy() - want_g) <= ulp * np.abs(want_g) + 1e-5 * np.abs(want_g).max()).all()
    with torch.autocast("cuda", dtype=dt):
        assert pl.LayerNormV3Func.apply(xt, 1e-6).dtype == torch.float32      # custom_fwd(cast_inputs=float32)


def test_full_size_properties(pl):
    """(8, 256, 128, 128) fp32: zero mean and unit variance per pixel, and the first image against the oracle."""
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((8, 256, 128 * 128), device="cuda", generator=g) * 2.0 + 0.7
    y = pl.LayerNormV3Func.apply(x, 1e-6)
    assert y.mean(dim=1).abs().max().item() < 1e-5
    assert (y.var(dim=1, unbiased=False) - 1).abs().max().item() < 1e-4
    want = oracle.layer_norm_forward(x[:1].cpu().numpy().astype(np.float64), 1e-6)
    assert np.abs(y[:1].cpu().numpy() - want).max() <= 1e-5
