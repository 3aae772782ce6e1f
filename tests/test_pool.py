"""Earliest-spike pooling: the numpy oracle against the reference's own formulation run through
PyTorch on the CPU (pad with 1e5, -maxpool(-x), autograd), and -- on the GPU -- the HIP kernels
against the oracle, bit for bit."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import closed_form as cf

CASES = [
    # B, H, W, C, Kh, Kw, Sh, Sw, same
    (2, 8, 8, 5, 2, 2, 2, 2, True),        # the example networks' 2x2 / 2
    (2, 9, 7, 3, 3, 3, 2, 2, True),        # ResNet stem pool, odd sizes: padding on both sides
    (1, 6, 10, 4, 3, 2, 1, 1, True),       # overlapping windows, stride 1
    (2, 7, 9, 2, 2, 3, 2, 3, False),       # VALID, ragged: trailing rows / columns are dropped
    (1, 5, 5, 1, 5, 5, 5, 5, True),        # one window over the whole image
]


def reference_formula(x, Kh, Kw, Sh, Sw, same, pad_value=1e5):
    """SNN_TC_Modules.py:215-246 with torch ops; returns (y, dx for upstream gradient g)."""
    xt = torch.from_numpy(x).requires_grad_(True)
    xp = xt
    if same:
        (top, bottom), (left, right) = cf.same_pad(x.shape[1], Kh, Sh), cf.same_pad(x.shape[2], Kw, Sw)
        xp = F.pad(xt, (0, 0, left, right, top, bottom), value=pad_value)
    y = -F.max_pool2d(-xp.permute(0, 3, 1, 2), (Kh, Kw), (Sh, Sw)).permute(0, 2, 3, 1)
    return xt, y


@pytest.mark.parametrize("B,H,W,C,Kh,Kw,Sh,Sw,same", CASES)
def test_oracle_matches_the_reference_formula(B, H, W, C, Kh, Kw, Sh, Sw, same):
    rng = np.random.default_rng(H * 100 + W)
    x = np.exp(rng.random((B, H, W, C))).astype(np.float32)          # no ties
    x[rng.random(x.shape) < 0.1] = np.float32(1e5)                   # never-fired pixels tie with the padding
    y, arg, pad = cf.min_pool(x, Kh, Kw, Sh, Sw, same)
    xt, yt = reference_formula(x, Kh, Kw, Sh, Sw, same)
    assert tuple(yt.shape) == y.shape
    assert np.array_equal(yt.detach().numpy(), y)
    g = rng.standard_normal(y.shape).astype(np.float32)
    g[y >= 1e5] = 0.0                    # windows without a spike carry no gradient (their source is masked upstream)
    yt.backward(torch.from_numpy(g))
    dx = cf.min_pool_grad(g, arg, x.shape, Kh, Kw, Sh, Sw, pad)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-6, atol=1e-7)


def test_first_position_wins_a_tie():
    x = np.full((1, 2, 2, 1), 3.0, np.float32)
    y, arg, pad = cf.min_pool(x, 2, 2, 2, 2, same=False)
    assert y.item() == 3.0 and arg.item() == 0
    dx = cf.min_pool_grad(np.ones_like(y), arg, x.shape, 2, 2, 2, 2, pad)
    assert dx.ravel().tolist() == [1.0, 0.0, 0.0, 0.0]


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,W,C,Kh,Kw,Sh,Sw,same", CASES + [(4, 32, 32, 64, 2, 2, 2, 2, True),
                                                              (2, 112, 112, 64, 3, 3, 2, 2, True)])
def test_hip_pooling_matches_the_oracle(B, H, W, C, Kh, Kw, Sh, Sw, same):
    import snntc_amd as snn
    rng = np.random.default_rng(C * 7 + H)
    x = np.exp(rng.random((B, H, W, C))).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = np.float32(1e5)
    x[0, :2, :2, :] = np.float32(2.0)                                # ties inside a window
    y, arg, pad = cf.min_pool(x, Kh, Kw, Sh, Sw, same)
    layer = snn.SNN_maxpool2d((Kh, Kw), (Sh, Sw), 'SAME' if same else 'VALID')
    xt = torch.from_numpy(x).to("cuda:0").requires_grad_(True)
    yt = layer(xt)
    assert np.array_equal(yt.detach().cpu().numpy(), y)
    g = rng.standard_normal(y.shape).astype(np.float32)
    yt.backward(torch.from_numpy(g).to("cuda:0"))
    dx = cf.min_pool_grad(g, arg, x.shape, Kh, Kw, Sh, Sw, pad)
    assert np.array_equal(xt.grad.cpu().numpy(), dx)
    # the op-level call returns the recorded positions themselves
    y2, arg2 = snn.min_pool(xt.detach(), (Kh, Kw), (Sh, Sw), pad, y.shape[1:3])
    assert np.array_equal(arg2.cpu().numpy(), arg) and np.array_equal(y2.cpu().numpy(), y)


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,W,C", [(32, 7, 7, 512), (3, 5, 9, 7), (2, 1, 1, 4), (1, 14, 14, 256)])
def test_hip_global_min_pool_matches_the_oracle(B, H, W, C):
    """SNN_globalminpool2d = one VALID window the size of the image (the ImageNet-shaped net's head):
    values and the routed gradient against the pooling oracle, bit for bit; never-fired channels
    (all pixels at 1e5) and ties included."""
    import snntc_amd as snn
    rng = np.random.default_rng(H * 31 + C)
    x = np.exp(rng.random((B, H, W, C))).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = np.float32(1e5)
    x[0, :, :, 0] = np.float32(1e5)                                  # a channel without any spike
    x[-1, :, :, -1] = np.float32(2.5)                                # every pixel ties: the first one wins
    y, arg, pad = cf.min_pool(x, H, W, H, W, same=False)
    xt = torch.from_numpy(x).to("cuda:0").requires_grad_(True)
    yt = snn.SNN_globalminpool2d()(xt)
    assert tuple(yt.shape) == (B, C)
    assert np.array_equal(yt.detach().cpu().numpy(), y.reshape(B, C))
    assert np.array_equal(yt.detach().cpu().numpy(), x.min(axis=(1, 2)))
    g = rng.standard_normal((B, C)).astype(np.float32)
    yt.backward(torch.from_numpy(g).to("cuda:0"))
    dx = cf.min_pool_grad(g.reshape(B, 1, 1, C), arg, x.shape, H, W, H, W, pad)
    assert np.array_equal(xt.grad.cpu().numpy(), dx)


@pytest.mark.gpu
def test_pooling_argument_errors():
    import snntc_amd as snn
    x = torch.ones((1, 4, 4, 2), device="cuda:0")
    with pytest.raises(ValueError):
        snn.min_pool(x, (2, 2), (2, 2), (2, 0), (3, 2))              # padding as large as the kernel
    with pytest.raises(ValueError):
        snn.min_pool(x, (2, 2), (2, 2), (0, 0), (4, 2))              # a window wholly outside the image
    with pytest.raises(ValueError):
        snn.min_pool(x, (0, 2), (2, 2), (0, 0), (2, 2))


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,W,C,pads", [(2, 5, 7, 3, (1, 1, 1, 1)), (3, 8, 8, 32, (0, 1, 0, 1)),
                                          (2, 32, 32, 64, (1, 1, 1, 1)), (1, 224, 224, 3, (2, 3, 2, 3)),
                                          (2, 4, 6, 8, (3, 0, 0, 2))])
def test_hip_padding_matches_constant_pad(B, H, W, C, pads):
    """SAME padding with MAX_SPIKE_TIME in one pass, and its gradient (the interior of the upstream)."""
    import snntc_amd as snn
    top, bottom, left, right = pads
    rng = np.random.default_rng(H + C)
    x = torch.from_numpy(rng.random((B, H, W, C)).astype(np.float32)).to("cuda:0").requires_grad_(True)
    ref = F.pad(x.detach(), (0, 0, left, right, top, bottom), value=1e5)
    out = snn.SnnPadTime.apply(x, top, bottom, left, right, 1e5)
    assert torch.equal(out, ref)
    g = torch.from_numpy(rng.standard_normal(tuple(ref.shape)).astype(np.float32)).to("cuda:0")
    out.backward(g)
    assert torch.equal(x.grad, g[:, top:top + H, left:left + W, :])
    # the layer takes the same path
    conv = snn.SNN_conv(C, 4, 3, 1, 'SAME')
    assert torch.equal(conv.prepare_input(x.detach()), F.pad(x.detach(), (0, 0, 1, 1, 1, 1), value=1e5))

