"""Layer chaining: a conv or pooling layer that also writes its spike times into the padded input of the
conv layer after it, and a conv backward pass that stores the gradient of the un-padded image directly.
Both must give the bits of the separate padding / cropping passes they replace
(SNN_conv.__call__, SNN_TC_Modules.py:147-170)."""
import numpy as np
import pytest
import torch

from helpers import conv_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


@pytest.mark.parametrize("seed,B,H,W,C,Kc,K,S,dist", [
    (0, 3, 10, 10, 32, 32, 3, 1, "baseline"),      # channel-lane dX kernel, merged patch sort
    (1, 2, 9, 13, 64, 48, 3, 1, "reftest"),        # non-square image
    (2, 4, 8, 8, 3, 16, 3, 1, "baseline"),         # few input channels: channel lanes, the wavefront in parts
    (3, 2, 11, 11, 40, 32, 3, 2, "baseline"),      # stride 2: uneven SAME padding
    (4, 2, 12, 12, 16, 8, 5, 1, "reftest"),        # 5x5 kernel, two pixels of padding: patch-space dX + col2im
    (5, 300, 8, 8, 32, 64, 3, 1, "baseline"),      # a launch large enough for the filtered scan
    (6, 2, 9, 70, 8, 16, 3, 1, "baseline"),        # eight channels, rows of two 64-pixel tiles
])
def test_conv_ops_with_a_second_destination_and_a_gradient_window(seed, B, H, W, C, Kc, K, S, dist):
    import snntc_amd as snn
    x, xpad, w, p, g = conv_case(seed, B, H, W, C, Kc, K, K, S, S, True, True, dist)
    top, left = (xpad.shape[1] - H) // 2, (xpad.shape[2] - W) // 2      # SAME: the smaller half goes in front
    X, Wt, G = t(xpad), t(w), t(g)
    ref = snn.snncv(X, Wt, p)
    Nh, Nw = ref.shape[1], ref.shape[2]
    # destination: a padded tensor for a following 3x3 layer, with a recognisable border
    nxt = torch.full((B, Nh + 3, Nw + 2, Kc), -7.0, device=DEV)
    out = snn.snncv(X, Wt, p, next_xpad=nxt, next_offset=(2, 1))
    assert torch.equal(out, ref), "the op's own output changed"
    assert torch.equal(nxt[:, 2:2 + Nh, 1:1 + Nw, :], ref[:B]), "interior of the destination differs from Y[:B]"
    border = nxt.clone()
    border[:, 2:2 + Nh, 1:1 + Nw, :] = -7.0
    assert bool((border == -7.0).all()), "the destination's border was touched"

    dx_full, dw_full, _ = snn.snncv_grad(G, X, Wt, p, ref, want_dparams=False)
    dx_win, dw_win, _ = snn.snncv_grad(G, X, Wt, p, ref, want_dparams=False, crop=(H, W, top, left))
    assert torch.equal(dw_win, dw_full)
    assert torch.equal(dx_win, dx_full[:, top:top + H, left:left + W, :].contiguous())
    # any window inside the padded image, not only the un-padded one
    dx_odd, _, _ = snn.snncv_grad(G, X, Wt, p, ref, want_dparams=False, want_dw=False, crop=(H - 1, W, 0, left))
    assert torch.equal(dx_odd, dx_full[:, 0:H - 1, left:left + W, :].contiguous())


@pytest.mark.parametrize("B,H,W,C,k,s", [(3, 8, 8, 32, 2, 2), (2, 9, 7, 5, 3, 2), (2, 6, 6, 64, 2, 2)])
def test_pooling_with_a_second_destination(B, H, W, C, k, s):
    import snntc_amd as snn
    rng = np.random.default_rng(B * 100 + C)
    x = t(np.exp(rng.random((B, H, W, C))).astype(np.float32))
    pool = snn.SNN_maxpool2d(k, s, 'SAME')
    ref = pool(x)
    nh, nw = ref.shape[1], ref.shape[2]
    from snntc_amd.layers import _same_pad
    pad = (_same_pad(H, k, s)[0], _same_pad(W, k, s)[0])
    nxt = torch.full((B, nh + 2, nw + 2, C), 1e5, device=DEV)
    y, _ = snn.min_pool(x, (k, k), (s, s), pad, (nh, nw), next_xpad=nxt, next_offset=(1, 1))
    assert torch.equal(y, ref)
    assert torch.equal(nxt[:, 1:1 + nh, 1:1 + nw, :], ref)
    nxt[:, 1:1 + nh, 1:1 + nw, :] = 1e5
    assert bool((nxt == 1e5).all())


SMALL_NET = [("conv", 3, 32, 3, 1), ("conv", 32, 32, 3, 1), ("pool", 2, 2), ("conv", 32, 64, 3, 1), ("pool", 2, 2),
             ("conv", 64, 32, 3, 2), ("flatten",), ("dense", 2 * 2 * 32, 10)]


def test_chained_network_matches_the_unchained_one_bit_for_bit():
    """Forward times, loss and every weight gradient of a conv / pool stack, with and without chaining, over
    three training steps in a row (the padded buffers are reused from step to step)."""
    from snntc_amd import networks
    rng = np.random.default_rng(5)
    B = 6
    z = t(np.exp(1.0 - rng.random((B, 16, 16, 3))).astype(np.float32))
    onehot = t(np.eye(10, dtype=np.float32)[rng.integers(0, 10, B)])
    weights = networks.draw_weights(SMALL_NET, rng)
    plain = networks.build(SMALL_NET, weights=[w.copy() for w in weights]).to(DEV)
    chained = networks.build(SMALL_NET, weights=[w.copy() for w in weights], chain=True).to(DEV)
    for step in range(3):
        lp, gp = networks.forward_backward(plain, z, onehot)
        lc, gc = networks.forward_backward(chained, z, onehot)
        assert torch.equal(lp, lc), f"step {step}: loss differs"
        for i, (a, b) in enumerate(zip(gp, gc)):
            assert torch.equal(a, b), f"step {step}: weight gradient of layer {i} differs"
        networks.sgd_update(plain.weights(), gp, 1e-3)
        networks.sgd_update(chained.weights(), gc, 1e-3)
        z = z * 1.01                                       # new inputs next step
    for a, b in zip(plain.weights(), chained.weights()):
        assert torch.equal(a, b)
    # the input gradient arrives un-padded and equal, too
    zin = z.clone().requires_grad_(True)
    zin2 = z.clone().requires_grad_(True)
    plain(zin).sum().backward()
    chained(zin2).sum().backward()
    assert torch.equal(zin.grad, zin2.grad)


def test_backward_after_a_second_forward_of_a_chained_network_is_refused():
    """The padded input buffers of chained layers belong to the latest forward pass.  A backward pass of
    an earlier forward would differentiate against the later pass's inputs; autograd refuses it because
    the kernels' writes advance the buffers' version counters.  Forward, backward, forward, backward (a
    training loop) is unaffected, and the layers keep a bounded number of buffers."""
    from snntc_amd import networks
    rng = np.random.default_rng(7)
    z1 = t(np.exp(1.0 - rng.random((2, 16, 16, 3))).astype(np.float32))
    z2 = t(np.exp(1.0 - rng.random((2, 16, 16, 3))).astype(np.float32))
    net = networks.build(SMALL_NET, weights=networks.draw_weights(SMALL_NET, rng), chain=True).to(DEV)
    y1 = net(z1)
    net(z2)                                                    # overwrites the padded buffers y1's graph saved
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        y1.sum().backward()
    for z in (z1, z2):                                         # the ordinary order still works
        net.zero_grad(set_to_none=True)
        net(z).sum().backward()
        assert all(w.grad is not None and bool(torch.isfinite(w.grad).all()) for w in net.weights())
    conv = [m for m in net if hasattr(m, "release_buffers")][1]
    for B in range(1, 8):                                      # ragged batches: buffers do not pile up
        net(z1[:1].expand(B, -1, -1, -1).contiguous())
    assert len(conv._padded) <= conv.MAX_PADDED_BUFFERS
    conv.release_buffers()
    assert len(conv._padded) == 0
