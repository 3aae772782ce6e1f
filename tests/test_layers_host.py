"""Host-side mirror of the reference's Python layers (no GPU): constructor contracts, Params layouts,
padding / cropping arithmetic, the stock-op layers, and the refusal to run the ops off-GPU."""
import numpy as np
import pytest
import torch

import snntc_amd as snn
from oracle import closed_form as cf


def test_dense_layer_contract():
    l = snn.SNN_dense(in_size=7, out_size=3)
    assert l.weight.shape == (8, 3) and l.in_size == 8 and l.out_size == 3          # bias row included
    assert torch.all(l.weight[7] == 0)                                              # init_weight: zero bias row
    assert l.Params.dtype == np.float32
    assert l.Params.tolist() == [np.float32(1e5), np.float32(1e-10), 1.0, 0.0, 0.0, 1.0]   # SNN_TC_Modules.py:48-49
    l0 = snn.SNN_dense(7, 3, biasvolt=0.0, MAX_SPIKE_TIME=50.0, Spike_Threshold=2.0, Thread_per_Block=64, Blocks=9)
    assert l0.weight.shape == (7, 3)
    assert l0.Params.tolist() == [50.0, np.float32(1e-10), 2.0, 64.0, 9.0, 0.0]
    w = np.arange(24, dtype=np.float64).reshape(8, 3)
    lw = snn.SNN_dense(7, 3, weight=w)
    assert lw.weight.dtype == torch.float32 and np.array_equal(lw.weight.detach().numpy(), w.astype(np.float32))
    with pytest.raises(ValueError):
        snn.SNN_dense(7, 3, weight=np.zeros((7, 3)))                                # bias row missing
    assert lw.name == 'fckernel'


def test_conv_layer_contract():
    c = snn.SNN_conv(in_channel=4, out_channel=6, kernel_sizes=(3, 2), strides=(2, 1), padding='same')
    assert c.weight.shape == (3 * 2 * 4 + 1, 6)
    # {MAX, tpb, blocks, eps, theta, cudaflag, Kh, Kw, Sh, Sw, SAME, biasvolt}  (SNN_TC_Modules.py:121-123)
    assert c.Params.tolist() == [np.float32(1e5), 0, 0, np.float32(1e-10), 1, 0, 3, 2, 2, 1, 1, 1]
    v = snn.SNN_conv(4, 6, 3, 1, padding='VALID', biasvolt=0.0)
    assert v.weight.shape == (36, 6) and v.Params[10] == 0 and v.Params[11] == 0
    assert v.name == 'convkernel' and v.rates == [1, 1]


SAME_CASES = [(32, 32, 3, 1), (224, 224, 7, 2), (9, 7, 5, 3), (8, 8, 2, 2), (5, 6, 4, 1)]


@pytest.mark.parametrize("H,W,K,S", SAME_CASES)
def test_conv_same_padding_rule(H, W, K, S):
    """The split of the SAME padding (SNN_TC_Modules.py:147-158) against the closed form the reference's
    tests recompute (test-snn-cv-forward.py:70-75), and the op's output size on the padded image."""
    c = snn.SNN_conv(2, 3, K, S, 'SAME')
    (t, b), (l, r) = cf.same_pad(H, K, S), cf.same_pad(W, K, S)
    assert c.same_pads(H, W) == (t, b, l, r)
    assert (H + t + b - K) // S + 1 == -(-H // S) and c.output_hw(H, W) == (-(-H // S), -(-W // S))


@pytest.mark.gpu
@pytest.mark.parametrize("H,W,K,S", SAME_CASES)
def test_conv_same_padding_uses_max_spike_time(H, W, K, S):
    c = snn.SNN_conv(2, 3, K, S, 'SAME')
    x = torch.rand(2, H, W, 2, device="cuda:0") + 1
    xp = c.prepare_input(x)
    (t, b), (l, r) = cf.same_pad(H, K, S), cf.same_pad(W, K, S)
    assert xp.shape == (2, H + t + b, W + l + r, 2)
    assert torch.equal(xp[:, t:t + H, l:l + W, :], x)
    border = torch.ones_like(xp, dtype=torch.bool); border[:, t:t + H, l:l + W, :] = False
    assert torch.all(xp[border] == 1e5)
    assert (xp.shape[1] - K) // S + 1 == -(-H // S)                    # op output = ceil(H/S)


@pytest.mark.parametrize("H,W,K,S", [(32, 32, 3, 1), (10, 11, 3, 2), (9, 7, 5, 3)])
def test_conv_valid_crops_to_whole_windows(H, W, K, S):
    c = snn.SNN_conv(2, 3, K, S, 'VALID')
    x = torch.rand(1, H, W, 2)
    xp = c.prepare_input(x)
    nh, nw = (H - K) // S + 1, (W - K) // S + 1
    assert xp.shape == (1, (nh - 1) * S + K, (nw - 1) * S + K, 2)       # SNN_TC_Modules.py:163-166
    assert torch.equal(xp, x[:, :xp.shape[1], :xp.shape[2], :])


def test_costs():
    w = np.array([[0.2, 0.9], [0.3, 0.4], [0.0, 0.0]], np.float32)
    l = snn.SNN_dense(2, 2, weight=w)
    assert abs(float(l.w_sum_cost().detach()) - 0.25) < 1e-7                     # mean(max(0, 1 - colsum)) = (0.5 + 0)/2
    assert abs(float(l.l2_cost().detach()) - float(np.mean(w ** 2))) < 1e-7


def _cost_gradient_check(dev):
    """Gradients of the weight-constraint costs against their closed forms (SNN_TC_Modules.py:77-84,
    snntc-mnist.py:55-59): d/dw_ij mean_j max(0, theta - sum_i w_ij) = -1/J on columns whose sum lies
    below the threshold and 0 elsewhere; d/dw mean(w^2) = 2 w / n; the constraint cost is
    K * sum_l (first) + K2 * sum_l (second) over the layers of a model."""
    from snntc_amd import train
    rng = np.random.default_rng(11)
    dense = snn.SNN_dense(40, 12, Spike_Threshold=1.5, weight=(rng.standard_normal((41, 12)) * 0.2 + 0.03).astype(np.float32))
    conv = snn.SNN_conv(3, 7, 3, 1, 'SAME', weight=(rng.standard_normal((28, 7)) * 0.2 + 0.04).astype(np.float32))
    model = torch.nn.Sequential(conv, dense).to(dev)
    for layer, theta in ((dense, 1.5), (conv, 1.0)):
        w = layer.weight.detach().cpu().numpy().astype(np.float64)
        below = w.sum(0) < theta
        assert below.any() and (~below).any(), "the draw should hold columns on both sides of the threshold"
        (gw,) = torch.autograd.grad(layer.w_sum_cost(), layer.weight)
        want = np.where(below, -1.0 / w.shape[1], 0.0)[None, :].repeat(w.shape[0], 0)
        assert np.allclose(gw.cpu().numpy(), want, rtol=0, atol=1e-7)
        (gl,) = torch.autograd.grad(layer.l2_cost(), layer.weight)
        assert np.allclose(gl.cpu().numpy(), 2.0 * w / w.size, rtol=1e-6, atol=1e-9)
    K, K2 = 100.0, 1e-2
    grads = torch.autograd.grad(train.constraint_cost(model, K, K2), [conv.weight, dense.weight])
    for layer, g in zip((conv, dense), grads):
        w = layer.weight.detach().cpu().numpy().astype(np.float64)
        below = w.sum(0) < 1.0                                  # constraint_cost uses 1.0 (snntc-mnist.py:57)
        want = K * np.where(below, -1.0 / w.shape[1], 0.0)[None, :] + K2 * 2.0 * w / w.size
        assert np.allclose(g.cpu().numpy(), want, rtol=1e-5, atol=1e-7)


def test_cost_gradients_against_closed_forms():
    _cost_gradient_check("cpu")


@pytest.mark.gpu
def test_cost_gradients_against_closed_forms_on_the_gpu():
    _cost_gradient_check("cuda:0")


def test_avg_pool_is_the_stock_op():
    x = torch.rand(2, 5, 7, 3) + 1
    ap = snn.SNN_avgpool2d(2, 2, 'VALID')
    ya = ap(x)
    assert ya.shape == (2, 2, 3, 3)
    assert np.allclose(ya.numpy(), x.numpy()[:, :4, :6].reshape(2, 2, 2, 3, 2, 3).mean(axis=(2, 4)), atol=1e-6)


def test_lrn_matches_its_formula():
    x = torch.rand(1, 2, 2, 6) + 1
    y = snn.SNN_LRN(depth_radius=5, bias=2, alpha=1e-4, beta=0.75)(x).numpy()
    sq = np.pad(x.numpy() ** 2, ((0, 0), (0, 0), (0, 0), (2, 2)), constant_values=1e5)
    scale = 2 + 1e-4 * sum(sq[..., i:i + 6] for i in range(5))
    assert np.allclose(y, x.numpy() / scale ** 0.75, rtol=1e-6)


@pytest.mark.gpu
def test_loss_is_cross_entropy_on_negated_times():
    logit = torch.tensor([[1.0, 2.0, 4.0], [3.0, 1.5, 1.2]], device="cuda:0")
    label = torch.tensor([[1.0, 0, 0], [0, 0, 1.0]], device="cuda:0")
    want = np.mean([-np.log(np.exp(-1) / np.exp([-1, -2, -4]).sum()), -np.log(np.exp(-1.2) / np.exp([-3, -1.5, -1.2]).sum())])
    assert abs(float(snn.loss_func(logit, label)) - want) < 1e-6


def test_glue_layers_refuse_cpu_tensors():
    """Pooling, SAME padding and the loss run device kernels, like the four ops: no host path."""
    x = torch.rand(2, 6, 6, 4) + 1
    for layer in (snn.SNN_maxpool2d(2, 2, 'SAME'), snn.SNN_globalminpool2d(), snn.SNN_conv(4, 3, 3, 1, 'SAME'),
                  snn.SNN_conv(4, 3, 3, 1, 'VALID')):
        with pytest.raises(snn.SnntcLibraryError, match="no CPU fallback"):
            layer(x)
    with pytest.raises(snn.SnntcLibraryError, match="no CPU fallback"):
        snn.SNN_conv(4, 3, 3, 1, 'SAME').prepare_input(x)
    with pytest.raises(snn.SnntcLibraryError, match="no CPU fallback"):
        snn.loss_func(torch.rand(3, 5), torch.eye(5)[:3])


def test_ops_refuse_cpu_tensors():
    l = snn.SNN_dense(4, 2)
    with pytest.raises(snn.SnntcLibraryError, match="no CPU fallback"):
        l(torch.rand(3, 4) + 1)
    with pytest.raises(snn.SnntcLibraryError):
        snn.snncv(torch.rand(1, 4, 4, 1), torch.rand(10, 2), snn.SNN_conv(1, 2, 3, 1).Params)


def test_init_weight_statistics():
    np.random.seed(0)
    w = snn.init_weight(400, 300, bias_volt=1.0, init_param=15.0)
    assert w.shape == (401, 300) and w.dtype == np.float32 and np.all(w[400] == 0)
    assert abs(w[:400].std() - np.sqrt(15.0 / 400)) < 0.005
    assert snn.init_weight(5, 2, bias_volt=0.0).shape == (5, 2)
