"""The layer stacks of the benchmark configurations, built from the SNN layers, and the plain-SGD
training step they are timed and tested with.

A network is described by a list of tuples

    ("conv", C_in, C_out, kernel, stride)     SNN_conv, SAME padding, bias input
    ("pool", kernel, stride)                  SNN_maxpool2d (earliest spike), SAME
    ("gmin",)                                 SNN_globalminpool2d
    ("flatten",)                              SNN_flatten
    ("dense", n_in, n_out)                    SNN_dense, bias input

in the style of the reference's example models (snntc-mnist.py:36-53, snntc-cifar10.py:73-106,
snntc-imagenet-example/snntc-imagenet.py:21-58), which stack these layer types.
"""
import numpy as np
import torch

from . import layers as L
from .ops import sgd_update, softmax_time_loss

#: 3-layer MLP 784-800-800-10
MLP = [("dense", 784, 800), ("dense", 800, 800), ("dense", 800, 10)]

#: CIFAR-shaped net on 32x32x3 inputs
CIFAR = [("conv", 3, 32, 3, 1), ("conv", 32, 32, 3, 1), ("pool", 2, 2),
         ("conv", 32, 64, 3, 1), ("conv", 64, 64, 3, 1), ("pool", 2, 2),
         ("conv", 64, 128, 3, 1), ("pool", 2, 2),
         ("flatten",), ("dense", 2048, 512), ("dense", 512, 10)]

#: ImageNet-shaped net on 224x224x3 inputs: 7x7/2 stem, four stages of two 3x3 convs, global pool, classifier
IMAGENET = [("conv", 3, 64, 7, 2), ("pool", 2, 2),
            ("conv", 64, 64, 3, 1), ("conv", 64, 64, 3, 1), ("pool", 2, 2),
            ("conv", 64, 128, 3, 1), ("conv", 128, 128, 3, 1), ("pool", 2, 2),
            ("conv", 128, 256, 3, 1), ("conv", 256, 256, 3, 1), ("pool", 2, 2),
            ("conv", 256, 512, 3, 1), ("conv", 512, 512, 3, 1),
            ("gmin",), ("dense", 512, 1000)]


def baseline_weight(rng, fan_in, fan_out, bias=True):
    """w ~ N(4/fan_in, variance 1/fan_in), the bias row drawn from the same law: column sums of about 4
    against the threshold 1, so that practically every neuron fires.  (The reference's own initialiser,
    init_weight, is randn * sqrt(15/fan_in) with a zero bias row, SNN_TC_Modules.py:19-25; under it many
    neurons of a wide layer stay silent, causal sets are shorter and a step is cheaper.)"""
    rows = fan_in + (1 if bias else 0)
    return (4.0 / fan_in + np.sqrt(1.0 / fan_in) * rng.standard_normal((rows, fan_out))).astype(np.float32)


def layer_weight_shapes(spec):
    """[(fan_in, fan_out)] of the weighted layers of `spec`, in order."""
    out = []
    for item in spec:
        if item[0] == "conv":
            _, ci, co, k, _s = item
            out.append((k * k * ci, co))
        elif item[0] == "dense":
            out.append((item[1], item[2]))
    return out


def draw_weights(spec, rng):
    """One baseline_weight draw per weighted layer of `spec` (with bias rows)."""
    return [baseline_weight(rng, fi, fo) for fi, fo in layer_weight_shapes(spec)]


class SnnSequential(torch.nn.Sequential):
    """The layers of a spec in order.  forward(x, keep=list) appends every layer's input to `keep`.

    chain=True removes the padding pass between a conv or pooling layer and the SAME-padded conv layer
    that follows it: the first writes its spike times into the second's padded input buffer as well (a
    buffer the second layer keeps, its border filled once), and the second reads from there.  Results
    are the same bit for bit.  The buffers hold the latest forward pass only: run backward before the
    next forward, as a training loop does."""

    def __init__(self, *mods, chain=False):
        super().__init__(*mods)
        self.chain = chain

    def forward(self, x, keep=None):
        layers = list(self)
        prefilled = False
        for i, layer in enumerate(layers):
            if keep is not None:
                keep.append(x)
            nxt = layers[i + 1] if i + 1 < len(layers) else None
            feed = None
            if (self.chain and x.is_cuda and isinstance(nxt, L.SNN_conv) and nxt.padding == 'SAME'
                    and isinstance(layer, (L.SNN_conv, L.SNN_maxpool2d))
                    and not (isinstance(layer, L.SNN_conv) and layer.padding != 'SAME')):
                feed = nxt
            if isinstance(layer, L.SNN_conv) and (prefilled or feed is not None):
                x = layer(x, prefilled=prefilled, feed=feed)
            elif isinstance(layer, L.SNN_maxpool2d) and feed is not None:
                x = layer(x, feed=feed)
            else:
                x = layer(x)
            prefilled = feed is not None
        return x

    def weights(self):
        return [l.weight for l in self if hasattr(l, "weight")]


def build(spec, weights=None, rng=None, chain=False):
    """SnnSequential for `spec`.  `weights`: one numpy array per weighted layer; drawn from
    baseline_weight with `rng` when omitted.  chain: see SnnSequential."""
    if weights is None:
        weights = draw_weights(spec, rng if rng is not None else np.random.default_rng(0))
    weights = list(weights)
    mods = []
    for item in spec:
        kind = item[0]
        if kind == "conv":
            _, ci, co, k, s = item
            mods.append(L.SNN_conv(ci, co, k, s, 'SAME', weight=weights.pop(0)))
        elif kind == "dense":
            mods.append(L.SNN_dense(item[1], item[2], weight=weights.pop(0)))
        elif kind == "pool":
            mods.append(L.SNN_maxpool2d(item[1], item[2], 'SAME'))
        elif kind == "gmin":
            mods.append(L.SNN_globalminpool2d())
        elif kind == "flatten":
            mods.append(L.SNN_flatten())
        else:
            raise ValueError(f"unknown layer kind {kind!r}")
    if weights:
        raise ValueError("more weight arrays than weighted layers")
    return SnnSequential(*mods, chain=chain)


def forward_backward(net, z, onehot):
    """Forward, softmax-on-negative-time loss and backward of `net` on spike times z.  Returns
    (per-sample loss[B], weight gradients in layer order).  Backpropagation starts from the loss kernel's
    gradient of the batch mean, so no scalar loss node is needed."""
    times = net(z)
    sample_loss, dtimes = softmax_time_loss(times.detach(), onehot)
    grads = torch.autograd.grad(times, net.weights(), grad_outputs=dtimes)
    return sample_loss, grads


def sgd_train_step(net, z, onehot, lr):
    """One plain-SGD training step (forward, loss, backward, w -= lr * dw for all layers in one launch).
    Returns the per-sample loss."""
    sample_loss, grads = forward_backward(net, z, onehot)
    sgd_update(net.weights(), grads, lr)
    return sample_loss
