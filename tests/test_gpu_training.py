"""End-to-end check of the ops under an optimiser: a small SNN classifier built from the layers must
learn a separable synthetic problem (loss falls, accuracy rises), its checkpoint must restore the exact
outputs, and the constraint cost must equal its definition."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class SmallNet(torch.nn.Module):
    """conv 3x3/2 -> conv 3x3/2 -> dense -> dense, the layout of the reference's MNIST example
    (snntc-mnist.py:37-53) at a reduced size."""

    def __init__(self, snn, rng):
        super().__init__()

        def w(fan_in, fan_out):
            # column sums around 4 > threshold 1, so that nearly every neuron fires from the first step (the
            # reference's default init leaves two thirds of such narrow layers silent for hundreds of steps)
            body = 4.0 / fan_in + np.sqrt(1.0 / fan_in) * rng.standard_normal((fan_in, fan_out))
            return np.concatenate((body, np.zeros((1, fan_out)))).astype(np.float32)

        self.layer1 = snn.SNN_conv(kernel_sizes=3, in_channel=1, out_channel=8, strides=2, weight=w(9, 8))
        self.layer2 = snn.SNN_conv(kernel_sizes=3, in_channel=8, out_channel=16, strides=2, weight=w(72, 16))
        self.layer3 = snn.SNN_dense(in_size=3 * 3 * 16, out_size=64, weight=w(144, 64))
        self.layer4 = snn.SNN_dense(in_size=64, out_size=4, weight=w(64, 4))

    def forward(self, x):
        h = self.layer2(self.layer1(x))
        return self.layer4(self.layer3(h.reshape(h.shape[0], -1)))


def make_data(n, rng):
    """Four classes: a bright quadrant of a 12x12 image."""
    labels = rng.integers(0, 4, n)
    img = 0.1 * rng.random((n, 12, 12, 1))
    for i, c in enumerate(labels):
        r, q = divmod(int(c), 2)
        img[i, 6 * r:6 * r + 6, 6 * q:6 * q + 6, 0] += 0.8
    return torch.from_numpy(img.astype(np.float32)).to(DEV), torch.from_numpy(labels).to(DEV)


def test_small_network_learns_and_checkpoints():
    import snntc_amd as snn
    from snntc_amd import train
    np.random.seed(0); torch.manual_seed(0)
    rng = np.random.default_rng(0)
    model = SmallNet(snn, rng).to(DEV)
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    images, labels = make_data(256, rng)
    first = last = None
    for it in range(60):
        loss, correct = train.train_step(model, opt, images, labels, 4, weight_k=100.0, weight_k2=1e-2)
        assert torch.isfinite(loss)
        if it == 0:
            first = (float(loss), int(correct))
        last = (float(loss), int(correct))
    assert last[0] < 0.6 * first[0], (first, last)
    test_images, test_labels = make_data(128, rng)
    tl, tc = train.test_step(model, test_images, test_labels, 4, weight_k=100.0, weight_k2=1e-2)
    assert int(tc) >= 0.9 * 128, (first, last, int(tc))

    # constraint cost against its definition (snntc-mnist.py:55-59)
    ws = [p.detach().double().cpu().numpy() for p in model.parameters()]
    want = 100.0 * sum(np.mean(np.maximum(0.0, 1.0 - w.sum(0))) for w in ws) + 1e-2 * sum(np.mean(w * w) for w in ws)
    got = float(train.constraint_cost(model, 100.0, 1e-2).detach())
    assert abs(got - want) <= 1e-5 * max(1.0, abs(want))

    # checkpoint round trip: a fresh model loaded from the state dict reproduces the outputs exactly
    state = {k: v.clone() for k, v in model.state_dict().items()}
    clone = SmallNet(snn, rng).to(DEV)
    clone.load_state_dict(state)
    with torch.no_grad():
        assert torch.equal(model(train.encode_input(test_images)), clone(train.encode_input(test_images)))
