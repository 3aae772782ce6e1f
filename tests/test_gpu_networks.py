"""Whole layer stacks of the benchmark configurations on the GPU against the oracle chain, in the
manner of the reference's multi-layer checks (snntc/test-snn-fc-layers.py, snntc/test-snn-cv-layers.py:
layers stacked, loss on the last one, gradients through all of them).

  * MLP 784-800-800-10 at its full batch of 256: forward bit-exact through all three layers, loss,
    every dX / dW layer by layer, the SGD-updated weights.
  * CIFAR-shaped net at B=2 and ImageNet-shaped net at B=1: the same, layer by layer.
  * Full batches (B=128 / B=32) through size-independent properties: the first samples of the full
    batch equal the oracle chain run on those samples alone (samples are independent in the forward
    pass), the weight gradient of the batch is the sum over sub-batches, the loss is finite.
"""
import numpy as np
import pytest
import torch

import net_oracle as no
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def make_inputs(spec_name, B, seed):
    rng = np.random.default_rng(seed)
    shape, classes = {"mlp": ((784,), 10), "cifar": ((32, 32, 3), 10), "imagenet": ((224, 224, 3), 1000)}[spec_name]
    z = np.exp(1.0 - rng.random((B,) + shape)).astype(np.float32)
    onehot = np.eye(classes, dtype=np.float32)[rng.integers(0, classes, B)]
    return rng, z, onehot


def specs():
    from snntc_amd import networks as N
    return {"mlp": N.MLP, "cifar": N.CIFAR, "imagenet": N.IMAGENET}


@pytest.mark.parametrize("name,B", [("mlp", 256), ("cifar", 2), ("imagenet", 1)])
def test_network_layer_by_layer_against_the_oracle(name, B):
    import snntc_amd as snn
    from snntc_amd import networks as N
    spec = specs()[name]
    rng, z, onehot = make_inputs(name, B, seed=3)
    weights = N.draw_weights(spec, rng)
    net = N.build(spec, weights=[w.copy() for w in weights]).to(DEV)
    acts, outs, sample_loss, dtimes = no.run_gpu_chain(torch, snn, net, t(z), t(onehot))
    # loss and its gradient against the float64 closed form on the GPU's own (bit-exact) spike times
    want_s, want_g = cf.softmax_time_loss(outs[-1].detach().cpu().numpy(), onehot)
    assert np.all(np.abs(sample_loss.cpu().numpy() - want_s) <= 1e-6 * np.maximum(1.0, np.abs(want_s)))
    assert np.all(np.abs(dtimes.cpu().numpy() - want_g) <= 1e-6 / B + 1e-6 * np.abs(want_g))
    report = no.check_layer_by_layer(spec, net, acts, outs)
    assert report, "no gradient was compared"
    print(name, "worst error / band per layer:", [(w, round(r, 3)) for w, r in report])


@pytest.mark.parametrize("name,B", [("mlp", 256), ("cifar", 2)])
def test_training_step_against_the_independent_oracle_chain(name, B):
    """One SGD step (the step bench.py times): spike times bit-exact against an oracle chain that feeds
    itself, weight gradients within the band widened by the number of layers the error passed
    through, updated weights = w - lr * dW."""
    import snntc_amd as snn
    from snntc_amd import networks as N
    spec = specs()[name]
    rng, z, onehot = make_inputs(name, B, seed=5)
    weights = N.draw_weights(spec, rng)
    net = N.build(spec, weights=[w.copy() for w in weights]).to(DEV)
    chain = no.OracleChain(spec, weights)
    ref_times = chain.forward(z)
    ref_loss, ref_dws, ref_adws = chain.loss_and_backward(onehot)

    with torch.no_grad():
        times = net(t(z))
    assert np.array_equal(times.cpu().numpy().view(np.uint32), ref_times.view(np.uint32)), "spike times not bit-exact"
    sample_loss, grads = N.forward_backward(net, t(z), t(onehot))
    assert np.all(np.abs(sample_loss.cpu().numpy() - ref_loss) <= 1e-6 * np.maximum(1.0, np.abs(ref_loss)))
    n_weighted = len(ref_dws)
    for li, (g, rdw, adw) in enumerate(zip(grads, ref_dws, ref_adws)):
        no.assert_in_band(g.cpu().numpy(), rdw, adw, f"{name} weighted layer {li} dW", depth=n_weighted - li)

    lr = 1e-2
    before = [w.detach().clone() for w in net.weights()]
    loss2 = N.sgd_train_step(net, t(z), t(onehot), lr)
    torch.cuda.synchronize()
    assert torch.equal(loss2, sample_loss), "the training step's loss differs from forward_backward's"
    for li, (w0, w1, g, rdw, adw) in enumerate(zip(before, net.weights(), grads, ref_dws, ref_adws)):
        w0n, w1n = w0.cpu().numpy().astype(np.float64), w1.detach().cpu().numpy().astype(np.float64)
        # the update itself: one fp32 rounding of w - lr * dw with the GPU's own gradient
        own = w0n - lr * g.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(w1n - own) <= 1.2e-7 * np.maximum(np.abs(own), np.abs(w0n)) + 1e-30), f"layer {li} update"
        # and against the oracle's gradient
        want = w0n - lr * rdw.astype(np.float64)
        lim = lr * no.grad_band(rdw, adw, depth=n_weighted - li) + 1.2e-7 * np.abs(w0n)
        assert np.all(np.abs(w1n - want) <= lim), f"layer {li}: updated weights outside the band"


@pytest.mark.parametrize("name,B,n_ref,sub", [("cifar", 128, 2, 32), ("imagenet", 32, 1, 8)])
def test_full_batch_network_properties(name, B, n_ref, sub):
    import snntc_amd as snn
    from snntc_amd import networks as N
    spec = specs()[name]
    rng, z, onehot = make_inputs(name, B, seed=7)
    weights = N.draw_weights(spec, rng)
    net = N.build(spec, weights=[w.copy() for w in weights]).to(DEV)
    Z, OH = t(z), t(onehot)
    with torch.no_grad():
        times = net(Z)
    # samples are independent in the forward pass: the first n_ref rows equal the oracle chain on them alone
    ref = no.OracleChain(spec, weights).forward(z[:n_ref])
    assert np.array_equal(times[:n_ref].cpu().numpy().view(np.uint32), ref.view(np.uint32))
    assert float((times < 1e5).float().mean()) > 0.9, "most output neurons should fire on these inputs"
    # ... and any sub-batch run alone reproduces its rows of the full batch bit for bit
    with torch.no_grad():
        assert torch.equal(net(Z[B - sub:]), times[B - sub:])
    sample_loss, grads = N.forward_backward(net, Z, OH)
    assert torch.isfinite(sample_loss).all()
    # dW of the batch = sum over sub-batches (each sub-batch's loss gradient rescaled to the full batch mean)
    acc = [torch.zeros_like(g, dtype=torch.float64) for g in grads]
    mag = [torch.zeros_like(g, dtype=torch.float64) for g in grads]
    for s0 in range(0, B, sub):
        tb = net(Z[s0:s0 + sub])
        _, dt = snn.softmax_time_loss(tb.detach(), OH[s0:s0 + sub])
        gs = torch.autograd.grad(tb, net.weights(), grad_outputs=dt * (sub / B))
        for a, m, g in zip(acc, mag, gs):
            a += g.double(); m += g.double().abs()
    for li, (a, m, g) in enumerate(zip(acc, mag, grads)):
        # the parts are themselves sums with cancellation: scale the absolute term by the largest entry too
        scale = torch.maximum(m, g.double().abs().max() * torch.ones_like(m))
        lim = (len(grads) - li) * (1e-5 * a.abs() + 1e-5 * scale + 1e-9)
        assert torch.all((a - g.double()).abs() <= lim), f"{name} weighted layer {li}: batch dW is not the sum of its parts"
