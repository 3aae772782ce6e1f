"""The HIP ops on the committed golden vectors (tests/golden/snntc_golden.npz): the reference's own
deterministic conv fixtures (snntc/test-snn-cv-backward.py:58-79, testmode 0/1/2) and the hand-built
tie / edge / random cases.  Forward results -- sorted values, permutation, causal-set sizes, spike
times and reciprocals -- must equal the stored vectors bit for bit; gradients within
rel 1e-5 / abs 1e-6 of the stored float64-accumulated values (the literal north-star bar: these sums
are short enough that no scaling of the absolute term is needed)."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "snntc_golden.npz"))

DENSE = ["fc_ties", "fc_edge", "fc_rand"]
CONV = ["cvtest0", "cvtest1", "cvtest2", "cv_rand"]


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _check_forward(name, out, sz, perm, ck):
    torch.cuda.synchronize()
    out, sz, perm, ck = (v.cpu().numpy() for v in (out, sz, perm, ck))
    assert np.array_equal(sz, GOLDEN[f"{name}_sorted"]), "sorted values differ"
    assert np.array_equal(perm, GOLDEN[f"{name}_perm"]), "permutation differs"
    assert np.array_equal(ck, GOLDEN[f"{name}_k"]), "causal-set sizes differ"
    assert np.array_equal(out.view(np.uint32), GOLDEN[f"{name}_out"].view(np.uint32)), "y / 1/S not bit-exact"


@pytest.mark.parametrize("name", DENSE)
def test_golden_dense_vectors_on_the_gpu(name):
    import snntc_amd as snn
    x, w, p, g = (GOLDEN[f"{name}_{k}"] for k in ("x", "w", "params", "grad"))
    out, sz, perm, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    _check_forward(name, out, sz, perm, ck)
    assert torch.equal(snn.snnfc(t(x), t(w), p), out)
    dx, dw, dp = snn.snnfc_grad(t(g), t(x), t(w), p, t(GOLDEN[f"{name}_out"]))
    torch.cuda.synchronize()
    assert_close(dx.cpu().numpy(), GOLDEN[f"{name}_dx"], what=f"{name} dX")
    assert_close(dw.cpu().numpy(), GOLDEN[f"{name}_dw"], what=f"{name} dW")
    assert torch.all(dp == 0)


@pytest.mark.parametrize("name", CONV)
def test_golden_conv_vectors_on_the_gpu(name):
    import snntc_amd as snn
    xpad, w, p, g = (GOLDEN[f"{name}_{k}"] for k in ("xpad", "w", "params", "grad"))
    out, sz, perm, ck = snn.snncv(t(xpad), t(w), p, return_aux=True)
    _check_forward(name, out, sz, perm, ck)
    assert torch.equal(snn.snncv(t(xpad), t(w), p), out)
    dx, dw, dp = snn.snncv_grad(t(g), t(xpad), t(w), p, t(GOLDEN[f"{name}_out"]))
    torch.cuda.synchronize()
    assert_close(dx.cpu().numpy(), GOLDEN[f"{name}_dx"], what=f"{name} dXpad")
    assert_close(dw.cpu().numpy(), GOLDEN[f"{name}_dw"], what=f"{name} dW")
    assert torch.all(dp == 0)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_reference_conv_fixture_through_the_layer(mode):
    """The same fixtures through SNN_conv and autograd, the way snntc/test-snn-cv-backward.py:81-110
    drives them: unpadded input, SAME padding done by the layer, gradient of sum(y)."""
    import snntc_amd as snn
    name = f"cvtest{mode}"
    xpad, w, p = GOLDEN[f"{name}_xpad"], GOLDEN[f"{name}_w"], GOLDEN[f"{name}_params"]
    B = xpad.shape[0]
    x = (np.arange(B * 4 * 4 * 2) + 1.1).astype(np.float32).reshape(B, 4, 4, 2)      # :58-79 of that script
    assert np.array_equal(xpad[:, :4, :4, :], x), "SAME padding of a 4x4 image, 3x3 stride 2: one row/column after"
    layer = snn.SNN_conv(2, w.shape[1], 3, 2, 'SAME', weight=w.copy()).to(DEV)
    X = t(x).requires_grad_(True)
    y = layer(X)
    y.sum().backward()
    torch.cuda.synchronize()
    assert np.array_equal(y.detach().cpu().numpy().view(np.uint32), GOLDEN[f"{name}_out"][:B].view(np.uint32))
    assert_close(X.grad.cpu().numpy(), GOLDEN[f"{name}_dx"][:, :4, :4, :], what="layer dX")
    assert_close(layer.weight.grad.cpu().numpy(), GOLDEN[f"{name}_dw"], what="layer dW")
