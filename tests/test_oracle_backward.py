"""Pins the backward half of the CPU oracle without a GPU: analytic derivatives over the
rank-defined causal sets (float64, independent formula), central finite differences of the
float64 closed-form forward, the structurally different host-semantics functors, and the
dense-on-patches identity for the conv layer."""
import numpy as np
import pytest

from helpers import assert_close, conv_case, dense_case
from oracle import capi, closed_form as cf

GOLDEN = np.load(__import__("os").path.join(__import__("os").path.dirname(__file__), "golden", "snntc_golden.npz"))


def _grad_scale(g, x, w, p, out):
    """Sum of absolute summands of every gradient element (conditioning of the sums)."""
    B = x.shape[0]
    absout = out.copy(); absout[B:] = np.abs(absout[B:])
    adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, absout, wide=True)
    return np.abs(adx), np.abs(adw)


@pytest.mark.parametrize("seed,B,I,J,bias,dist", [
    (0, 8, 50, 12, True, "reftest"), (1, 8, 50, 12, False, "reftest"), (2, 16, 120, 30, True, "baseline"),
])
def test_fc_backward_dev_is_the_analytic_derivative_over_causal_sets(seed, B, I, J, bias, dist):
    x, w, p, g = dense_case(seed, B, I, J, bias, dist)
    out, k, _, perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    dx, dw, dp = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    # membership from (perm, k): rank < k.  Independent of the x <= y mask the kernels use; the two
    # coincide unless y ties an input exactly, which these seeds do not produce.
    mask = cf.causal_mask_from_rank(perm, np.where(k >= 0, k, 0))
    y = out[:B].astype(np.float64)
    S = np.where(k >= 0, 1.0 / np.where(out[B:] != 0, out[B:], 1.0).astype(np.float64), 0.0)
    rdx, rdw = cf.analytic_grads(g[:B], x, w, y, S, mask, float(p[5]))
    sx, sw = _grad_scale(g, x, w, p, out)
    assert np.all(np.abs(dx - rdx) <= 1e-5 * np.abs(rdx) + 1e-6 * np.maximum(1, sx))
    assert np.all(np.abs(dw - rdw) <= 1e-5 * np.abs(rdw) + 1e-6 * np.maximum(1, sw))
    assert np.all(dp == 0)


def test_fc_backward_dev_matches_finite_differences():
    x, w, p, g = dense_case(3, 3, 12, 4, True, "baseline")
    out = capi.fc_forward_dev(x, w, p)
    dx, dw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    fx, fw = cf.fd_grads(g[:3], x, w, p, h=1e-5, probes=40, seed=1)
    for (b, i), v in fx:
        assert abs(dx[b, i] - v) <= 2e-3 * max(1.0, abs(v)), ("dx", b, i, dx[b, i], v)
    for (r, c), v in fw:
        assert abs(dw[r, c] - v) <= 2e-3 * max(1.0, abs(v)), ("dw", r, c, dw[r, c], v)


def test_fc_backward_fp32_and_wide_accumulation_agree():
    x, w, p, g = dense_case(4, 64, 300, 100, True, "baseline")
    out = capi.fc_forward_dev(x, w, p)
    a = capi.fc_backward_dev(g, x, w, p, out, wide=False)
    b = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    sx, sw = _grad_scale(g, x, w, p, out)
    assert np.all(np.abs(a[0] - b[0]) <= 1e-5 * np.abs(b[0]) + 1e-6 * np.maximum(1, sx))
    assert np.all(np.abs(a[1] - b[1]) <= 1e-5 * np.abs(b[1]) + 1e-6 * np.maximum(1, sw))


def test_fc_backward_host_agrees_with_dev_without_bias():
    """The reference's CPU functor recomputes S from the strict mask and divides; it has no bias
    support.  Without bias and without exact ties it is the same derivative."""
    x, w, p, g = dense_case(5, 12, 80, 20, False, "baseline")
    B = 12
    out = capi.fc_forward_dev(x, w, p)
    ddx, ddw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    hdx, hdw, hdp = capi.fc_backward_host(g, x, w, p, out)
    sx, sw = _grad_scale(g, x, w, p, out)
    assert np.all(np.abs(hdx - ddx) <= 1e-4 * np.abs(ddx) + 1e-5 * np.maximum(1, sx))
    assert np.all(np.abs(hdw - ddw) <= 1e-4 * np.abs(ddw) + 1e-5 * np.maximum(1, sw))
    assert np.all(hdp[:5] == 0)


def test_fc_backward_dev_mask_includes_equal_times_and_skips_unfired():
    """Documented tie rule of the kernels: an input with x == y counts (x <= y); outputs at MAX get
    no gradient."""
    p = capi.fc_params(0.0)
    x = np.array([[2.0, 3.0]], np.float32)
    w = np.array([[3.0, 0.2], [1.0, 0.3]], np.float32)          # neuron 0: y = 3 == x[1]; neuron 1 never fires
    out = capi.fc_forward_dev(x, w, p)
    assert out[0, 0] == 3.0 and out[0, 1] == np.float32(1e5)
    g = np.zeros((2, 2), np.float32); g[0] = [1.0, 1.0]
    dx, dw, _ = capi.fc_backward_dev(g, x, w, p, out)
    up = 1.0 * out[1, 0]
    assert np.allclose(dx, [[up * 3.0, up * 1.0]])               # the tying input is included
    assert np.allclose(dw[:, 0], [up * (2.0 - 3.0), 0.0]) and np.all(dw[:, 1] == 0)


@pytest.mark.parametrize("seed,B,H,W,C,Kc,Kh,Kw,Sh,Sw,same,bias", [
    (0, 2, 6, 7, 3, 5, 3, 3, 1, 1, True, True), (1, 2, 9, 8, 2, 4, 2, 4, 3, 2, False, True),
    (2, 1, 10, 10, 4, 3, 5, 5, 2, 2, True, False),
])
def test_cv_backward_dev_is_dense_backward_on_patches(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias):
    _, xpad, w, p, g = conv_case(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias, "reftest")
    out = capi.cv_forward_dev(xpad, w, p)
    dx, dw, dp = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
    patches = cf.im2col(xpad, Kh, Kw, Sh, Sw)
    S = patches.shape[0]
    p6 = np.array([p[0], p[3], p[4], 0, 0, p[11]], np.float32)
    pdx, pdw, _ = capi.fc_backward_dev(g.reshape(2 * S, Kc), patches, w, p6, out.reshape(2 * S, Kc), wide=True)
    # fold the patch gradients back onto the image (col2im) in float64
    Nh, Nw = (xpad.shape[1] - Kh) // Sh + 1, (xpad.shape[2] - Kw) // Sw + 1
    fold = np.zeros(xpad.shape, np.float64)
    pd = pdx.reshape(B, Nh, Nw, Kh, Kw, C).astype(np.float64)
    for nh in range(Nh):
        for nw in range(Nw):
            fold[:, nh * Sh:nh * Sh + Kh, nw * Sw:nw * Sw + Kw, :] += pd[:, nh, nw]
    scale = np.abs(fold).max() + 1.0
    assert np.all(np.abs(dx - fold) <= 1e-5 * np.abs(fold) + 1e-6 * scale)
    assert_close(dw, pdw, rtol=1e-5, atol=1e-6 * (np.abs(pdw).max() + 1.0), what="conv dW vs dense-on-patches dW")
    assert np.all(dp == 0)
    if same:                                    # padded pixels never receive gradient
        assert np.all(dx[xpad > 99999.0] == 0)


def test_cv_backward_host_agrees_with_dev():
    _, xpad, w, p, g = conv_case(3, 2, 8, 8, 3, 6, 3, 3, 1, 1, True, True, "baseline")
    out = capi.cv_forward_dev(xpad, w, p)
    ddx, ddw, _ = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
    hdx, hdw, hdp = capi.cv_backward_host(g, xpad, w, p, out)
    assert_close(hdx, ddx, rtol=1e-4, atol=1e-5 * (np.abs(ddx).max() + 1), what="host dX")
    assert_close(hdw, ddw, rtol=1e-4, atol=1e-5 * (np.abs(ddw).max() + 1), what="host dW")
    assert np.all(hdp[:10] == 0)


@pytest.mark.parametrize("name", ["fc_ties", "fc_edge", "fc_rand"])
def test_golden_dense_gradients(name):
    x, w, p, g, out = (GOLDEN[f"{name}_{n}"] for n in ("x", "w", "params", "grad", "out"))
    dx, dw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    assert np.array_equal(dx, GOLDEN[f"{name}_dx"]) and np.array_equal(dw, GOLDEN[f"{name}_dw"])


@pytest.mark.parametrize("name", ["cvtest0", "cvtest1", "cvtest2", "cv_rand"])
def test_golden_conv_gradients(name):
    xpad, w, p, g, out = (GOLDEN[f"{name}_{n}"] for n in ("xpad", "w", "params", "grad", "out"))
    dx, dw, _ = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
    assert np.array_equal(dx, GOLDEN[f"{name}_dx"]) and np.array_equal(dw, GOLDEN[f"{name}_dw"])


def test_loss_closed_form_value_and_gradient():
    """The float64 loss statement used to check the GPU loss kernel: a hand value, the uniform case,
    and its gradient against central differences of its own value."""
    from oracle.closed_form import softmax_time_loss
    # two classes, times (1, 3), label on the early class: p = e^-1/(e^-1+e^-3) -> loss = log(1 + e^-2)
    s, g = softmax_time_loss(np.array([[1.0, 3.0]]), np.array([[1.0, 0.0]]))
    assert abs(s[0] - np.log1p(np.exp(-2.0))) < 1e-14
    p = 1.0 / (1.0 + np.exp(-2.0))
    assert np.allclose(g, [[1.0 - p, -(1.0 - p)]], atol=1e-14)        # earlier true class: push its time down
    s, g = softmax_time_loss(np.full((3, 5), 2.5), np.eye(5)[[0, 2, 4]])
    assert np.allclose(s, np.log(5.0)) and np.allclose(g.sum(axis=1), 0.0)
    rng = np.random.default_rng(3)
    t = 1.0 + 3.0 * rng.random((6, 9)); y = np.eye(9)[rng.integers(0, 9, 6)]
    _, g = softmax_time_loss(t, y)
    h = 1e-6
    for (b, j) in [(0, 0), (2, 5), (5, 8), (3, 3)]:
        tp, tm = t.copy(), t.copy(); tp[b, j] += h; tm[b, j] -= h
        fd = (softmax_time_loss(tp, y)[0].mean() - softmax_time_loss(tm, y)[0].mean()) / (2 * h)
        assert abs(fd - g[b, j]) < 1e-8
