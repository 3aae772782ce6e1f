"""Seeded input generators and comparison helpers shared by the tests."""
import numpy as np

from oracle import capi


def dense_case(seed, B, I, J, bias=True, dist="baseline", sigma2=True):
    """Inputs of one dense layer.

    dist="baseline": z = exp(1 - U[0,1)), w ~ N(4/I, 1/I) (variance 1/I when sigma2 else std 1/I),
                     bias row drawn from the same law.
    dist="reftest" : the reference scripts' law, x = exp(|randn|), w = randn
                     (snntc/test-snn-fc-forward.py:30-32).
    """
    rng = np.random.default_rng(seed)
    rows = I + (1 if bias else 0)
    if dist == "baseline":
        x = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
        std = np.sqrt(1.0 / I) if sigma2 else 1.0 / I
        w = (4.0 / I + std * rng.standard_normal((rows, J))).astype(np.float32)
    elif dist == "reftest":
        x = np.exp(np.abs(rng.standard_normal((B, I)))).astype(np.float32)
        w = rng.standard_normal((rows, J)).astype(np.float32)
    else:
        raise ValueError(dist)
    g = np.zeros((2 * B, J), np.float32)
    g[:B] = rng.standard_normal((B, J)).astype(np.float32)
    return x, w, capi.fc_params(1.0 if bias else 0.0), g


def conv_case(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same=True, bias=True, dist="baseline"):
    """Inputs of one conv layer; returns the padded/cropped input the op sees."""
    from oracle.closed_form import same_pad
    rng = np.random.default_rng(seed)
    P = Kh * Kw * C
    rows = P + (1 if bias else 0)
    if dist == "baseline":
        x = np.exp(rng.random((B, H, W, C))).astype(np.float32)
        w = (4.0 / P + np.sqrt(1.0 / P) * rng.standard_normal((rows, Kc))).astype(np.float32)
    else:
        x = np.exp(np.abs(rng.standard_normal((B, H, W, C)))).astype(np.float32)
        w = rng.standard_normal((rows, Kc)).astype(np.float32)
    if same:
        (t, b), (l, r) = same_pad(H, Kh, Sh), same_pad(W, Kw, Sw)
        xpad = np.pad(x, ((0, 0), (t, b), (l, r), (0, 0)), constant_values=np.float32(1e5))
    else:
        nh, nw = (H - Kh) // Sh + 1, (W - Kw) // Sw + 1
        xpad = x[:, :(nh - 1) * Sh + Kh, :(nw - 1) * Sw + Kw, :]
    xpad = np.ascontiguousarray(xpad, np.float32)
    params = capi.cv_params(Kh, Kw, Sh, Sw, same=same, biasvolt=1.0 if bias else 0.0)
    Nh, Nw, _ = capi.cv_dims(xpad.shape, params)
    g = np.zeros((2 * B, Nh, Nw, Kc), np.float32)
    g[:B] = rng.standard_normal((B, Nh, Nw, Kc)).astype(np.float32)
    return x, xpad, w, params, g


def assert_close(actual, expected, rtol=1e-5, atol=1e-6, what=""):
    """|a - e| <= atol + rtol*|e| elementwise, reporting the worst element."""
    a = np.asarray(actual, np.float64)
    e = np.asarray(expected, np.float64)
    assert a.shape == e.shape, f"{what}: shape {a.shape} vs {e.shape}"
    err = np.abs(a - e)
    lim = atol + rtol * np.abs(e)
    bad = err > lim
    if bad.any():
        idx = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} elements out of tolerance; worst at {idx}: "
                             f"got {a[idx]!r}, want {e[idx]!r}, |diff| {err[idx]:.3e} > {lim[idx]:.3e}")


def grad_band(ref, ref_abs, depth=1):
    """Tolerance of a gradient entry that is an fp32 sum: rel 1e-5 / abs 1e-6 of the value, plus
    5e-7 (about 8 ulp) of the sum of the magnitudes of its summands, `ref_abs` -- two fp32 summation
    orders of the same terms differ by a multiple of that, whatever the size of the sum itself.
    `depth` widens the band for errors carried through that many layers."""
    return depth * (1e-5 * np.abs(ref) + 1e-6 * np.maximum(1.0, 0.5 * np.abs(ref_abs)))
