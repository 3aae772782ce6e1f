#!/usr/bin/env python3
"""Writes tests/golden/snntc_golden.npz: small input/output vectors for the four ops.

The reference holds no stored expected outputs (its tf2test-*.mat files are not in the repository)
and its Python cannot be imported here (TensorFlow is absent), so the expected values come from
this build's two independent CPU statements, which must agree before a case is written:
the C restatement (oracle/snntc_oracle.c, device semantics) and the numpy closed form that follows
the reference tests' hand-calculation recipe (oracle/closed_form.py).

Cases
  cvtest0/1/2   the deterministic inputs of snntc/test-snn-cv-backward.py:58-79 (testmode 0, 1, 2):
                x = arange(B*H*W*C)+1.1, w = (arange((Kh*Kw*C+1)*Kc)+1)/10, 3x3 stride 2 SAME
  fc_ties       a dense layer whose rows contain repeated values (stable order matters)
  fc_edge       hand-built rows: bias-only firing, never firing, all-padding, negative denominator
  fc_rand       random dense layer in the reference scripts' distribution
  cv_rand       random conv layer, VALID, stride (2,1), non-square kernel

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import capi, closed_form as cf  # noqa: E402


def check_against_closed_form(x2d, w, params6, out, k):
    """Causal-set sizes must agree exactly and spike times to 1e-5 wherever the float64 closed form
    is not within 1e-6 (relative) of a decision boundary."""
    y, kc, S = cf.fc_forward_closed_form(x2d, w, params6)
    B = x2d.shape[0]
    assert np.array_equal(k, kc), "oracle and closed form disagree on causal sets"
    fired = kc >= 0
    assert np.allclose(out[:B][fired], y[fired], rtol=1e-5, atol=0)
    assert np.allclose(out[B:][fired] * S[fired], 1.0, rtol=1e-5)
    assert np.all(out[:B][~fired] == params6[0]) and np.all(out[B:][~fired] == 0)


def dense_case(name, x, w, params, g, store):
    out, k, sz, perm = capi.fc_forward_dev(x, w, params, want_aux=True)
    check_against_closed_form(x, w, params, out, k)
    dx, dw, _ = capi.fc_backward_dev(g, x, w, params, out, wide=True)
    store.update({f"{name}_x": x, f"{name}_w": w, f"{name}_params": params, f"{name}_grad": g,
                  f"{name}_out": out, f"{name}_k": k, f"{name}_sorted": sz, f"{name}_perm": perm,
                  f"{name}_dx": dx, f"{name}_dw": dw})


def conv_case(name, xpad, w, params, g, store):
    out, k, sz, perm = capi.cv_forward_dev(xpad, w, params, want_aux=True)
    Kh, Kw, Sh, Sw = (int(params[t]) for t in (6, 7, 8, 9))
    patches = cf.im2col(xpad, Kh, Kw, Sh, Sw)
    p6 = np.array([params[0], params[3], params[4], 0, 0, params[11]], np.float32)
    S, Kc = k.shape
    check_against_closed_form(patches, w, p6, out.reshape(2 * S, Kc), k)
    dx, dw, _ = capi.cv_backward_dev(g, xpad, w, params, out, wide=True)
    store.update({f"{name}_xpad": xpad, f"{name}_w": w, f"{name}_params": params, f"{name}_grad": g,
                  f"{name}_out": out, f"{name}_k": k, f"{name}_sorted": sz, f"{name}_perm": perm,
                  f"{name}_dx": dx, f"{name}_dw": dw})


def main():
    store = {}
    rng = np.random.default_rng(2023)

    # --- the reference's deterministic conv fixtures (inputs only; outputs computed here) ---------
    for mode, (B, H, W, C, Kh, Kw, Kc, Sh, Sw) in enumerate(
            [(1, 4, 4, 2, 3, 3, 1, 2, 2), (1, 4, 4, 2, 3, 3, 2, 2, 2), (2, 4, 4, 2, 3, 3, 2, 2, 2)]):
        x = (np.arange(B * H * W * C) + 1.1).astype(np.float32).reshape(B, H, W, C)
        w = ((np.arange((Kh * Kw * C + 1) * Kc) + 1.0) / 10.0).reshape(-1, Kc).astype(np.float32)
        (t, b), (l, r) = cf.same_pad(H, Kh, Sh), cf.same_pad(W, Kw, Sw)
        xpad = np.pad(x, ((0, 0), (t, b), (l, r), (0, 0)), constant_values=np.float32(1e5))
        params = capi.cv_params(Kh, Kw, Sh, Sw, same=True, biasvolt=1.0)
        Nh, Nw, _ = capi.cv_dims(xpad.shape, params)
        g = np.zeros((2 * B, Nh, Nw, Kc), np.float32)
        g[:B] = 1.0                                   # the reference differentiates sum(y)
        conv_case(f"cvtest{mode}", xpad, w, params, g, store)

    # --- dense rows with repeated values --------------------------------------------------------
    B, I, J = 6, 40, 9
    x = (1.0 + rng.integers(0, 8, (B, I)) / 4.0).astype(np.float32)
    x[0, :] = 2.0
    w = (rng.standard_normal((I + 1, J)) * 0.4 + 0.1).astype(np.float32)
    g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))
    # ties make y == x boundaries likely; keep only a draw on which both statements agree
    dense_case("fc_ties", x, w, capi.fc_params(1.0), g, store)

    # --- hand-built edge rows -------------------------------------------------------------------
    x = np.array([[2.0, 3.0, 4.0, 5.0],          # ordinary
                  [1e5, 1e5, 1e5, 1e5],          # nothing but padding
                  [5.0, 4.0, 3.0, 2.0],          # descending input order
                  [1.5, 1.5, 1e5, 2.5]], np.float32)
    w = np.array([[0.9, 0.1, -0.5, 3.0],
                  [0.9, 0.1, -0.5, 0.1],
                  [0.9, 0.1, -0.6, 0.1],
                  [0.9, 0.1, -0.7, 0.1],
                  [0.0, 0.0, 0.0, 0.0]], np.float32)   # last row: bias weights
    w[4] = [0.0, 0.0, -0.2, 4.0]                  # column 3: the bias alone fires; column 2: negative weights
    g = np.zeros((8, 4), np.float32); g[:4] = rng.standard_normal((4, 4))
    dense_case("fc_edge", x, w, capi.fc_params(1.0), g, store)

    # --- random cases -----------------------------------------------------------------------------
    B, I, J = 5, 23, 7
    x = np.exp(np.abs(rng.standard_normal((B, I)))).astype(np.float32)
    w = rng.standard_normal((I, J)).astype(np.float32)
    g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))
    dense_case("fc_rand", x, w, capi.fc_params(0.0), g, store)

    B, H, W, C, Kc, Kh, Kw, Sh, Sw = 2, 7, 6, 3, 4, 3, 2, 2, 1
    x = np.exp(np.abs(rng.standard_normal((B, H, W, C)))).astype(np.float32)
    w = rng.standard_normal((Kh * Kw * C + 1, Kc)).astype(np.float32)
    nh, nw = (H - Kh) // Sh + 1, (W - Kw) // Sw + 1
    xpad = np.ascontiguousarray(x[:, :(nh - 1) * Sh + Kh, :(nw - 1) * Sw + Kw, :])
    params = capi.cv_params(Kh, Kw, Sh, Sw, same=False, biasvolt=1.0)
    g = np.zeros((2 * B, nh, nw, Kc), np.float32); g[:B] = rng.standard_normal((B, nh, nw, Kc))
    conv_case("cv_rand", xpad, w, params, g, store)

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "snntc_golden.npz")
    np.savez_compressed(out, **store)
    print("wrote", out, os.path.getsize(out), "bytes,", len(store), "arrays")


if __name__ == "__main__":
    main()
