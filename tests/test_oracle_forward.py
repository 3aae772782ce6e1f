"""Pins the forward half of the CPU oracle (oracle/snntc_oracle.c) without a GPU.

Every check compares the C restatement with something that does not share code with it: numpy's
stable argsort, the hand-calculation recipe of the reference's tests (oracle/closed_form.py),
the reference's pure-TF formulation restated in numpy, algebraic invariants of the neuron, a
structurally different algorithm (the reference's event-driven CPU conv), and hand-worked cases.
"""
import numpy as np
import pytest

from helpers import conv_case, dense_case
from oracle import capi, closed_form as cf

GOLDEN = np.load(__import__("os").path.join(__import__("os").path.dirname(__file__), "golden", "snntc_golden.npz"))


# ---------------------------------------------------------------------------------------------
# sort
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 7, 32, 33, 100, 577, 1000])
def test_sort_is_numpy_stable_argsort(n):
    rng = np.random.default_rng(n)
    x = rng.integers(0, max(2, n // 3), (5, n)).astype(np.float32) / 4        # many ties
    x[0, ::3] = 1e5                                                             # padding values
    x[1, :] = 3.0                                                               # one value only
    sorted_, perm = capi.sort_segments(x)
    want = np.argsort(x, axis=1, kind="stable").astype(np.int32)
    assert np.array_equal(perm, want)
    assert np.array_equal(sorted_, np.take_along_axis(x, want, axis=1))


def test_sort_negative_values_and_zero_signs():
    x = np.array([[0.0, -0.0, -1.5, 2.0, -0.0, 0.0, -3.0]], np.float32)
    _, perm = capi.sort_segments(x)
    assert perm.tolist() == [[6, 2, 0, 1, 4, 5, 3]]        # -0 == +0: index order decides


# ---------------------------------------------------------------------------------------------
# dense forward, device semantics
# ---------------------------------------------------------------------------------------------
def _margins(x, w, params):
    """Relative distance of every neuron's float64 spike time from its two decision boundaries."""
    y, k, S = cf.fc_forward_closed_form(x, w, params)
    return y, k, S


@pytest.mark.parametrize("seed,B,I,J,bias,dist", [
    (0, 8, 60, 20, True, "reftest"), (1, 8, 60, 20, False, "reftest"),
    (2, 6, 200, 33, True, "baseline"), (3, 6, 200, 33, False, "baseline"), (4, 3, 1, 5, True, "reftest"),
])
def test_fc_forward_dev_matches_reference_test_recipe(seed, B, I, J, bias, dist):
    x, w, p, _ = dense_case(seed, B, I, J, bias, dist)
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    y, kc, S = cf.fc_forward_closed_form(x, w, p)
    # fp32 and fp64 may legitimately pick different prefixes only when a decision is closer than
    # fp32 resolution; these seeds have none
    assert np.array_equal(k, kc)
    fired = kc >= 0
    assert fired.any()
    # y = ysum/S loses 1/|S| digits to cancellation in S = sum(w) - 1
    cond = np.maximum(1.0, 1.0 / np.abs(S[fired]))
    assert np.all(np.abs(out[:B][fired] - y[fired]) <= 2e-5 * np.abs(y[fired]) * cond)
    assert np.all(np.abs(out[B:][fired] * S[fired] - 1.0) <= 2e-5 * cond)
    assert np.all(out[:B][~fired] == np.float32(1e5)) and np.all(out[B:][~fired] == 0)


def test_fc_forward_dev_bias_first_equals_recipe_with_appended_bias():
    """The reference tests append x=1 and sort it with the inputs; the kernels take the bias first.
    For inputs >= 1 (z = exp(t), t >= 0) both give the same neuron."""
    x, w, p, _ = dense_case(11, 4, 30, 6, True, "reftest")
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    for b in range(4):
        for j in range(6):
            y, kk, S = cf.neuron_closed_form(x[b], w[:30, j], w[30, j], bias_first=False)
            assert kk == k[b, j]
            if kk >= 0:      # y = ysum/S loses 1/|S| digits to cancellation in S = sum(w) - 1
                assert abs(out[b, j] - y) <= 2e-5 * abs(y) * max(1.0, 1.0 / abs(S))


def test_fc_forward_dev_matches_pure_tf_formulation():
    """cumsum / where / reduce_min statement of snntc/SNN_TC_pyref.py:28-53.  Valid where that
    formulation and the kernels share semantics: inputs >= 1, positive denominators."""
    x, w, p, _ = dense_case(5, 6, 80, 12, True, "baseline")
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    ref = cf.fc_forward_pyref(x, w, bias=True)
    fired = k >= 0
    assert fired.all()
    assert np.all(1.0 / out[6:] > 0)                     # no negative-denominator firing here
    np.testing.assert_allclose(out[:6], ref, rtol=2e-5)


def test_fc_forward_dev_invariants():
    x, w, p, _ = dense_case(6, 10, 120, 40, True, "reftest")
    B, I = x.shape
    out, k, sorted_, perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    y, r = out[:B].astype(np.float64), out[B:].astype(np.float64)
    fired = k >= 0
    for b, j in zip(*np.nonzero(fired)):
        kk = k[b, j]
        last = sorted_[b, kk - 1] if kk > 0 else 1.0          # bias input when k == 0
        assert y[b, j] >= last * (1 - 1e-6)                    # spike after its last causal input
        if kk < I:
            assert y[b, j] <= sorted_[b, kk] * (1 + 1e-6)      # and not after the next input
        idx = perm[b, :kk]
        S = w[idx, j].astype(np.float64).sum() + w[I, j] - 1.0
        ysum = (w[idx, j].astype(np.float64) * x[b, idx]).sum() + w[I, j]
        assert abs(r[b, j] * S - 1) < 1e-4
        assert abs(y[b, j] * S - ysum) <= 1e-4 * max(1.0, abs(ysum))
    assert np.all(out[:B][~fired] == np.float32(1e5)) and np.all(out[B:][~fired] == 0)


def test_fc_forward_dev_is_invariant_to_input_permutation():
    x, w, p, _ = dense_case(7, 5, 64, 9, True, "baseline")
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    rng = np.random.default_rng(0)
    sh = rng.permutation(64)
    w2 = np.concatenate((w[:64][sh], w[64:]))
    out2, k2, _, _ = capi.fc_forward_dev(x[:, sh], w2, p, want_aux=True)
    assert np.array_equal(k, k2) and np.array_equal(out, out2)   # distinct inputs: same sorted sequence


def test_fc_forward_dev_hand_worked_neurons():
    p = capi.fc_params(0.0)
    # two inputs 2 and 3 with weights 1.5 and 1: prefix {2}: y = 3/0.5 = 6 > 3 -> not closed;
    # prefix {2,3}: y = (3+3)/1.5 = 4 > 3 and nothing follows -> fires at 4, 1/S = 1/1.5
    out, k, _, _ = capi.fc_forward_dev(np.array([[3.0, 2.0]], np.float32), np.array([[1.0], [1.5]], np.float32), p,
                                       want_aux=True)
    assert k[0, 0] == 2 and out[0, 0] == np.float32(4.0) and out[1, 0] == np.float32(1 / 1.5)
    # weights 3 and 1: prefix {2}: y = 6/2 = 3 > 2 and <= next input 3 -> fires at 3 with one input
    out, k, _, _ = capi.fc_forward_dev(np.array([[2.0, 3.0]], np.float32), np.array([[3.0], [1.0]], np.float32), p,
                                       want_aux=True)
    assert k[0, 0] == 1 and out[0, 0] == np.float32(3.0) and out[1, 0] == np.float32(0.5)
    # sum of weights below the threshold and positive sums: never fires
    out, k, _, _ = capi.fc_forward_dev(np.array([[2.0, 3.0]], np.float32), np.array([[0.2], [0.3]], np.float32), p,
                                       want_aux=True)
    assert k[0, 0] == -1 and out[0, 0] == np.float32(1e5) and out[1, 0] == 0
    # bias alone fires: bias weight 4 -> y = 4/3 > 1 and <= first input 2 -> k = 0
    pb = capi.fc_params(1.0)
    out, k, _, _ = capi.fc_forward_dev(np.array([[2.0, 3.0]], np.float32),
                                       np.array([[0.1], [0.1], [4.0]], np.float32), pb, want_aux=True)
    assert k[0, 0] == 0 and out[0, 0] == np.float32(np.float32(4.0) * (np.float32(1.0) / np.float32(3.0)))
    # all inputs are padding: bias decides alone
    out, k, _, _ = capi.fc_forward_dev(np.full((1, 3), 1e5, np.float32),
                                       np.array([[0.1], [0.1], [0.1], [4.0]], np.float32), pb, want_aux=True)
    assert k[0, 0] == 0 and abs(out[0, 0] - 4 / 3) < 1e-6


def test_fc_forward_dev_stops_at_padding_inputs():
    """Inputs above MAX-0.1 end the scan (snntc/snnfc_kernels.cu.cc:45): their weights never count."""
    p = capi.fc_params(0.0)
    x = np.array([[2.0, 1e5, 3.0]], np.float32)
    w = np.array([[0.8], [100.0], [0.8]], np.float32)
    out, k, _, perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    # prefix {2,3}: S = 0.6, y = (1.6+2.4)/0.6 = 6.67 > 3, next is padding -> fires with k = 2
    assert perm.tolist() == [[0, 2, 1]] and k[0, 0] == 2
    assert abs(out[0, 0] - 4.0 / 0.6) < 1e-5


# ---------------------------------------------------------------------------------------------
# host-semantics forward (the timed CPU baseline) against the device semantics
# ---------------------------------------------------------------------------------------------
def test_fc_forward_host_agrees_with_dev_away_from_documented_divergences():
    x, w, p, _ = dense_case(8, 16, 100, 30, True, "baseline")
    w[100] = 0.0                                  # zero bias row: the host bias `break` cannot trigger
    B = 16
    dev = capi.fc_forward_dev(x, w, p)
    host = capi.fc_forward_host(x, w, p)
    np.testing.assert_allclose(host[:B], dev[:B], rtol=1e-5)
    fired = dev[B:] != 0
    np.testing.assert_allclose(host[B:][fired] * dev[B:][fired], 1.0, rtol=1e-5)   # host stores S, dev 1/S


def test_fc_forward_host_bias_break_quirk():
    """When the bias alone fires output j, the reference's CPU loop leaves the j loop of that sample
    (snntc/snnfc_kernels.cc:122): later outputs keep MAX.  The device semantics do not."""
    p = capi.fc_params(1.0)
    x = np.array([[2.0, 3.0]], np.float32)
    w = np.array([[3.0, 3.0, 3.0], [1.0, 1.0, 1.0], [0.0, 4.0, 0.0]], np.float32)
    host = capi.fc_forward_host(x, w, p)
    dev = capi.fc_forward_dev(x, w, p)
    assert host[0, 0] == np.float32(3.0) and abs(host[0, 1] - 4 / 3) < 1e-6 and host[0, 2] == np.float32(1e5)
    assert dev[0, 0] == np.float32(3.0) and abs(dev[0, 1] - 4 / 3) < 1e-6 and dev[0, 2] == np.float32(3.0)


# ---------------------------------------------------------------------------------------------
# conv forward
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed,B,H,W,C,Kc,Kh,Kw,Sh,Sw,same,bias", [
    (0, 2, 6, 7, 3, 5, 3, 3, 1, 1, True, True), (1, 2, 9, 8, 2, 4, 2, 4, 3, 2, False, True),
    (2, 1, 10, 10, 4, 3, 5, 5, 2, 2, True, False), (3, 2, 5, 5, 1, 2, 6, 6, 1, 1, True, True),
])
def test_cv_forward_dev_is_dense_on_numpy_patches(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias):
    _, xpad, w, p, _ = conv_case(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias, "reftest")
    out, k, sorted_, perm = capi.cv_forward_dev(xpad, w, p, want_aux=True)
    patches = cf.im2col(xpad, Kh, Kw, Sh, Sw)                      # numpy slicing, not the C im2col
    assert np.array_equal(capi.im2col(xpad, p), patches)
    p6 = np.array([p[0], p[3], p[4], 0, 0, p[11]], np.float32)
    out2, k2, s2, perm2 = capi.fc_forward_dev(patches, w, p6, want_aux=True)
    S = patches.shape[0]
    assert np.array_equal(out.reshape(2 * S, Kc), out2) and np.array_equal(k, k2)
    assert np.array_equal(perm, perm2) and np.array_equal(sorted_, s2)
    y, kc, _ = cf.fc_forward_closed_form(patches, w, p6)
    assert np.array_equal(k, kc)


@pytest.mark.parametrize("seed,B,H,W,C,Kc,Kh,Kw,Sh,Sw,same", [
    (0, 2, 8, 8, 3, 6, 3, 3, 1, 1, True), (1, 1, 9, 7, 2, 4, 3, 2, 2, 1, False), (2, 1, 12, 12, 3, 5, 7, 7, 2, 2, True),
])
def test_cv_forward_host_event_driven_algorithm_agrees_with_dev(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same):
    """The reference's CPU conv (one global sort + event scatter) is a structurally different
    algorithm; on tie-free inputs it must give the kernels' spike times."""
    _, xpad, w, p, _ = conv_case(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, True, "baseline")
    dev = capi.cv_forward_dev(xpad, w, p)
    host = capi.cv_forward_host(xpad, w, p)
    np.testing.assert_allclose(host, dev[:B], rtol=1e-5)


def test_reference_deterministic_conv_fixtures():
    """Inputs of snntc/test-snn-cv-backward.py testmode 0/1/2; expected values from the committed
    golden file (oracle and closed form agreed when it was written)."""
    for mode in range(3):
        xpad, w, p = (GOLDEN[f"cvtest{mode}_{n}"] for n in ("xpad", "w", "params"))
        out, k, sorted_, perm = capi.cv_forward_dev(xpad, w, p, want_aux=True)
        assert np.array_equal(out, GOLDEN[f"cvtest{mode}_out"])
        assert np.array_equal(k, GOLDEN[f"cvtest{mode}_k"])
        assert np.array_equal(perm, GOLDEN[f"cvtest{mode}_perm"])
        assert np.all(out[:out.shape[0] // 2] > 1)      # "Something wrong: some outputs <= 1" check of the reference tests
        # the hand-calculation recipe of the reference (bias appended as x = 1 and sorted with the rest)
        Kh, Kw, Sh, Sw = (int(p[t]) for t in (6, 7, 8, 9))
        patches = cf.im2col(xpad, Kh, Kw, Sh, Sw)
        P = patches.shape[1]
        flat = out[:out.shape[0] // 2].reshape(-1, w.shape[1])
        for s in range(patches.shape[0]):
            for kc in range(w.shape[1]):
                y, kk, SS = cf.neuron_closed_form(patches[s], w[:P, kc], w[P, kc], bias_first=False)
                assert kk == k[s, kc] and abs(flat[s, kc] - y) <= 2e-5 * abs(y) * max(1.0, 1.0 / abs(SS))


@pytest.mark.parametrize("name", ["fc_ties", "fc_edge", "fc_rand"])
def test_golden_dense_vectors(name):
    x, w, p = (GOLDEN[f"{name}_{n}"] for n in ("x", "w", "params"))
    out, k, sorted_, perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    assert np.array_equal(out, GOLDEN[f"{name}_out"]) and np.array_equal(k, GOLDEN[f"{name}_k"])
    assert np.array_equal(perm, GOLDEN[f"{name}_perm"]) and np.array_equal(sorted_, GOLDEN[f"{name}_sorted"])


def test_same_padding_rule():
    """SNN_conv's split (SNN_TC_Modules.py:147-161) equals TensorFlow's documented SAME rule
    (total = max((ceil(n/s)-1)*s + k - n, 0), smaller half first) whenever the total is >= 0."""
    for n in range(1, 40):
        for k in range(1, 8):
            for s in range(1, 4):
                before, after = cf.same_pad(n, k, s)
                total = (-(-n // s) - 1) * s + k - n
                assert before + after == total
                if total >= 0:
                    assert before == total // 2 and after == total - total // 2
                    assert (n + total - k) // s + 1 == -(-n // s)          # output size ceil(n/s)


@pytest.mark.parametrize("biasvolt,theta,max_time", [(0.7, 1.0, 1e5), (2.5, 0.5, 1e5), (1.0, 2.0, 50.0), (0.0, 1.5, 20.0)])
def test_fc_forward_dev_non_default_parameters_match_closed_form(biasvolt, theta, max_time):
    """biasvolt, threshold and MAX away from their defaults, with MAX sentinels among the inputs: the
    oracle against the float64 closed form (first valid prefix of the sorted inputs)."""
    rng = np.random.default_rng(int(10 * biasvolt + 100 * theta))
    B, I, J = 9, 80, 17
    rows = I + (1 if biasvolt > 1e-8 else 0)
    x = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
    x[rng.random((B, I)) < 0.15] = np.float32(max_time)
    x[2, :] = np.float32(max_time)
    w = ((4.0 / I + np.sqrt(1.0 / I) * rng.standard_normal((rows, J))) * theta).astype(np.float32)
    p = capi.fc_params(biasvolt, max_time=max_time, theta=theta)
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    y, kc, S = cf.fc_forward_closed_form(x, w, p)
    assert np.array_equal(k, kc)
    fired = kc >= 0
    assert fired.any() and (~fired).any()
    cond = np.maximum(1.0, 1.0 / np.abs(S[fired]))
    assert np.all(np.abs(out[:B][fired] - y[fired]) <= 2e-5 * np.abs(y[fired]) * cond)
    assert np.all(out[:B][~fired] == np.float32(max_time)) and np.all(out[B:][~fired] == 0)
    assert np.all(out[:B][2] == np.float32(max_time)) or biasvolt > 1e-8     # a row of sentinels: only the bias can fire
