"""Metamorphic properties of the CPU oracle's forward pass, explored with hypothesis.

None of them restates the neuron's formula: each says how the result must change (or not change)
when the input is transformed in a way whose effect follows from the definition alone.  All
expectations are bit-exact, because the transformations are exact in binary floating point.
"""
import numpy as np
from hypothesis import given, settings, strategies as st

from oracle import capi


def _case(seed, B, I, J, bias):
    rng = np.random.default_rng(seed)
    x = np.exp(2.0 * rng.random((B, I))).astype(np.float32)               # distinct with probability 1
    w = (3.0 / I + rng.standard_normal((I + (1 if bias else 0), J)) * np.sqrt(2.0 / I)).astype(np.float32)
    return x, w


CASES = dict(seed=st.integers(0, 10**6), B=st.integers(1, 4), I=st.integers(1, 40), J=st.integers(1, 9),
             bias=st.booleans())


def _forward(x, w, bias, theta=1.0, max_time=1e5):
    p = capi.fc_params(1.0 if bias else 0.0, max_time=max_time, theta=theta)
    out, k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    B = x.shape[0]
    return out[:B], out[B:], k


@settings(max_examples=60, deadline=None)
@given(m=st.integers(-3, 3), **CASES)
def test_scaling_the_weights_and_the_threshold_leaves_spike_times_unchanged(m, seed, B, I, J, bias):
    """(w, theta) -> 2^m (w, theta): every sum scales exactly, every comparison keeps its outcome."""
    x, w = _case(seed, B, I, J, bias)
    c = np.float32(2.0 ** m)
    y0, r0, k0 = _forward(x, w, bias)
    y1, r1, k1 = _forward(x, w * c, bias, theta=float(c))
    assert np.array_equal(k0, k1)
    assert np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
    assert np.array_equal((r0 / c).view(np.uint32), r1.view(np.uint32))


@settings(max_examples=60, deadline=None)
@given(m=st.integers(-2, 2), **CASES)
def test_scaling_the_spike_times_scales_the_output(m, seed, B, I, J, bias):
    """x -> 2^m x (bias input included): y -> 2^m y, same causal sets, same 1/S."""
    x, w = _case(seed, B, I, J, bias)
    c = np.float32(2.0 ** m)
    p0 = capi.fc_params(1.0 if bias else 0.0)
    p1 = capi.fc_params(float(c) if bias else 0.0)                         # the bias input is a spike time too
    o0, k0, _, _ = capi.fc_forward_dev(x, w, p0, want_aux=True)
    o1, k1, _, _ = capi.fc_forward_dev(x * c, w, p1, want_aux=True)
    fired = k0 >= 0
    assert np.array_equal(k0, k1)
    assert np.array_equal((o0[:B][fired] * c).view(np.uint32), o1[:B][fired].view(np.uint32))
    assert np.array_equal(o0[B:].view(np.uint32), o1[B:].view(np.uint32))


@settings(max_examples=60, deadline=None)
@given(extra=st.integers(1, 5), **CASES)
def test_inputs_that_never_arrive_change_nothing(extra, seed, B, I, J, bias):
    """Extra inputs at MAX_SPIKE_TIME (the padding value), with arbitrary weights, are never consumed."""
    x, w = _case(seed, B, I, J, bias)
    rng = np.random.default_rng(seed + 1)
    x2 = np.concatenate([x, np.full((B, extra), 1e5, np.float32)], axis=1)
    w_extra = (10.0 * rng.standard_normal((extra, J))).astype(np.float32)
    w2 = np.concatenate([w[:I], w_extra, w[I:]], axis=0)                    # the bias row stays last
    y0, r0, k0 = _forward(x, w, bias)
    y1, r1, k1 = _forward(x2, w2, bias)
    assert np.array_equal(k0, k1)
    assert np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
    assert np.array_equal(r0.view(np.uint32), r1.view(np.uint32))


@settings(max_examples=60, deadline=None)
@given(**CASES)
def test_reordering_the_inputs_with_their_weights_changes_nothing(seed, B, I, J, bias):
    """The neuron sees its inputs in time order whatever their position (times distinct here)."""
    x, w = _case(seed, B, I, J, bias)
    order = np.random.default_rng(seed + 2).permutation(I)
    w2 = w.copy()
    w2[:I] = w[order]
    y0, r0, k0 = _forward(x, w, bias)
    y1, r1, k1 = _forward(np.ascontiguousarray(x[:, order]), w2, bias)
    assert np.array_equal(k0, k1)
    assert np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
    assert np.array_equal(r0.view(np.uint32), r1.view(np.uint32))


@settings(max_examples=40, deadline=None)
@given(cut=st.floats(1.2, 6.0), **CASES)
def test_lowering_max_spike_time_only_removes_late_inputs(cut, seed, B, I, J, bias):
    """With MAX_SPIKE_TIME = cut, inputs later than cut - 0.1 are never consumed: the result equals the
    one for the same inputs moved to the padding value (unless the output itself lies beyond cut,
    where it is reported as not fired)."""
    x, w = _case(seed, B, I, J, bias)
    cutf = np.float32(cut)
    late = x > cutf - np.float32(0.1)
    x_moved = np.where(late, np.float32(1e5), x)
    y_cut, r_cut, k_cut = _forward(x, w, bias, max_time=float(cutf))
    y_ref, r_ref, k_ref = _forward(x_moved, w, bias)
    inside = (k_ref >= 0) & (y_ref < cutf)
    assert np.array_equal(k_cut[inside], k_ref[inside])
    assert np.array_equal(y_cut[inside].view(np.uint32), y_ref[inside].view(np.uint32))
    assert np.array_equal(r_cut[inside].view(np.uint32), r_ref[inside].view(np.uint32))
    assert np.all(y_cut[~inside] == cutf) and np.all(r_cut[~inside] == 0) and np.all(k_cut[~inside] == -1)


# ---------------------------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------------------------
def _backward(g, x, w, bias, out):
    p = capi.fc_params(1.0 if bias else 0.0)
    return capi.fc_backward_dev(g, x, w, p, out)


def _fwd_out(x, w, bias):
    return capi.fc_forward_dev(x, w, capi.fc_params(1.0 if bias else 0.0))


@settings(max_examples=40, deadline=None)
@given(m=st.integers(-3, 3), **CASES)
def test_gradients_are_linear_in_the_upstream_gradient(m, seed, B, I, J, bias):
    x, w = _case(seed, B, I, J, bias)
    out = _fwd_out(x, w, bias)
    g = np.zeros((2 * B, J), np.float32)
    g[:B] = np.random.default_rng(seed + 3).standard_normal((B, J))
    c = np.float32(2.0 ** m)
    dx0, dw0, _ = _backward(g, x, w, bias, out)
    dx1, dw1, _ = _backward(g * c, x, w, bias, out)
    assert np.array_equal((dx0 * c).view(np.uint32), dx1.view(np.uint32))
    assert np.array_equal((dw0 * c).view(np.uint32), dw1.view(np.uint32))


@settings(max_examples=40, deadline=None)
@given(**CASES)
def test_samples_are_independent_in_dx_and_add_up_in_dw(seed, B, I, J, bias):
    x, w = _case(seed, B + 1, I, J, bias)
    Bt = B + 1
    out = _fwd_out(x, w, bias)
    g = np.zeros((2 * Bt, J), np.float32)
    g[:Bt] = np.random.default_rng(seed + 4).standard_normal((Bt, J))
    dx, dw, _ = _backward(g, x, w, bias, out)
    dw_sum = np.zeros_like(dw, dtype=np.float64)
    mag = np.zeros_like(dw, dtype=np.float64)
    for b in range(Bt):
        o1 = np.stack((out[b], out[Bt + b]))
        g1 = np.stack((g[b], g[Bt + b]))
        dx1, dw1, _ = _backward(g1, x[b:b + 1], w, bias, o1)
        assert np.array_equal(dx1[0].view(np.uint32), dx[b].view(np.uint32))       # no other sample enters
        dw_sum += dw1
        mag += np.abs(dw1)
    assert np.all(np.abs(dw - dw_sum) <= 1e-6 * np.maximum(mag, 1e-30) * Bt)       # fp32 sum over the batch


@settings(max_examples=40, deadline=None)
@given(extra=st.integers(1, 4), **CASES)
def test_inputs_that_never_arrive_get_no_gradient(extra, seed, B, I, J, bias):
    x, w = _case(seed, B, I, J, bias)
    rng = np.random.default_rng(seed + 5)
    x2 = np.concatenate([x, np.full((B, extra), 1e5, np.float32)], axis=1)
    w2 = np.concatenate([w[:I], rng.standard_normal((extra, J)).astype(np.float32), w[I:]], axis=0)
    out = _fwd_out(x2, w2, bias)
    g = np.zeros((2 * B, J), np.float32)
    g[:B] = rng.standard_normal((B, J))
    dx, dw, _ = _backward(g, x2, w2, bias, out)
    assert np.all(dx[:, I:I + extra] == 0) and np.all(dw[I:I + extra] == 0)
    dx0, dw0, _ = _backward(g, x, w, bias, _fwd_out(x, w, bias))
    assert np.array_equal(dx[:, :I].view(np.uint32), dx0.view(np.uint32))
    assert np.array_equal(dw[:I].view(np.uint32), dw0[:I].view(np.uint32))
