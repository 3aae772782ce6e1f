"""GPU parity: the HIP library (through the Python ops, i.e. through the C ABI) against the CPU
oracle on the same seeded inputs.

Bars: sorted values, permutations and causal-set sizes bit-exact; spike times and reciprocals
bit-exact (the scan reproduces the oracle's fp32 operation order); gradients within
rel 1e-5 / abs 1e-6 of the float64-accumulated oracle plus 5e-7 of the sum of the absolute summands
(helpers.grad_band: two fp32 summation orders of the same terms differ by a multiple of that).
"""
import numpy as np
import pytest
import torch

from helpers import assert_close, conv_case, dense_case, grad_band
from oracle import capi

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def check_grad(actual, ref, ref_abs, what):
    a = np.asarray(actual, np.float64); e = np.asarray(ref, np.float64)
    lim = grad_band(e, ref_abs)
    err = np.abs(a - e)
    bad = err > lim
    if bad.any():
        idx = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: {bad.sum()}/{bad.size} out of tolerance; worst {idx}: got {a[idx]!r} "
                             f"want {e[idx]!r} diff {err[idx]:.3e} lim {lim[idx]:.3e}")
    import os
    if os.environ.get("SNNTC_BAND_LOG") and a.size:
        with open(os.environ["SNNTC_BAND_LOG"], "a") as f:
            f.write(f"{what} n={a.size} worst_ratio={float((err / lim).max()):.4f}\n")


DENSE_CASES = [
    # seed, B, I, J, bias, dist
    (0, 128, 784, 800, True, "baseline"),      # BASELINE config 1
    (1, 128, 784, 800, False, "baseline"),
    (2, 32, 800, 10, True, "baseline"),        # classifier head: J < one wavefront
    (3, 7, 1, 3, True, "reftest"),             # shortest possible segment
    (4, 5, 33, 65, False, "reftest"),
    (5, 19, 257, 129, True, "reftest"),
    (6, 3, 1000, 70, True, "reftest"),
    (7, 4, 2048, 96, True, "baseline"),        # cross-wavefront sort
    (8, 2, 5000, 40, False, "reftest"),        # 8192-wide sort
    # layers with at most 16 outputs take a backward pass of their own (one launch for the masked
    # upstream values, dX and dW; 256 samples per block, 16 weight rows per wavefront)
    (9, 256, 800, 10, True, "baseline"),       # the MLP's head at its batch
    (10, 600, 95, 16, True, "reftest"),        # three blocks of samples, the last one partial
    (11, 257, 17, 1, False, "reftest"),        # one output, no bias row, one sample past a block
    (12, 33, 48, 13, True, "reftest"),         # bias row opens a block of its own
    (13, 40, 64, 17, True, "reftest"),         # first width past that pass
    # the remaining dense layers of the benchmark networks at their batch sizes
    (14, 256, 800, 800, True, "baseline"),     # MLP hidden layer
    (15, 128, 2048, 512, True, "baseline"),    # CIFAR-shaped net, first dense layer
    (16, 128, 512, 10, True, "baseline"),      # CIFAR-shaped net, head
    (17, 32, 512, 1000, True, "baseline"),     # ImageNet-shaped net, classifier
    # inputs so long that not even 8 weight columns fit in LDS beside the kernels' chunk buffers: the scan
    # streams the weight rows (I + bias > 5054), and the last size that still uses the LDS-resident slice
    (18, 3, 5053, 24, True, "baseline"),       # 5054 rows x 8 columns: the largest slice that is kept in LDS
    (27, 2800, 5053, 24, True, "baseline"),    # the same slice under the filter kernel (a large batch)
    (28, 3, 5054, 24, True, "baseline"),       # 5055 rows: first size that streams
    (29, 2800, 5100, 24, True, "baseline"),    # 5055..5120 rows at a large batch: streaming scan
    (19, 3, 5120, 24, False, "baseline"),      # 160 KB exactly: streaming scan
    (20, 3, 5120, 70, True, "baseline"),       # streaming scan, two column blocks
    (21, 2, 8192, 33, True, "reftest"),        # the longest segment one sorting network takes
    # longer segments: sorted in pieces of 8192 and merged in global memory
    (23, 3, 8193, 20, True, "reftest"),        # two pieces, the second with a single input
    (24, 2, 12000, 70, False, "baseline"),     # two pieces, one merge pass
    (25, 2, 20000, 24, True, "reftest"),       # three pieces: a pass with an unpaired run
    (26, 1, 41000, 9, True, "baseline"),       # six pieces, three passes; narrow backward pass
    (22, 5, 6000, 7, False, "reftest"),        # streaming scan with a narrow layer (the narrow backward pass)
]


@pytest.mark.parametrize("seed,B,I,J,bias,dist", DENSE_CASES)
def test_dense_forward_backward(seed, B, I, J, bias, dist):
    import snntc_amd as snn
    x, w, p, g = dense_case(seed, B, I, J, bias, dist)
    ref_out, ref_k, ref_sorted, ref_perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, sz, perm, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    out2 = snn.snnfc(t(x), t(w), p)
    torch.cuda.synchronize()
    out, sz, perm, ck, out2 = (v.cpu().numpy() for v in (out, sz, perm, ck, out2))
    assert np.array_equal(sz, ref_sorted), "sorted values differ"
    assert np.array_equal(perm, ref_perm), "permutation differs"
    assert np.array_equal(ck, ref_k), f"causal-set sizes differ at {np.argwhere(ck != ref_k)[:5]}"
    assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y / 1/S not bit-exact"
    assert np.array_equal(out2.view(np.uint32), out.view(np.uint32)), "plain and _ex entry points differ"

    dx, dw, dp = snn.snnfc_grad(t(g), t(x), t(w), p, t(ref_out))
    torch.cuda.synchronize()
    dx, dw, dp = dx.cpu().numpy(), dw.cpu().numpy(), dp.cpu().numpy()
    rdx, rdw, _ = capi.fc_backward_dev(g, x, w, p, ref_out, wide=True)
    absout = ref_out.copy(); absout[B:] = np.abs(absout[B:])
    adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, absout, wide=True)
    check_grad(dx, rdx, adx, "dX")
    check_grad(dw, rdw, adw, "dW")
    assert np.all(dp == 0)
    # the fp32 sequential oracle must sit inside the same band
    sdx, sdw, _ = capi.fc_backward_dev(g, x, w, p, ref_out)
    check_grad(sdx, rdx, adx * 8, "oracle fp32 dX")
    check_grad(sdw, rdw, adw * 8, "oracle fp32 dW")


def _adversarial_dense(kind, seed, B, I, J):
    """Inputs that take the scan off its common path: weights of both signs (neurons that fire on a
    negative weight sum, that never fire, whose weight sum crosses zero many times), exact ties between
    an output and an input, inputs below zero, all-zero weights, a bias that fires alone."""
    rng = np.random.default_rng(seed)
    if kind == "randn":                      # the reference scripts' law
        x = np.exp(np.abs(rng.standard_normal((B, I))))
        w = rng.standard_normal((I + 1, J))
    elif kind == "ties":                     # few distinct times, weights on a coarse grid: y == x happens
        x = 1.0 + rng.integers(0, 8, (B, I)) / 4.0
        w = rng.integers(-2, 6, (I + 1, J)) / 16.0
    elif kind == "negative":                 # times below zero
        x = rng.standard_normal((B, I)) * 2.0
        w = 0.3 * rng.standard_normal((I + 1, J)) + 0.1
    elif kind == "sparse":                   # mostly zero weights, some columns all zero
        x = np.exp(rng.random((B, I)))
        w = rng.standard_normal((I + 1, J)) * (rng.random((I + 1, J)) < 0.1)
        w[:, ::7] = 0.0
    elif kind == "bias_fires":               # bias weight above the threshold: fired before the first input
        x = np.exp(1.0 + rng.random((B, I)))
        w = 4.0 / I + np.sqrt(1.0 / I) * rng.standard_normal((I + 1, J))
        w[I, ::2] = 1.5 + rng.random(J)[::2]
    elif kind == "late":                     # small weights: sets close near the end of the row or not at all
        x = np.exp(rng.random((B, I)))
        w = (1.05 / I) * (1.0 + 0.2 * rng.standard_normal((I + 1, J)))
    else:
        raise ValueError(kind)
    return x.astype(np.float32), w.astype(np.float32)


@pytest.mark.parametrize("kind,seed,B,I,J", [
    # one neuron per lane, one segment per wavefront (64-column slices), and two segments (32-column slices)
    ("randn", 0, 4096, 64, 64), ("ties", 1, 4096, 64, 64), ("negative", 2, 4096, 72, 64),
    ("sparse", 3, 3000, 203, 130), ("bias_fires", 4, 3000, 131, 70), ("late", 5, 2500, 330, 96),
    ("randn", 6, 1500, 700, 100), ("ties", 7, 2000, 1000, 40),
    # two neurons per lane (launches with many work items)
    ("randn", 8, 20000, 40, 64), ("ties", 9, 20000, 48, 33), ("negative", 10, 18000, 27, 64),
    ("bias_fires", 11, 20000, 35, 20), ("late", 12, 9000, 100, 128), ("sparse", 13, 17000, 19, 8),
])
def test_filtered_scan_off_the_common_path(kind, seed, B, I, J):
    """Launches large enough for the scan that skips provably idle tests, on inputs chosen so that its
    rare branches run: chunks stepped through without closing, scans that return to the fast loop or
    stay on the step-by-step path, rows with tails, neurons that fired before the first input."""
    import snntc_amd as snn
    x, w = _adversarial_dense(kind, seed, B, I, J)
    p = capi.fc_params(1.0)
    ref_out, ref_k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, _, _, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    out2 = snn.snnfc(t(x), t(w), p)
    torch.cuda.synchronize()
    out, ck, out2 = out.cpu().numpy(), ck.cpu().numpy(), out2.cpu().numpy()
    assert np.array_equal(ck, ref_k), f"causal-set sizes differ at {np.argwhere(ck != ref_k)[:5]}"
    assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y / 1/S not bit-exact"
    assert np.array_equal(out2.view(np.uint32), out.view(np.uint32)), "plain and _ex entry points differ"


@pytest.mark.parametrize("B,I,J", [(300, 70, 10), (64, 100, 48)])
def test_dense_backward_single_gradient_calls_match_the_joint_call(B, I, J):
    """A NULL dX or dW output is simply not computed; the other one must not change by a bit."""
    import snntc_amd as snn
    x, w, p, g = dense_case(21, B, I, J, True, "reftest")
    out = snn.snnfc(t(x), t(w), p)
    dx, dw, _ = snn.snnfc_grad(t(g), t(x), t(w), p, out)
    dx_only, none_w, _ = snn.snnfc_grad(t(g), t(x), t(w), p, out, want_dw=False)
    none_x, dw_only, _ = snn.snnfc_grad(t(g), t(x), t(w), p, out, want_dx=False)
    torch.cuda.synchronize()
    assert none_w is None and none_x is None
    assert torch.equal(dx_only, dx), "dX changes when dW is not asked for"
    assert torch.equal(dw_only, dw), "dW changes when dX is not asked for"


CONV_CASES = [
    # seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias, dist
    (0, 2, 32, 32, 64, 64, 3, 3, 1, 1, True, True, "baseline"),     # BASELINE config 3 shape, small batch
    (1, 4, 32, 32, 3, 32, 3, 3, 1, 1, True, True, "baseline"),      # first CIFAR layer, P = 27
    (2, 2, 16, 16, 32, 64, 3, 3, 1, 1, True, False, "baseline"),
    (3, 2, 29, 23, 3, 16, 7, 7, 2, 2, True, True, "baseline"),      # 7x7 stride 2
    (4, 3, 11, 13, 5, 7, 2, 4, 3, 1, False, True, "reftest"),       # VALID, ragged everything
    (5, 2, 9, 9, 4, 70, 5, 6, 2, 3, True, False, "reftest"),
    (6, 1, 8, 8, 128, 128, 3, 3, 1, 1, True, True, "baseline"),     # P = 1152
    (7, 1, 4, 4, 512, 96, 3, 3, 1, 1, True, True, "baseline"),      # P = 4608
    (8, 2, 10, 9, 48, 20, 3, 2, 2, 1, True, True, "reftest"),       # channels not a power of two
    (9, 2, 9, 9, 32, 16, 3, 3, 2, 2, True, False, "baseline"),      # stride 2 with 32 channels
    (10, 1, 12, 7, 40, 8, 2, 3, 1, 2, False, True, "reftest"),      # VALID, ragged kernel and stride
    (11, 1, 3, 4, 1024, 24, 3, 3, 1, 1, True, True, "baseline"),    # P = 9216: patches longer than one sorting network
    # patches whose merge buffers fit in LDS only once per workgroup (merged by all its wavefronts together)
    (12, 2, 7, 7, 512, 8, 3, 3, 1, 1, True, True, "baseline"),      # rows of 7 patches: tiles of 4 and 3
    (13, 1, 6, 9, 512, 8, 3, 2, 2, 2, False, True, "reftest"),      # VALID, stride 2, two-column kernel
    (14, 1, 4, 5, 640, 8, 3, 3, 1, 1, True, False, "reftest"),      # channel count not a power of two, P = 5760
    # few input channels and patches of at least 64 entries: the patch order comes from counts shared between
    # neighbouring patches
    (15, 2, 40, 37, 3, 16, 7, 7, 2, 2, True, True, "baseline"),     # the 7x7/2 stem on an odd image: partial last tiles
    (16, 2, 12, 12, 1, 8, 8, 8, 1, 1, True, True, "reftest"),       # one channel
    (17, 1, 9, 20, 16, 8, 3, 3, 1, 1, False, True, "reftest"),      # 16 channels, VALID
    (18, 1, 10, 9, 31, 8, 8, 2, 1, 1, True, False, "reftest"),      # columns of 248 entries
    (19, 2, 9, 30, 8, 8, 3, 3, 2, 5, False, True, "reftest"),       # stride wider than the kernel: no shared columns
    (20, 2, 13, 7, 96, 4, 3, 6, 3, 2, False, True, "reftest"),      # many channels, a single patch per output row
    # fewer than 32 input channels with a multiple of 16 output channels: dX by channel lanes with the wavefront cut
    # into 4, 8 or 16 parts that take neighbouring tiles
    (21, 2, 14, 30, 16, 32, 3, 3, 1, 1, True, True, "baseline"),    # 16 channels: four parts
    (22, 2, 10, 70, 8, 16, 3, 3, 1, 1, True, False, "baseline"),    # 8 channels: eight parts, two tiles per row
    (23, 1, 9, 150, 4, 16, 3, 3, 1, 1, True, True, "baseline"),     # 4 channels: sixteen parts, tiles of 128 pixels
    (24, 2, 11, 40, 24, 48, 5, 5, 1, 1, True, True, "baseline"),    # 24 of 32 lanes per part, five-column kernel
    (25, 2, 12, 33, 12, 64, 3, 3, 2, 2, True, False, "baseline"),   # 12 of 16 lanes, stride 2: every second slot empty
    (26, 1, 8, 20, 2, 16, 3, 3, 1, 2, False, True, "reftest"),      # two channels, VALID, column stride 2
]


@pytest.mark.parametrize("seed,B,H,W,C,Kc,Kh,Kw,Sh,Sw,same,bias,dist", CONV_CASES)
def test_conv_forward_backward(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias, dist):
    import snntc_amd as snn
    _, xpad, w, p, g = conv_case(seed, B, H, W, C, Kc, Kh, Kw, Sh, Sw, same, bias, dist)
    ref_out, ref_k, ref_sorted, ref_perm = capi.cv_forward_dev(xpad, w, p, want_aux=True)
    out, sz, perm, ck = snn.snncv(t(xpad), t(w), p, return_aux=True)
    out2 = snn.snncv(t(xpad), t(w), p)
    torch.cuda.synchronize()
    out, sz, perm, ck, out2 = (v.cpu().numpy() for v in (out, sz, perm, ck, out2))
    assert out.shape == ref_out.shape
    assert np.array_equal(sz, ref_sorted), "sorted values differ"
    assert np.array_equal(perm, ref_perm), "permutation differs"
    assert np.array_equal(ck, ref_k), "causal-set sizes differ"
    assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y / 1/S not bit-exact"
    assert np.array_equal(out2.view(np.uint32), out.view(np.uint32))

    dx, dw, dp = snn.snncv_grad(t(g), t(xpad), t(w), p, t(ref_out))
    torch.cuda.synchronize()
    dx, dw, dp = dx.cpu().numpy(), dw.cpu().numpy(), dp.cpu().numpy()
    rdx, rdw, _ = capi.cv_backward_dev(g, xpad, w, p, ref_out, wide=True)
    absout = ref_out.copy(); absout[B:] = np.abs(absout[B:])
    adx, adw, _ = capi.cv_backward_dev(np.abs(g), xpad, np.abs(w), p, absout, wide=True)
    check_grad(dx, rdx, adx, "dXpad")
    check_grad(dw, rdw, adw, "dW")
    assert np.all(dp == 0)


@pytest.mark.parametrize("C,Kh,Kw,Sh,Sw", [(32, 3, 3, 1, 1), (64, 3, 3, 1, 1), (3, 3, 3, 1, 1), (40, 2, 3, 1, 2),
                                           (3, 7, 7, 2, 2), (8, 3, 5, 1, 2),
                                           (128, 3, 3, 1, 1), (256, 3, 3, 1, 1), (512, 3, 3, 1, 1)])
def test_conv_sort_with_heavy_ties(C, Kh, Kw, Sh, Sw):
    """Quantised inputs: most values repeat inside a patch (and SAME padding adds runs of 1e5), so
    the permutation is decided by the stable tie rule (kh, kw, c) almost everywhere."""
    import snntc_amd as snn
    from oracle.closed_form import same_pad
    rng = np.random.default_rng(C + Kh)
    B, H, W, Kc = 2, 7, 9, 16
    x = (1.0 + rng.integers(0, 6, (B, H, W, C)) / 4.0).astype(np.float32)
    (tp, bt), (lf, rt) = same_pad(H, Kh, Sh), same_pad(W, Kw, Sw)
    xpad = np.ascontiguousarray(np.pad(x, ((0, 0), (tp, bt), (lf, rt), (0, 0)), constant_values=np.float32(1e5)))
    w = (rng.standard_normal((Kh * Kw * C + 1, Kc)) * 0.3 + 0.05).astype(np.float32)
    p = capi.cv_params(Kh, Kw, Sh, Sw, same=True, biasvolt=1.0)
    ref_out, ref_k, ref_sorted, ref_perm = capi.cv_forward_dev(xpad, w, p, want_aux=True)
    out, sz, perm, ck = snn.snncv(t(xpad), t(w), p, return_aux=True)
    torch.cuda.synchronize()
    assert np.array_equal(perm.cpu().numpy(), ref_perm), "permutation differs"
    assert np.array_equal(sz.cpu().numpy(), ref_sorted)
    assert np.array_equal(ck.cpu().numpy(), ref_k)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref_out.view(np.uint32))


@pytest.mark.parametrize("I", [8200, 16385, 30000])
def test_long_segment_sort_with_heavy_ties(I):
    """Segments longer than one sorting network, quantised so that equal values sit in different
    pieces: the merge passes must keep them in index order; some inputs lie above MAX_SPIKE_TIME - 0.1
    (they sort last and do not count as scan inputs), one row has none below it."""
    import snntc_amd as snn
    rng = np.random.default_rng(I)
    B, J = 3, 5
    x = (1.0 + rng.integers(0, 9, (B, I)) / 8.0).astype(np.float32)
    x[0, rng.integers(0, I, 40)] = 2e5
    x[2, :] = 3e5
    w = (rng.standard_normal((I + 1, J)) * 0.05 + 4.0 / I).astype(np.float32)
    p = capi.fc_params(1.0)
    ref_out, ref_k, ref_sorted, ref_perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, sz, perm, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    torch.cuda.synchronize()
    assert np.array_equal(perm.cpu().numpy(), ref_perm), "permutation differs"
    assert np.array_equal(sz.cpu().numpy(), ref_sorted)
    assert np.array_equal(ck.cpu().numpy(), ref_k)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref_out.view(np.uint32))


@pytest.mark.parametrize("I", [147, 200, 256])
def test_many_short_segments_take_the_two_per_wavefront_sort(I):
    """65 536 and more segments of 129..256 inputs (the patches of a 7x7x3 stem) are sorted two per
    wavefront with eight elements per thread; quantised values make ties that must keep index order,
    a few rows carry inputs above MAX_SPIKE_TIME - 0.1.  Everything bit for bit against the oracle."""
    import snntc_amd as snn
    rng = np.random.default_rng(I)
    B, J = 65536 + 3, 4
    x = (1.0 + rng.integers(0, 40, (B, I)) / 16.0).astype(np.float32)
    x[5, rng.integers(0, I, 9)] = 2e5
    x[B - 1, :] = 3e5
    w = (rng.standard_normal((I + 1, J)) * 0.1 + 4.0 / I).astype(np.float32)
    p = capi.fc_params(1.0)
    ref_out, ref_k, ref_sorted, ref_perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, sz, perm, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    torch.cuda.synchronize()
    assert np.array_equal(perm.cpu().numpy(), ref_perm), "permutation differs"
    assert np.array_equal(sz.cpu().numpy(), ref_sorted)
    assert np.array_equal(ck.cpu().numpy(), ref_k)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref_out.view(np.uint32))


@pytest.mark.parametrize("B,I", [(2100, 600), (40, 400), (2049, 400), (60, 1500), (600, 1500)])
def test_row_sorts_on_either_side_of_their_shape_switches(B, I):
    """Rows of 257..512, 513..1024 and 1025..2048 inputs are sorted by several wavefronts per row
    while the batch is small (for 513..1024 always) and by one or four beyond; both sides of every
    switch, with ties and rows that carry inputs above MAX_SPIKE_TIME - 0.1, bit for bit against the oracle."""
    import snntc_amd as snn
    rng = np.random.default_rng(B + I)
    J = 3
    x = (1.0 + rng.integers(0, 60, (B, I)) / 16.0).astype(np.float32)
    x[3, rng.integers(0, I, 11)] = 2e5
    x[B - 1, :] = 3e5
    w = (rng.standard_normal((I + 1, J)) * 0.1 + 4.0 / I).astype(np.float32)
    p = capi.fc_params(1.0)
    ref_out, ref_k, ref_sorted, ref_perm = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, sz, perm, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    torch.cuda.synchronize()
    assert np.array_equal(perm.cpu().numpy(), ref_perm), "permutation differs"
    assert np.array_equal(sz.cpu().numpy(), ref_sorted)
    assert np.array_equal(ck.cpu().numpy(), ref_k)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref_out.view(np.uint32))


def test_layer_autograd_matches_op_level_chain():
    """SNN_dense / SNN_conv hand the [B,...] upstream gradient to the backward op directly; the result
    must equal slicing the full op output under autograd (zero-extended gradient), bit for bit."""
    import snntc_amd as snn
    x, w, p, g = dense_case(11, 24, 120, 50, True, "baseline")
    B = x.shape[0]
    layer = snn.SNN_dense(x.shape[1], w.shape[1], weight=w.copy()).to(DEV)
    X1 = t(x).requires_grad_(True)
    y1 = layer(X1)
    (y1 * t(g[:B])).sum().backward()
    X2 = t(x).requires_grad_(True)
    W2 = t(w).requires_grad_(True)
    y2 = snn.SnnFc.apply(X2, W2, layer.Params)[:B]
    (y2 * t(g[:B])).sum().backward()
    assert torch.equal(y1, y2)
    assert torch.equal(X1.grad, X2.grad) and torch.equal(layer.weight.grad, W2.grad)

    xraw, xpad, w, p, g = conv_case(12, 2, 9, 9, 32, 16, 3, 3, 1, 1, True, True, "baseline")
    B = xraw.shape[0]
    conv = snn.SNN_conv(32, 16, 3, 1, 'SAME', weight=w.copy()).to(DEV)
    X1 = t(xraw).requires_grad_(True)
    y1 = conv(X1)
    (y1 * t(g[:B])).sum().backward()
    X2 = t(xpad).requires_grad_(True)
    W2 = t(w).requires_grad_(True)
    y2 = snn.SnnCv.apply(X2, W2, conv.Params)[:B]
    (y2 * t(g[:B])).sum().backward()
    assert torch.equal(y1, y2)
    assert torch.equal(conv.weight.grad, W2.grad)
    # dX of the layer is the padded gradient cropped back to the unpadded image
    assert torch.equal(X1.grad, X2.grad[:, 1:-1, 1:-1, :])


@pytest.mark.parametrize("B,J", [(256, 10), (1, 1), (33, 1000), (7, 65)])
def test_loss_kernel_against_closed_form(B, J):
    """Fused loss kernel: per-sample loss and gradient within 1e-6 (relative to max(1, |value|)) of the
    float64 closed form; unfired outputs (time = 1e5) take no probability and no gradient."""
    import snntc_amd as snn
    from oracle.closed_form import softmax_time_loss
    rng = np.random.default_rng(B + J)
    times = (1.0 + 4.0 * rng.random((B, J))).astype(np.float32)
    if J > 2:
        times[:, -1] = 1e5                                   # a neuron that never fired
    label = np.eye(J, dtype=np.float32)[rng.integers(0, max(J - 1, 1), B)]
    want_s, want_g = softmax_time_loss(times, label)
    got_s, got_g = snn.softmax_time_loss(t(times), t(label))
    assert np.all(np.abs(got_s.cpu().numpy() - want_s) <= 1e-6 * np.maximum(1.0, np.abs(want_s)))
    assert np.all(np.abs(got_g.cpu().numpy() - want_g) <= 1e-6 / B + 1e-6 * np.abs(want_g))
    if J > 2:
        assert np.all(got_g.cpu().numpy()[:, -1] == 0.0)
    # through loss_func and autograd: same mean and gradient, scaled by the upstream factor
    T = t(times).requires_grad_(True)
    (3.0 * snn.loss_func(T, t(label))).backward()
    assert abs(float(snn.loss_func(T.detach(), t(label))) - want_s.mean()) <= 1e-6 * max(1.0, want_s.mean())
    assert np.all(np.abs(T.grad.cpu().numpy() - 3.0 * want_g) <= 3e-6 / B + 3e-6 * np.abs(want_g))


HEAD_CASES = [
    # seed, B, I, J, bias: classifier heads, i.e. fewer (sample group, column slice) work items than CUs
    (20, 70, 800, 10, True),       # batch not a multiple of the segments a wavefront holds
    (21, 9, 512, 10, False),
    (22, 33, 2048, 5, True),
    (23, 130, 264, 16, True),      # J equal to the slice width (vector weight copy)
    (24, 6, 72, 3, True),
    (25, 40, 300, 5, True),        # 8-column slice: four samples per work item
    (26, 50, 200, 24, False),      # 32-column slice
    (27, 20, 136, 40, True),       # 64-column slice, rows barely long enough to be shared
    (28, 100, 264, 70, True),      # two column slices, the second mostly empty
]


@pytest.mark.parametrize("seed,B,I,J,bias", HEAD_CASES)
def test_dense_head_forward_bit_exact(seed, B, I, J, bias):
    """Layers with a handful of outputs, where the wavefronts of a workgroup share one scan.  Rows
    differ in their number of real inputs (some inputs lie above MAX-0.1, a few rows have none at
    all), weights of both signs make neurons fire and stop firing again, and some neurons never fire:
    y, 1/S and the causal-set sizes must equal the oracle bit for bit, with and without the extra outputs."""
    import snntc_amd as snn
    rng = np.random.default_rng(seed)
    x = np.exp(2.0 * rng.random((B, I))).astype(np.float32)
    late = rng.random((B, I)) < rng.random((B, 1)) * 0.5          # per-row share of never-arriving inputs
    x[late] = np.float32(1e5)
    x[0] = np.float32(1e5)                                         # a row without any real input
    rows = I + (1 if bias else 0)
    w = ((3.0 / I) + rng.standard_normal((rows, J)) * np.sqrt(2.0 / I)).astype(np.float32)
    w[:, 0] = -np.abs(w[:, 0])                                     # a neuron that can never fire
    p = capi.fc_params(1.0 if bias else 0.0)
    ref_out, ref_k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
    out, _, _, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
    out2 = snn.snnfc(t(x), t(w), p)
    torch.cuda.synchronize()
    out, ck, out2 = out.cpu().numpy(), ck.cpu().numpy(), out2.cpu().numpy()
    assert np.array_equal(ck, ref_k), f"causal-set sizes differ at {np.argwhere(ck != ref_k)[:5]}"
    assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y / 1/S not bit-exact"
    assert np.array_equal(out2.view(np.uint32), ref_out.view(np.uint32)), "plain entry point not bit-exact"
    assert np.all(ref_k[:, 0] == -1) and (ref_k >= 0).any(), "the case should hold firing and silent neurons"


def test_head_scan_bounded_wait_gives_up_visibly():
    """The classifier-head scan hands running sums from one wavefront to the others behind a bounded
    wait.  With the poll limit at zero (a host-side test hook; every kernel still runs to its end) a
    waiting wavefront gives up on its first poll unless the sums are already there: the call still
    returns SNNTC_OK, every output is either the oracle's bits or NaN in BOTH halves of `out`, the
    status word counts the wavefronts that gave up, and check_scan_health() raises.  With the limit
    restored the same call is bit-exact again and the count stays where it was."""
    import snntc_amd as snn
    from snntc_amd import _lib
    rng = np.random.default_rng(5)
    B, I, J = 32, 800, 10                                          # 16 work items of one workgroup each
    x = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
    w = ((4.0 / I) + rng.standard_normal((I + 1, J)) * np.sqrt(1.0 / I)).astype(np.float32)
    p = capi.fc_params(1.0)
    ref = capi.fc_forward_dev(x, w, p)
    xt, wt = t(x), t(w)
    snn.check_scan_health(DEV)                                     # settles the count seen so far
    before = _lib.scan_giveups()
    _lib.set_scan_wait_polls(0)
    try:
        out = snn.snnfc(xt, wt, p)                                 # no exception: status SNNTC_OK
        torch.cuda.synchronize()
    finally:
        _lib.set_scan_wait_polls(-1)
    out = out.cpu().numpy()
    gave_up = _lib.scan_giveups() - before
    y, r = out[:B], out[B:]
    poisoned = np.isnan(y)
    assert np.array_equal(poisoned, np.isnan(r)), "a poisoned neuron must be NaN in both halves"
    good = ~poisoned
    assert np.array_equal(y[good].view(np.uint32), ref[:B][good].view(np.uint32))
    assert np.array_equal(r[good].view(np.uint32), ref[B:][good].view(np.uint32))
    # a lone wavefront needs microseconds for the first chunk's sums; the testers poll within nanoseconds
    assert poisoned.any() and gave_up > 0, "the give-up path did not run"
    with pytest.raises(snn.SnntcError, match="gave up"):
        snn.check_scan_health(DEV)
    out = snn.snnfc(xt, wt, p).cpu().numpy()
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32)), "default wait: not bit-exact"
    assert snn.check_scan_health(DEV) == before + gave_up


def test_sgd_update_matches_numpy():
    """w -= lr*dw over tensors of awkward sizes (empty, shorter than a vector, unaligned views, more
    than one table of 32): within one rounding of the float32 formula, and nothing else is touched."""
    import snntc_amd as snn
    rng = np.random.default_rng(5)
    sizes = [(785, 800), (801, 10), (0, 7), (1,), (3,), (5, 1023)] + [(int(n),) for n in rng.integers(1, 5000, 34)]
    ws = [rng.standard_normal(sz).astype(np.float32) for sz in sizes]
    gs = [rng.standard_normal(sz).astype(np.float32) for sz in sizes]
    lr = 0.0123
    dev_w = [t(w) for w in ws]
    # one weight is a view that starts 4 bytes into its buffer: the vector path must not be taken for it
    backing = torch.zeros(ws[5].size + 1, device=DEV)
    backing[1:] = t(ws[5]).reshape(-1)
    dev_w[5] = backing[1:].view(sizes[5])
    snn.sgd_update(dev_w, [t(g) for g in gs], lr)
    for w, g, got in zip(ws, gs, dev_w):
        want = w.astype(np.float64) - lr * g.astype(np.float64)
        err = np.abs(got.cpu().numpy() - want)
        assert np.all(err <= 1.2e-7 * np.maximum(np.abs(want), np.abs(w)) + 1e-30)
    assert float(backing[0]) == 0.0
    with pytest.raises(ValueError):
        snn.sgd_update(dev_w[:2], [t(gs[0])], lr)
    with pytest.raises(ValueError):
        snn.sgd_update(dev_w[:1], [t(gs[1])], lr)


PARAM_SWEEP = [
    # biasvolt, theta, max_time
    (0.7, 1.0, 1e5),
    (2.5, 0.5, 1e5),
    (1.0, 2.0, 50.0),        # small MAX: inputs above MAX-0.1 are treated as never-fired
    (0.0, 1.5, 20.0),
]


def _compare_forward_backward(fwd_ref, bwd_ref, fwd_gpu, bwd_gpu, g, B):
    ref_out, ref_k, ref_sorted, ref_perm = fwd_ref()
    out, sz, perm, ck = (v.cpu().numpy() for v in fwd_gpu())
    assert np.array_equal(sz, ref_sorted) and np.array_equal(perm, ref_perm)
    assert np.array_equal(ck, ref_k), f"causal-set sizes differ at {np.argwhere(ck != ref_k)[:5]}"
    assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y / 1/S not bit-exact"
    dx, dw, _ = (v.cpu().numpy() for v in bwd_gpu(ref_out))
    rdx, rdw, adx, adw = bwd_ref(ref_out)
    check_grad(dx, rdx, adx, "dX")
    check_grad(dw, rdw, adw, "dW")


@pytest.mark.parametrize("biasvolt,theta,max_time", PARAM_SWEEP)
def test_dense_non_default_parameters_and_sentinel_inputs(biasvolt, theta, max_time):
    """biasvolt, threshold and MAX other than the defaults; some inputs are the MAX sentinel (an upstream
    neuron that never fired), one row consists of sentinels only, one weight column is all negative."""
    import snntc_amd as snn
    rng = np.random.default_rng(int(10 * biasvolt + 100 * theta))
    B, I, J = 37, 150, 45
    rows = I + (1 if biasvolt > 1e-8 else 0)
    x = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
    x[rng.random((B, I)) < 0.15] = np.float32(max_time)
    x[5, :] = np.float32(max_time)
    x[6, : I // 2] = np.float32(max_time - 0.05)            # above MAX - 0.1: still "never fired"
    w = (4.0 / I + np.sqrt(1.0 / I) * rng.standard_normal((rows, J))).astype(np.float32) * np.float32(theta)
    w[:, 3] = -np.abs(w[:, 3])
    p = capi.fc_params(biasvolt, max_time=max_time, theta=theta)
    g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))

    def bwd_ref(out):
        rdx, rdw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
        ao = out.copy(); ao[B:] = np.abs(ao[B:])
        adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, ao, wide=True)
        return rdx, rdw, adx, adw

    _compare_forward_backward(lambda: capi.fc_forward_dev(x, w, p, want_aux=True), bwd_ref,
                              lambda: snn.snnfc(t(x), t(w), p, return_aux=True),
                              lambda out: snn.snnfc_grad(t(g), t(x), t(w), p, t(out)), g, B)


@pytest.mark.parametrize("max_time", [1.0, 12.0, 1e5, 3e6])
@pytest.mark.parametrize("J", [9, 70])
def test_dense_weight_gradient_over_the_whole_range_of_time_differences(max_time, J):
    """The dW kernels evaluate min(x - y, 0) through a scaled, clamped difference that is exact while
    y - x stays below 2 * MAX.  Inputs here run from -0.9 * MAX up to the sentinel, outputs up to
    MAX - 0.1, so the differences cover (almost) that whole range, for MAX below, at and far above
    the default, and for both dW kernels (narrow head and general)."""
    import snntc_amd as snn
    rng = np.random.default_rng(int(max_time) % 1000 + J)
    B, I = 70, 40
    x = ((rng.random((B, I)) * 1.85 - 0.9) * max_time).astype(np.float32)
    x[rng.random((B, I)) < 0.1] = np.float32(max_time)
    w = rng.standard_normal((I + 1, J)).astype(np.float32)
    p = capi.fc_params(1.0, max_time=max_time)
    # a forward output written by hand: spike times anywhere in [0, MAX - 0.1], a few never-fired
    out = np.zeros((2 * B, J), np.float32)
    out[:B] = (rng.random((B, J)) * (np.float32(max_time) - np.float32(0.1))).astype(np.float32)
    out[B:] = rng.standard_normal((B, J)).astype(np.float32)
    dead = rng.random((B, J)) < 0.1
    out[:B][dead] = np.float32(max_time); out[B:][dead] = 0.0
    g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))
    dx, dw, _ = snn.snnfc_grad(t(g), t(x), t(w), p, t(out))
    torch.cuda.synchronize()
    rdx, rdw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    ao = out.copy(); ao[B:] = np.abs(ao[B:])
    adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, ao, wide=True)
    check_grad(dx.cpu().numpy(), rdx, adx, "dX")
    check_grad(dw.cpu().numpy(), rdw, adw, "dW")
    assert np.isfinite(dw.cpu().numpy()).all()


@pytest.mark.parametrize("biasvolt,theta,max_time", PARAM_SWEEP)
@pytest.mark.parametrize("C,Kc", [(32, 32), (64, 16), (5, 9)])
def test_conv_non_default_parameters_and_sentinel_inputs(biasvolt, theta, max_time, C, Kc):
    import snntc_amd as snn
    from oracle.closed_form import same_pad
    rng = np.random.default_rng(int(10 * biasvolt + 100 * theta) + C)
    B, H, W, K = 2, 11, 10, 3
    P = K * K * C
    rows = P + (1 if biasvolt > 1e-8 else 0)
    x = np.exp(rng.random((B, H, W, C))).astype(np.float32)
    x[rng.random((B, H, W, C)) < 0.1] = np.float32(max_time)          # unfired upstream neurons
    x[0, 4:7, 3:6, :] = np.float32(max_time)                          # a whole patch of them
    (tp, bt), (lf, rt) = same_pad(H, K, 1), same_pad(W, K, 1)
    xpad = np.pad(x, ((0, 0), (tp, bt), (lf, rt), (0, 0)), constant_values=np.float32(max_time))
    w = (4.0 / P + np.sqrt(1.0 / P) * rng.standard_normal((rows, Kc))).astype(np.float32) * np.float32(theta)
    p = capi.cv_params(K, K, 1, 1, same=True, biasvolt=biasvolt, max_time=max_time, theta=theta)
    Nh, Nw, _ = capi.cv_dims(xpad.shape, p)
    g = np.zeros((2 * B, Nh, Nw, Kc), np.float32); g[:B] = rng.standard_normal((B, Nh, Nw, Kc))

    def bwd_ref(out):
        rdx, rdw, _ = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
        ao = out.copy(); ao[B:] = np.abs(ao[B:])
        adx, adw, _ = capi.cv_backward_dev(np.abs(g), xpad, np.abs(w), p, ao, wide=True)
        return rdx, rdw, adx, adw

    _compare_forward_backward(lambda: capi.cv_forward_dev(xpad, w, p, want_aux=True), bwd_ref,
                              lambda: snn.snncv(t(xpad), t(w), p, return_aux=True),
                              lambda out: snn.snncv_grad(t(g), t(xpad), t(w), p, t(out)), g, B)


@pytest.mark.parametrize("max_time", [2.0, 1e5, 3e6])
@pytest.mark.parametrize("C,Kc", [(32, 64), (8, 48), (32, 16)])
def test_conv_weight_gradient_over_the_whole_range_of_time_differences(max_time, C, Kc):
    """As the dense test of the same name, for the conv dW kernels (wide: Kc > 32, narrow: Kc <= 32)
    and the generic one (C = 8): pixel times from -0.9 * MAX up to the sentinel, spike times written
    by hand anywhere in [0, MAX - 0.1]."""
    import snntc_amd as snn
    rng = np.random.default_rng(int(max_time) % 1000 + C + Kc)
    B, H, W, K = 2, 9, 10, 3
    P = K * K * C
    xpad = ((rng.random((B, H + 2, W + 2, C)) * 1.85 - 0.9) * max_time).astype(np.float32)
    xpad[rng.random(xpad.shape) < 0.1] = np.float32(max_time)
    w = rng.standard_normal((P + 1, Kc)).astype(np.float32)
    p = capi.cv_params(K, K, 1, 1, same=True, biasvolt=1.0, max_time=max_time)
    Nh, Nw, _ = capi.cv_dims(xpad.shape, p)
    out = np.zeros((2 * B, Nh, Nw, Kc), np.float32)
    out[:B] = (rng.random((B, Nh, Nw, Kc)) * (np.float32(max_time) - np.float32(0.1))).astype(np.float32)
    out[B:] = rng.standard_normal((B, Nh, Nw, Kc)).astype(np.float32)
    dead = rng.random((B, Nh, Nw, Kc)) < 0.1
    out[:B][dead] = np.float32(max_time); out[B:][dead] = 0.0
    g = np.zeros((2 * B, Nh, Nw, Kc), np.float32); g[:B] = rng.standard_normal((B, Nh, Nw, Kc))
    dx, dw, _ = snn.snncv_grad(t(g), t(xpad), t(w), p, t(out))
    torch.cuda.synchronize()
    rdx, rdw, _ = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
    ao = out.copy(); ao[B:] = np.abs(ao[B:])
    adx, adw, _ = capi.cv_backward_dev(np.abs(g), xpad, np.abs(w), p, ao, wide=True)
    check_grad(dx.cpu().numpy(), rdx, adx, "dX")
    check_grad(dw.cpu().numpy(), rdw, adw, "dW")
    assert np.isfinite(dw.cpu().numpy()).all()


@pytest.mark.parametrize("C,Kc,K", [(32, 64, 3), (64, 32, 3), (32, 16, 5)])
def test_conv_input_gradient_mask_at_its_edges(C, Kc, K):
    """The channel dX kernels evaluate the mask x <= y arithmetically, as clamp01((x - y) * 2^109) (for
    MAX_SPIKE_TIME = 1e5).  Pixel and spike times from a handful of values, so that most pairs are exact ties
    (mask true), neighbouring floats (1 and the float above it), zeros on both sides, and values a few powers of two above
    the smallest difference the scale resolves: one wrong decision moves dX by a whole term, far outside the
    band.  K = 3 takes the slot-major sweep, K = 5 the tap-major one."""
    import snntc_amd as snn
    max_time = 1e5
    rng = np.random.default_rng(C + Kc + K)
    one_up = np.nextafter(np.float32(1), np.float32(2))
    values = np.array([0.0, 2.0 ** -100, 2.0 ** -60, 1.0, one_up, 1.5, 7.0, 99999.0], np.float32)
    B, H, W = 2, 9, 12
    pad = K // 2
    xpad = values[rng.integers(0, len(values), (B, H + 2 * pad, W + 2 * pad, C))]
    xpad[rng.random(xpad.shape) < 0.05] = np.float32(max_time)
    P = K * K * C
    w = rng.standard_normal((P + 1, Kc)).astype(np.float32)
    p = capi.cv_params(K, K, 1, 1, same=True, biasvolt=1.0, max_time=max_time)
    Nh, Nw, _ = capi.cv_dims(xpad.shape, p)
    out = np.zeros((2 * B, Nh, Nw, Kc), np.float32)
    out[:B] = values[rng.integers(0, len(values), (B, Nh, Nw, Kc))]
    out[B:] = rng.standard_normal((B, Nh, Nw, Kc)).astype(np.float32)
    dead = rng.random((B, Nh, Nw, Kc)) < 0.1
    out[:B][dead] = np.float32(max_time); out[B:][dead] = 0.0
    g = np.zeros((2 * B, Nh, Nw, Kc), np.float32); g[:B] = rng.standard_normal((B, Nh, Nw, Kc))
    dx, dw, _ = snn.snncv_grad(t(g), t(xpad), t(w), p, t(out))
    torch.cuda.synchronize()
    rdx, rdw, _ = capi.cv_backward_dev(g, xpad, w, p, out, wide=True)
    ao = out.copy(); ao[B:] = np.abs(ao[B:])
    adx, adw, _ = capi.cv_backward_dev(np.abs(g), xpad, np.abs(w), p, ao, wide=True)
    check_grad(dx.cpu().numpy(), rdx, adx, "dX")
    check_grad(dw.cpu().numpy(), rdw, adw, "dW")


@pytest.mark.parametrize("J", [9, 70])
def test_dense_weight_gradient_at_the_edge_of_its_input_domain(J):
    """The dW kernels are exact for inputs down to -MAX_SPIKE_TIME (they scale y - x by the power of two
    above 2 * MAX and clamp at 1).  Inputs exactly at -MAX, just above it, and outputs up to MAX - 0.1:
    the largest differences the domain allows, against the float64 oracle."""
    import snntc_amd as snn
    max_time = 1e5
    rng = np.random.default_rng(J)
    B, I = 48, 24
    x = np.full((B, I), -max_time, np.float32)
    x[:, 1::3] = np.nextafter(np.float32(-max_time), np.float32(0))
    x[:, 2::3] = (rng.random((B, len(range(2, I, 3)))) * 10).astype(np.float32)
    w = rng.standard_normal((I + 1, J)).astype(np.float32)
    p = capi.fc_params(1.0, max_time=max_time)
    out = np.zeros((2 * B, J), np.float32)
    out[:B] = np.float32(max_time) - np.float32(0.1) - (rng.random((B, J)) * 3).astype(np.float32)
    out[:B, 0] = np.float32(max_time) - np.float32(0.1)              # the largest output that still counts
    out[B:] = rng.standard_normal((B, J)).astype(np.float32)
    g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))
    dx, dw, _ = snn.snnfc_grad(t(g), t(x), t(w), p, t(out))
    torch.cuda.synchronize()
    rdx, rdw, _ = capi.fc_backward_dev(g, x, w, p, out, wide=True)
    ao = out.copy(); ao[B:] = np.abs(ao[B:])
    adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, ao, wide=True)
    check_grad(dx.cpu().numpy(), rdx, adx, "dX")
    check_grad(dw.cpu().numpy(), rdw, adw, "dW")


def test_empty_batch_and_single_elements():
    """B = 0 yields empty outputs and an all-zero weight gradient; 1x1x1 shapes work."""
    import snntc_amd as snn
    p = capi.fc_params(1.0)
    w = np.ones((6, 4), np.float32)
    y = snn.snnfc(torch.empty((0, 5), device=DEV), t(w), p)
    assert tuple(y.shape) == (0, 4)
    dx, dw, dp = snn.snnfc_grad(torch.empty((0, 4), device=DEV), torch.empty((0, 5), device=DEV), t(w), p, y)
    assert tuple(dx.shape) == (0, 5) and torch.all(dw == 0) and torch.all(dp == 0)
    pc = capi.cv_params(3, 3, 1, 1, same=True, biasvolt=1.0)
    wc = np.ones((9 * 2 + 1, 3), np.float32)
    yc = snn.snncv(torch.empty((0, 6, 6, 2), device=DEV), t(wc), pc)
    assert tuple(yc.shape) == (0, 4, 4, 3)
    dxc, dwc, _ = snn.snncv_grad(torch.empty((0, 4, 4, 3), device=DEV), torch.empty((0, 6, 6, 2), device=DEV), t(wc), pc, yc)
    assert tuple(dxc.shape) == (0, 6, 6, 2) and torch.all(dwc == 0)
    # one sample, one input, one output, no bias: y = w z / (w - 1) for w > 1
    x1 = np.array([[2.0]], np.float32); w1 = np.array([[3.0]], np.float32)
    y1 = snn.snnfc(t(x1), t(w1), capi.fc_params(0.0)).cpu().numpy()
    assert y1[0, 0] == np.float32(3.0) and y1[1, 0] == np.float32(0.5)
    ref = capi.fc_forward_dev(x1, w1, capi.fc_params(0.0))
    assert np.array_equal(y1, ref[0] if isinstance(ref, tuple) else ref)
