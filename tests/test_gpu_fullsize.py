"""Parity at the BASELINE configurations' full sizes, where the oracle is too slow to run whole:
size-independent properties on the complete GPU result plus exact oracle comparison on a slice that
is independent of the rest (single images / samples)."""
import numpy as np
import pytest
import torch

from helpers import conv_case, dense_case, grad_band
from oracle import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def check_forward_properties(x_seg, w, out, sz, perm, ck, bias, max_time=1e5):
    """x_seg[S,I] (device) are the segments; all arguments torch tensors on the GPU."""
    S, I = x_seg.shape
    J = w.shape[1]
    # sorted ascending, perm is a permutation that reproduces the sort, ties in index order
    assert torch.all(sz[:, 1:] >= sz[:, :-1])
    assert torch.equal(torch.gather(x_seg, 1, perm.long()), sz)
    assert torch.equal(torch.sort(perm, dim=1).values, torch.arange(I, device=DEV, dtype=perm.dtype).expand(S, I))
    tie = sz[:, 1:] == sz[:, :-1]
    assert torch.all(perm[:, 1:][tie] > perm[:, :-1][tie])
    y, r = out[:S].reshape(S, J), out[S:].reshape(S, J)
    fired = ck >= 0
    assert torch.all(y[~fired] == max_time) and torch.all(r[~fired] == 0)
    assert torch.all(r[fired] != 0) and torch.all(y[fired] < max_time)
    # the spike lies after the last causal input and not after the next one (1 ulp of slack for
    # y = ysum * (1/wsum) versus the division-free test the kernel decides with)
    k = ck.clamp(min=0).long()
    last = torch.where(k > 0, torch.gather(sz, 1, (k - 1).clamp(min=0)), torch.ones_like(y) if bias else torch.zeros_like(y))
    nxt = torch.where(k < I, torch.gather(sz, 1, k.clamp(max=I - 1)), torch.full_like(y, max_time))
    slack = 4e-7 * y.abs()
    assert torch.all((y + slack >= last)[fired])
    assert torch.all((y - slack <= nxt)[fired])


def test_dense_north_star_layer_full_batch():
    """B=256, 784 -> 800 with bias (BASELINE config 2, layer 1)."""
    import snntc_amd as snn
    x, w, p, g = dense_case(10, 256, 784, 800, True, "baseline")
    X, W, G = t(x), t(w), t(g)
    out, sz, perm, ck = snn.snnfc(X, W, p, return_aux=True)
    check_forward_properties(X, W, out, sz, perm, ck, True)
    # samples are independent: the first 8 and the last 8 must equal the oracle exactly
    for sl in (slice(0, 8), slice(248, 256)):
        ref, rk, _, rperm = capi.fc_forward_dev(x[sl], w, p, want_aux=True)
        n = sl.stop - sl.start
        got = torch.cat((out[sl], out[256 + sl.start:256 + sl.stop])).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
        assert np.array_equal(ck[sl].cpu().numpy(), rk) and np.array_equal(perm[sl].cpu().numpy(), rperm)
    # backward: linear in the upstream gradient, dX independent per sample, dW additive over samples
    dx, dw, _ = snn.snnfc_grad(G, X, W, p, out)
    dx2, dw2, _ = snn.snnfc_grad(2 * G, X, W, p, out)
    assert torch.equal(dx2, 2 * dx) and torch.equal(dw2, 2 * dw)           # scaling by 2 is exact in fp32
    half = 128
    oa = torch.cat((out[:half], out[256:256 + half])); ob = torch.cat((out[half:256], out[256 + half:]))
    ga = torch.cat((G[:half], G[256:256 + half])); gb = torch.cat((G[half:256], G[256 + half:]))
    dxa, dwa, _ = snn.snnfc_grad(ga, X[:half], W, p, oa)
    dxb, dwb, _ = snn.snnfc_grad(gb, X[half:], W, p, ob)
    assert torch.equal(torch.cat((dxa, dxb)), dx)
    # two summation orders of the same fp32 terms: compare on the scale of the summed magnitudes
    oabs = out.clone(); oabs[256:] = oabs[256:].abs()
    _, dw_mag, _ = snn.snnfc_grad(G.abs(), X, W, p, oabs)               # = -sum |x - y| |up|
    assert torch.all((dwa + dwb - dw).abs() <= 1e-5 * dw.abs() + 1e-6 * dw_mag.abs().clamp(min=1.0))
    g8 = np.concatenate((g[:8], g[256:264]))
    o8 = np.concatenate((out[:8].cpu().numpy(), out[256:264].cpu().numpy()))
    rdx, _, _ = capi.fc_backward_dev(g8, x[:8], w, p, o8, wide=True)
    o8a = o8.copy(); o8a[8:] = np.abs(o8a[8:])
    adx, _, _ = capi.fc_backward_dev(np.abs(g8), x[:8], np.abs(w), p, o8a, wide=True)     # sums of |summands|
    assert np.all(np.abs(dx[:8].cpu().numpy() - rdx) <= grad_band(rdx, adx))


def test_conv_north_star_layer_full_batch():
    """B=64, 32x32x64 -> 64, 3x3 SAME with bias (BASELINE config 3): 65 536 patches of 576."""
    import snntc_amd as snn
    B = 64
    _, xpad, w, p, g = conv_case(11, B, 32, 32, 64, 64, 3, 3, 1, 1, True, True, "baseline")
    X, W, G = t(xpad), t(w), t(g)
    out, sz, perm, ck = snn.snncv(X, W, p, return_aux=True)
    # patches as the op sees them (built with torch.unfold on the device, independent of the kernels)
    patches = X.unfold(1, 3, 1).unfold(2, 3, 1)                       # [B,Nh,Nw,C,kh,kw]
    patches = patches.permute(0, 1, 2, 4, 5, 3).reshape(B * 32 * 32, 576)
    check_forward_properties(patches, W, out.reshape(2 * B * 1024, 64), sz, perm, ck, True)
    # images are independent: first and last image against the oracle, exactly
    for b in (0, B - 1):
        ref, rk, _, rperm = capi.cv_forward_dev(xpad[b:b + 1], w, p, want_aux=True)
        got = torch.stack((out[b], out[B + b])).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
        assert np.array_equal(ck[b * 1024:(b + 1) * 1024].cpu().numpy(), rk)
        assert np.array_equal(perm[b * 1024:(b + 1) * 1024].cpu().numpy(), rperm)
    dx, dw, _ = snn.snncv_grad(G, X, W, p, out)
    dx2, dw2, _ = snn.snncv_grad(2 * G, X, W, p, out)
    assert torch.equal(dx2, 2 * dx) and torch.equal(dw2, 2 * dw)
    assert torch.all(dx[X > 99999.0] == 0)                             # padding receives no gradient
    # one image: dX exact slice of the batch result, and against the oracle
    o1 = torch.stack((out[0], out[B])); g1 = torch.stack((G[0], G[B]))
    dx1, dw1, _ = snn.snncv_grad(g1, X[:1], W, p, o1)
    assert torch.equal(dx1[0], dx[0])
    rdx, rdw, _ = capi.cv_backward_dev(g1.cpu().numpy(), xpad[:1], w, p, o1.cpu().numpy(), wide=True)
    o1a = o1.cpu().numpy().copy(); o1a[1] = np.abs(o1a[1])
    adx, adw, _ = capi.cv_backward_dev(np.abs(g1.cpu().numpy()), xpad[:1], np.abs(w), p, o1a, wide=True)
    assert np.all(np.abs(dx1.cpu().numpy() - rdx) <= grad_band(rdx, adx))
    assert np.all(np.abs(dw1.cpu().numpy() - rdw) <= grad_band(rdw, adw))
    # dW of the batch = sum of per-image dW (computed by the same kernels on single images)
    acc = torch.zeros_like(dw, dtype=torch.float64)
    for b in range(0, B, 8):
        ob = torch.cat((out[b:b + 8], out[B + b:B + b + 8])); gb = torch.cat((G[b:b + 8], G[B + b:B + b + 8]))
        _, dwb, _ = snn.snncv_grad(gb, X[b:b + 8], W, p, ob)
        acc += dwb.double()
    oabs = out.clone(); oabs[B:] = oabs[B:].abs()
    _, dw_mag, _ = snn.snncv_grad(G.abs(), X, W, p, oabs)               # = -sum |x - y| |up|
    assert torch.all((acc - dw.double()).abs() <= 1e-5 * acc.abs() + 1e-6 * dw_mag.abs().double().clamp(min=1.0))


# Layers of BASELINE configs 4 (CIFAR-10 net, B=128) and 5 (ResNet-18-shaped net, B=32) at full size.
LAYER_SHAPES = [
    # name,                    B,   H,   W,   C,  Kc, K, S
    ("cifar conv 3->32 @32",   128, 32,  32,  3,   32,  3, 1),
    ("cifar conv 32->32 @32",  128, 32,  32,  32,  32,  3, 1),
    ("cifar conv 32->64 @16",  128, 16,  16,  32,  64,  3, 1),
    ("cifar conv 64->64 @16",  128, 16,  16,  64,  64,  3, 1),
    ("cifar conv 64->128 @8",  128, 8,   8,   64,  128, 3, 1),
    ("resnet stem 7x7/2",      32,  224, 224, 3,   64,  7, 2),
    ("resnet 64->64 @56",      32,  56,  56,  64,  64,  3, 1),
    ("resnet 64->128 @28",     32,  28,  28,  64,  128, 3, 1),
    ("resnet 128->128 @28",    32,  28,  28,  128, 128, 3, 1),
    ("resnet 128->256 @14",    32,  14,  14,  128, 256, 3, 1),
    ("resnet 256->256 @14",    32,  14,  14,  256, 256, 3, 1),
    ("resnet 256->512 @7",     32,  7,   7,   256, 512, 3, 1),
    ("resnet 512->512 @7",     32,  7,   7,   512, 512, 3, 1),
]


@pytest.mark.parametrize("name,B,H,W,C,Kc,K,S", LAYER_SHAPES, ids=[s[0] for s in LAYER_SHAPES])
def test_conv_layer_shapes_of_the_baseline_networks(name, B, H, W, C, Kc, K, S):
    import snntc_amd as snn
    _, xpad, w, p, g = conv_case(20 + C + K, B, H, W, C, Kc, K, K, S, S, True, True, "baseline")
    X, Wt, G = t(xpad), t(w), t(g)
    out, sz, perm, ck = snn.snncv(X, Wt, p, return_aux=True)
    Nh, Nw = out.shape[1], out.shape[2]
    n_img = Nh * Nw
    patches = X.unfold(1, K, S).unfold(2, K, S).permute(0, 1, 2, 4, 5, 3).reshape(B * n_img, K * K * C)
    check_forward_properties(patches, Wt, out.reshape(2 * B * n_img, Kc), sz, perm, ck, True)
    del patches
    for b in (0, B - 1):                                   # images are independent: exact against the oracle
        ref, rk, _, rperm = capi.cv_forward_dev(xpad[b:b + 1], w, p, want_aux=True)
        got = torch.stack((out[b], out[B + b])).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
        assert np.array_equal(ck[b * n_img:(b + 1) * n_img].cpu().numpy(), rk)
        assert np.array_equal(perm[b * n_img:(b + 1) * n_img].cpu().numpy(), rperm)
    del sz, perm, ck
    dx, dw, _ = snn.snncv_grad(G, X, Wt, p, out)
    dx2, dw2, _ = snn.snncv_grad(2 * G, X, Wt, p, out)
    assert torch.equal(dx2, 2 * dx) and torch.equal(dw2, 2 * dw)
    assert torch.all(dx[X > 99999.0] == 0)
    b = B - 1                                              # last image alone: same dX, oracle dX / dW
    o1 = torch.stack((out[b], out[B + b])); g1 = torch.stack((G[b], G[B + b]))
    dx1, dw1, _ = snn.snncv_grad(g1, X[b:b + 1], Wt, p, o1)
    assert torch.equal(dx1[0], dx[b])
    rdx, rdw, _ = capi.cv_backward_dev(g1.cpu().numpy(), xpad[b:b + 1], w, p, o1.cpu().numpy(), wide=True)
    o1a = o1.clone(); o1a[1] = o1a[1].abs()
    mdx, mdw, _ = snn.snncv_grad(g1.abs(), X[b:b + 1], Wt.abs(), p, o1a)      # sums of |summands|
    tol_dx = grad_band(rdx, mdx.cpu().numpy())
    tol_dw = grad_band(rdw, mdw.cpu().numpy())
    assert np.all(np.abs(dx1.cpu().numpy() - rdx) <= tol_dx)
    assert np.all(np.abs(dw1.cpu().numpy() - rdw) <= tol_dw)


def literal_bar_statistics(actual, ref):
    """Share of elements outside the literal bar |a - e| <= 1e-5 * |e| + 1e-6, and the worst ratio of
    the error to that bar."""
    a = np.asarray(actual, np.float64); e = np.asarray(ref, np.float64)
    ratio = np.abs(a - e) / (1e-5 * np.abs(e) + 1e-6)
    return float((ratio > 1.0).mean()), float(ratio.max())


LITERAL_BAR_CASES = [
    # name, kind, shape
    ("dense 784->800 B=128 (config 1)", "dense", (128, 784, 800)),
    ("conv 3x3 64->64 @32x32 B=16 (config 3 layer, a quarter of its batch)", "conv", (16, 32, 32, 64, 64)),
]


@pytest.mark.parametrize("name,kind,shape", LITERAL_BAR_CASES, ids=["config1", "config3"])
def test_gradients_against_the_literal_tolerance(name, kind, shape):
    """How the gradients stand against the literal bar rel 1e-5 / abs 1e-6 (no scaling by the size of the
    sums), with the float64-accumulated oracle as the reference value: for the HIP result and for the
    oracle run in the reference kernels' own fp32 sequential order.  Long fp32 sums cannot all meet the
    literal bar in any order; the HIP result must not be worse than the reference's order on either count
    (share of elements outside up to a factor of 1.5 and a floor of one element in a thousand, worst
    excess up to a factor of 2)."""
    import json
    import os
    import snntc_amd as snn
    if kind == "dense":
        B, I, J = shape
        x, w, p, g = dense_case(0, B, I, J, True, "baseline")
        out = capi.fc_forward_dev(x, w, p)
        wide = capi.fc_backward_dev(g, x, w, p, out, wide=True)
        seq = capi.fc_backward_dev(g, x, w, p, out)
        dx, dw, _ = snn.snnfc_grad(t(g), t(x), t(w), p, t(out))
    else:
        B, H, C, Kc = shape[0], shape[1], shape[3], shape[4]
        _, x, w, p, g = conv_case(0, B, H, H, C, Kc, 3, 3, 1, 1, True, True, "baseline")
        out = capi.cv_forward_dev(x, w, p)
        wide = capi.cv_backward_dev(g, x, w, p, out, wide=True)
        seq = capi.cv_backward_dev(g, x, w, p, out)
        dx, dw, _ = snn.snncv_grad(t(g), t(x), t(w), p, t(out))
    torch.cuda.synchronize()
    stats = {"case": name}
    for label, got, ref, ref_seq in (("dX", dx, wide[0], seq[0]), ("dW", dw, wide[1], seq[1])):
        share_hip, worst_hip = literal_bar_statistics(got.cpu().numpy(), ref)
        share_seq, worst_seq = literal_bar_statistics(ref_seq, ref)
        stats[label] = {"hip_share_outside": share_hip, "hip_worst_ratio": worst_hip,
                        "fp32_sequential_share_outside": share_seq, "fp32_sequential_worst_ratio": worst_seq,
                        "max_abs_ref": float(np.abs(ref).max())}
        assert share_hip <= max(1.5 * share_seq, 1e-3), (label, stats[label])
        assert worst_hip <= max(2.0 * worst_seq, 1.0), (label, stats[label])
    print(json.dumps(stats))
    stats_dir = os.environ.get("SNNTC_STATS_DIR")
    if stats_dir and os.path.isdir(stats_dir):
        with open(os.path.join(stats_dir, f"literal_bar_{kind}.json"), "w") as f:
            json.dump(stats, f, indent=1)
