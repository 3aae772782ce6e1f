"""Seeded random sweep: many small dense and conv problems with random shapes (ragged channel counts,
kernel sizes, strides, SAME / VALID), non-default biasvolt / threshold / MAX, quantised inputs (heavy
ties) and MAX sentinels among the inputs.  Same bars as test_gpu_parity: sorted values, permutations,
causal-set sizes, spike times and reciprocals bit-exact against the oracle; gradients within
1e-5 * |ref| + 1e-6 * max(1, half the sum of |summands|) (helpers.grad_band)."""
import numpy as np
import pytest
import torch

from oracle import capi
from oracle.closed_form import same_pad
from test_gpu_parity import check_grad, t

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed0", [11, 12, 13])
def test_random_shapes_and_parameters(seed0):
    import snntc_amd as snn
    n_cases, fails = 120, []
    for case in range(n_cases):
        rng = np.random.default_rng(seed0 * 100000 + case)
        kind = "dense" if rng.random() < 0.4 else "conv"
        biasvolt = float(rng.choice([0.0, 1.0, 1.0, 0.6, 2.0]))
        theta = float(rng.choice([1.0, 1.0, 0.5, 2.0]))
        max_time = float(rng.choice([1e5, 1e5, 30.0]))
        quant = rng.random() < 0.3          # heavy ties
        sent = rng.random() < 0.4           # sentinel inputs
        try:
            if kind == "dense":
                B = int(rng.integers(1, 70)); I = int(rng.choice([1, 2, 7, 31, 64, 65, 200, 511, 784, 1025, 2049, int(rng.integers(1, 3000))]))
                J = int(rng.choice([1, 3, 10, 16, 33, 64, 65, 130, int(rng.integers(1, 300))]))
                if B * I * J > 6e6: J = max(1, int(6e6 / (B * I)))
                rows = I + (1 if biasvolt > 1e-8 else 0)
                x = np.exp(1.0 - rng.random((B, I))).astype(np.float32)
                if quant: x = (np.round(x * 4) / 4).astype(np.float32)
                if sent: x[rng.random((B, I)) < 0.2] = np.float32(max_time)
                scale = rng.choice([1.0, 0.3, 3.0])
                w = ((4.0 / I + np.sqrt(1.0 / I) * rng.standard_normal((rows, J))) * theta * scale).astype(np.float32)
                if rng.random() < 0.3: w = rng.standard_normal((rows, J)).astype(np.float32)
                p = capi.fc_params(biasvolt, max_time=max_time, theta=theta)
                g = np.zeros((2 * B, J), np.float32); g[:B] = rng.standard_normal((B, J))
                desc = f"dense B={B} I={I} J={J}"
                ref_out, ref_k, ref_sorted, ref_perm = capi.fc_forward_dev(x, w, p, want_aux=True)
                out, sz, perm, ck = (v.cpu().numpy() for v in snn.snnfc(t(x), t(w), p, return_aux=True))
                dx, dw, _ = (v.cpu().numpy() for v in snn.snnfc_grad(t(g), t(x), t(w), p, t(ref_out)))
                rdx, rdw, _ = capi.fc_backward_dev(g, x, w, p, ref_out, wide=True)
                ao = ref_out.copy(); ao[B:] = np.abs(ao[B:])
                adx, adw, _ = capi.fc_backward_dev(np.abs(g), x, np.abs(w), p, ao, wide=True)
            else:
                B = int(rng.integers(1, 4)); H = int(rng.integers(3, 20)); W = int(rng.integers(3, 20))
                C = int(rng.choice([1, 2, 3, 4, 8, 16, 31, 32, 33, 48, 64, 96, 128]))
                Kc = int(rng.choice([1, 5, 16, 32, 48, 64, 80, 128]))
                Kh = int(rng.integers(1, min(H, 6) + 1)); Kw = int(rng.integers(1, min(W, 6) + 1))
                Sh = int(rng.integers(1, 4)); Sw = int(rng.integers(1, 4))
                same = bool(rng.random() < 0.6)
                if same and (Kh < Sh or Kw < Sw): same = False
                P = Kh * Kw * C
                rows = P + (1 if biasvolt > 1e-8 else 0)
                x = np.exp(rng.random((B, H, W, C))).astype(np.float32)
                if quant: x = (np.round(x * 4) / 4).astype(np.float32)
                if sent: x[rng.random((B, H, W, C)) < 0.15] = np.float32(max_time)
                if same:
                    (tp, bt), (lf, rt) = same_pad(H, Kh, Sh), same_pad(W, Kw, Sw)
                    if min(tp, bt, lf, rt) < 0: continue
                    xpad = np.pad(x, ((0, 0), (tp, bt), (lf, rt), (0, 0)), constant_values=np.float32(max_time))
                else:
                    nh, nw = (H - Kh) // Sh + 1, (W - Kw) // Sw + 1
                    xpad = np.ascontiguousarray(x[:, :(nh - 1) * Sh + Kh, :(nw - 1) * Sw + Kw, :])
                w = ((4.0 / P + np.sqrt(1.0 / P) * rng.standard_normal((rows, Kc))) * theta).astype(np.float32)
                p = capi.cv_params(Kh, Kw, Sh, Sw, same=same, biasvolt=biasvolt, max_time=max_time, theta=theta)
                Nh, Nw, _ = capi.cv_dims(xpad.shape, p)
                g = np.zeros((2 * B, Nh, Nw, Kc), np.float32); g[:B] = rng.standard_normal((B, Nh, Nw, Kc))
                desc = f"conv B={B} {H}x{W}x{C}->{Kc} k={Kh}x{Kw} s={Sh}x{Sw} same={same}"
                ref_out, ref_k, ref_sorted, ref_perm = capi.cv_forward_dev(xpad, w, p, want_aux=True)
                out, sz, perm, ck = (v.cpu().numpy() for v in snn.snncv(t(xpad), t(w), p, return_aux=True))
                dx, dw, _ = (v.cpu().numpy() for v in snn.snncv_grad(t(g), t(xpad), t(w), p, t(ref_out)))
                rdx, rdw, _ = capi.cv_backward_dev(g, xpad, w, p, ref_out, wide=True)
                ao = ref_out.copy(); ao[B:] = np.abs(ao[B:])
                adx, adw, _ = capi.cv_backward_dev(np.abs(g), xpad, np.abs(w), p, ao, wide=True)
            desc += f" bias={biasvolt} theta={theta} max={max_time} quant={quant} sent={sent}"
            assert np.array_equal(sz, ref_sorted), "sorted"
            assert np.array_equal(perm, ref_perm), "perm"
            assert np.array_equal(ck, ref_k), "k"
            assert np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)), "y/r"
            check_grad(dx, rdx, adx, "dX"); check_grad(dw, rdw, adw, "dW")
        except AssertionError as e:
            fails.append(f"case {seed0}/{case}: {desc}: {str(e)[:300]}")
    assert not fails, "\n".join(fails)


@pytest.mark.parametrize("seed0", [21, 22])
def test_random_classifier_heads(seed0):
    """Layers with few work items (few outputs, moderate batch), where the wavefronts of a workgroup share
    one scan: random row lengths 128..1000, every column-slice width, one or more slices, batches up to
    what the kernel takes, ragged numbers of real inputs, rows without any, ties, weights of both signs,
    columns that never fire.  y, 1/S and the causal-set sizes bit-exact, with and without the extra outputs."""
    import snntc_amd as snn
    n_cases, fails = 100, []
    for case in range(n_cases):
        rng = np.random.default_rng(seed0 * 100000 + case)
        biasvolt = float(rng.choice([0.0, 1.0, 1.0, 0.6]))
        theta = float(rng.choice([1.0, 1.0, 0.5, 2.0]))
        max_time = float(rng.choice([1e5, 1e5, 30.0]))
        I = int(rng.choice([128, 129, 136, 200, 264, 511, 512, 784, 800, 900, int(rng.integers(128, 1000))]))
        J = int(rng.choice([1, 3, 5, 8, 9, 10, 16, 17, 24, 32, 33, 40, 64, 70, 100]))
        cols = 64                                            # the library's slice width for this J
        while cols > 8 and cols // 2 >= J:
            cols //= 2
        segs = (64 if cols == 64 else 32) // cols            # samples per work item
        slices = (J + cols - 1) // cols
        B = int(rng.integers(1, min(max(1, 256 // slices * segs), 300) + 1))
        rows = I + (1 if biasvolt > 1e-8 else 0)
        x = np.exp(1.5 * rng.random((B, I))).astype(np.float32)
        if rng.random() < 0.3: x = (np.round(x * 4) / 4).astype(np.float32)
        if rng.random() < 0.5: x[rng.random((B, I)) < rng.random((B, 1)) * 0.6] = np.float32(max_time)
        if rng.random() < 0.3: x[int(rng.integers(0, B))] = np.float32(max_time)
        w = ((3.0 / I + np.sqrt(2.0 / I) * rng.standard_normal((rows, J))) * theta * rng.choice([1.0, 0.3, 3.0])).astype(np.float32)
        if rng.random() < 0.2: w = rng.standard_normal((rows, J)).astype(np.float32)
        if rng.random() < 0.3: w[:, int(rng.integers(0, J))] = -np.abs(w[:, 0])
        p = capi.fc_params(biasvolt, max_time=max_time, theta=theta)
        ref_out, ref_k, _, _ = capi.fc_forward_dev(x, w, p, want_aux=True)
        out, _, _, ck = snn.snnfc(t(x), t(w), p, return_aux=True)
        out2 = snn.snnfc(t(x), t(w), p)
        torch.cuda.synchronize()
        out, ck, out2 = out.cpu().numpy(), ck.cpu().numpy(), out2.cpu().numpy()
        desc = f"case {seed0}/{case}: B={B} I={I} J={J} bias={biasvolt} theta={theta} max={max_time}"
        if not np.array_equal(ck, ref_k): fails.append(desc + ": k")
        elif not np.array_equal(out.view(np.uint32), ref_out.view(np.uint32)): fails.append(desc + ": y/r")
        elif not np.array_equal(out2.view(np.uint32), ref_out.view(np.uint32)): fails.append(desc + ": y/r (plain)")
    assert not fails, "\n".join(fails)
