"""CPU oracle for whole layer stacks (test infrastructure): runs the network descriptions of
snntc_amd.networks through the C oracle (conv / dense), the numpy closed forms (pooling, loss) and
plain numpy (flatten, global minimum), forward and backward.

Two uses:
  * OracleChain.forward / backward: an independent chain -- oracle activations feed oracle layers,
    oracle gradients feed oracle backward passes;
  * check_layer_by_layer: every layer of a GPU run is compared with the oracle applied to that
    layer's GPU inputs (activations and upstream gradient), so each comparison is a single-layer one
    and the tolerance does not have to grow with depth.
"""
import numpy as np

from helpers import grad_band
from oracle import capi, closed_form as cf


def assert_in_band(actual, ref, ref_abs, what, depth=1):
    a = np.asarray(actual, np.float64); e = np.asarray(ref, np.float64)
    assert a.shape == e.shape, f"{what}: shape {a.shape} vs {e.shape}"
    lim = grad_band(e, ref_abs, depth)
    err = np.abs(a - e)
    bad = err > lim
    if bad.any():
        idx = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: {bad.sum()}/{bad.size} out of tolerance; worst {idx}: got {a[idx]!r} "
                             f"want {e[idx]!r} diff {err[idx]:.3e} lim {lim[idx]:.3e}")


class OracleLayer:
    """One layer of a spec with numpy weights; forward(x) keeps what backward(g) needs."""

    def __init__(self, item, weight=None, max_time=1e5):
        self.item, self.kind, self.w, self.max_time = item, item[0], weight, max_time
        if self.kind == "conv":
            _, _ci, _co, k, s = item
            self.k, self.s = k, s
            self.params = capi.cv_params(k, k, s, s, same=True, biasvolt=1.0, max_time=max_time)
        elif self.kind == "dense":
            self.params = capi.fc_params(1.0, max_time=max_time)

    # ---- forward ---------------------------------------------------------------------------------
    def forward(self, x):
        self.x = x
        B = x.shape[0]
        if self.kind == "conv":
            (t, b), (l, r) = cf.same_pad(x.shape[1], self.k, self.s), cf.same_pad(x.shape[2], self.k, self.s)
            self.pad = (t, b, l, r)
            self.xin = np.ascontiguousarray(
                np.pad(x, ((0, 0), (t, b), (l, r), (0, 0)), constant_values=np.float32(self.max_time)))
            self.out = capi.cv_forward_dev(self.xin, self.w, self.params)
            return np.ascontiguousarray(self.out[:B])
        if self.kind == "dense":
            self.xin = np.ascontiguousarray(x)
            self.out = capi.fc_forward_dev(self.xin, self.w, self.params)
            return np.ascontiguousarray(self.out[:B])
        if self.kind == "pool":
            y, self.arg, self.pool_pad = cf.min_pool(x, self.item[1], self.item[1], self.item[2], self.item[2], True)
            return y
        if self.kind == "gmin":
            flat = x.reshape(B, -1, x.shape[3])
            self.arg = flat.argmin(axis=1)                      # first position attaining the minimum
            return np.ascontiguousarray(flat.min(axis=1))
        if self.kind == "flatten":
            return np.ascontiguousarray(x.reshape(B, -1))
        raise ValueError(self.kind)

    # ---- backward: returns (dx, dw or None, |dx| scale, |dw| scale or None) ------------------------
    def backward(self, g, want_abs=True):
        B = self.x.shape[0]
        if self.kind in ("conv", "dense"):
            full = np.zeros_like(self.out)
            full[:B] = g
            fn = capi.cv_backward_dev if self.kind == "conv" else capi.fc_backward_dev
            dx, dw, _ = fn(full, self.xin, self.w, self.params, self.out, wide=True)
            adx = adw = None
            if want_abs:
                ao = self.out.copy(); ao[B:] = np.abs(ao[B:])
                adx, adw, _ = fn(np.abs(full), self.xin, np.abs(self.w), self.params, ao, wide=True)
            if self.kind == "conv":
                t, b, l, r = self.pad
                H, W = self.x.shape[1], self.x.shape[2]
                dx = np.ascontiguousarray(dx[:, t:t + H, l:l + W, :])
                if want_abs:
                    adx = np.ascontiguousarray(adx[:, t:t + H, l:l + W, :])
            return dx, dw, adx, adw
        if self.kind == "pool":
            k, s = self.item[1], self.item[2]
            dx = cf.min_pool_grad(g, self.arg, self.x.shape, k, k, s, s, self.pool_pad)
            return dx, None, np.abs(dx), None
        if self.kind == "gmin":
            dx = np.zeros((B, self.x.shape[1] * self.x.shape[2], self.x.shape[3]), np.float32)
            np.put_along_axis(dx, self.arg[:, None, :], np.asarray(g, np.float32)[:, None, :], axis=1)
            dx = dx.reshape(self.x.shape)
            return dx, None, np.abs(dx), None
        if self.kind == "flatten":
            dx = np.asarray(g, np.float32).reshape(self.x.shape)
            return dx, None, np.abs(dx), None
        raise ValueError(self.kind)


class OracleChain:
    def __init__(self, spec, weights):
        weights = list(weights)
        self.layers = [OracleLayer(item, weights.pop(0) if item[0] in ("conv", "dense") else None) for item in spec]

    def forward(self, z):
        h = np.ascontiguousarray(z, np.float32)
        self.acts = []
        for layer in self.layers:
            self.acts.append(h)
            h = layer.forward(h)
        self.times = h
        return h

    def loss_and_backward(self, onehot):
        """Returns (sample_loss[B] float64, [dW per weighted layer], [|dW| scale per weighted layer])."""
        sample, g = cf.softmax_time_loss(self.times, onehot)
        g = g.astype(np.float32)
        dws, adws = [], []
        for layer in reversed(self.layers):
            dx, dw, _, adw = layer.backward(g)
            if dw is not None:
                dws.append(dw); adws.append(adw)
            g = dx
        self.dz = g
        return sample, dws[::-1], adws[::-1]


def run_gpu_chain(torch, snn, net, z, onehot, input_grad=True):
    """Forward + loss + backward of `net` under autograd, keeping every layer's input, output and the
    gradient that reached its output.  Returns (acts_in, outs, sample_loss, dtimes)."""
    z = z.clone().requires_grad_(input_grad)
    acts, outs = [], []
    h = z
    for layer in net:
        acts.append(h)
        h = layer(h)
        if h.requires_grad:
            h.retain_grad()
        outs.append(h)
    sample_loss, dtimes = snn.softmax_time_loss(h.detach(), onehot)
    for w in net.weights():
        w.grad = None
    h.backward(dtimes)
    torch.cuda.synchronize()
    return acts, outs, sample_loss, dtimes


def check_layer_by_layer(spec, net, acts, outs, check_input_grad=True):
    """Every layer of the GPU run against the oracle applied to that layer's GPU inputs: forward results
    bit-exact, dX / dW within the single-layer band.  Returns the per-layer worst error / band ratios."""
    report = []
    for i, (item, mod) in enumerate(zip(spec, net)):
        w = mod.weight.detach().cpu().numpy() if hasattr(mod, "weight") else None
        ol = OracleLayer(item, w)
        x = acts[i].detach().cpu().numpy()
        ref = ol.forward(x)
        got = outs[i].detach().cpu().numpy()
        assert got.shape == ref.shape, f"layer {i} {item}: shape {got.shape} vs {ref.shape}"
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"layer {i} {item}: forward not bit-exact"
        g = outs[i].grad
        if g is None:
            continue
        dx, dw, adx, adw = ol.backward(g.cpu().numpy())
        what = f"layer {i} {item}"
        if acts[i].grad is not None and (check_input_grad or i > 0):
            gdx = acts[i].grad.cpu().numpy()
            if ol.kind in ("pool", "gmin", "flatten"):
                assert np.array_equal(gdx, dx), f"{what}: dX is a plain routing of the gradient and must be exact"
            else:
                assert_in_band(gdx, dx, adx, what + " dX")
                report.append((what + " dX", float(np.max(np.abs(gdx - dx) / grad_band(dx, adx)))))
        if dw is not None:
            gdw = mod.weight.grad.cpu().numpy()
            assert_in_band(gdw, dw, adw, what + " dW")
            report.append((what + " dW", float(np.max(np.abs(gdw - dw) / grad_band(dw, adw)))))
    return report
