"""Independent numpy (float64) statements of the SNN-TC neuron, used to pin the C restatement.

Test infrastructure only.  Nothing here shares code with ``snntc_oracle.c``:

* ``neuron_closed_form`` / ``fc_forward_closed_form`` follow the hand-calculation recipe the
  reference's own tests carry (snntc/test-snn-fc-forward.py:83-89,
  snntc/test-snn-cv-forward.py:133-146 and mycompare, :150-171):

      ind = argsort(x); x2, w2 = x[ind], w[ind]
      y2  = cumsum(x2*w2) / (cumsum(w2) - 1)
      valid = (y2 > x2) & (y2 <= concatenate(x2[1:], [1e5]));  out = y2[valid][0]

* ``fc_forward_pyref`` restates the cumsum / where / reduce_min formulation of the reference's
  pure-TensorFlow layer (snntc/SNN_TC_pyref.py:28-53), which treats the bias as an ordinary input
  of value 1.0 and never fires while sum(w) < 1.
* ``analytic_grads`` are the textbook derivatives of y = sum_C(w x) / (sum_C w - theta) over the
  causal set C; ``fd_grads`` are central finite differences of the float64 forward.
* ``min_pool`` / ``min_pool_grad`` restate SNN_maxpool2d (SNN_TC_Modules.py:215-246) literally:
  pad with padvalue, negate, VALID max pooling, negate; the gradient goes to the first position of
  the padded window (row-major) that holds the maximum of -x.
* ``same_pad`` is the SAME-padding split of SNN_conv (SNN_TC_Modules.py:147-161), which the
  reference's test recomputes independently (snntc/test-snn-cv-forward.py:70-75,126-131).
"""
import numpy as np

MAX_TIME = 1e5


def neuron_closed_form(x, wcol, bias_w=None, biasvolt=1.0, theta=1.0, max_time=MAX_TIME,
                       bias_first=True):
    """One neuron.  Returns (y, k, S): spike time, number of *real* inputs in the causal set and
    S = sum_C w - theta; (max_time, -1, 0.0) when the neuron never fires.

    bias_first=True puts the bias ahead of every input (what the reference's kernels do,
    snntc/snnfc_kernels.cu.cc:15-18,34-40); bias_first=False sorts it with the rest, exactly as
    the reference test's recipe does (x=1 appended, snntc/test-snn-cv-forward.py:134-137).
    """
    x = np.asarray(x, np.float64)
    wcol = np.asarray(wcol, np.float64)
    order = np.argsort(x, kind="stable")
    xs, ws = x[order], wcol[order]
    is_bias = np.zeros(xs.shape, bool)
    if bias_w is not None:
        if bias_first:
            xs = np.concatenate(([biasvolt], xs)); ws = np.concatenate(([bias_w], ws))
            is_bias = np.concatenate(([True], is_bias))
        else:
            xa = np.concatenate((x, [biasvolt])); wa = np.concatenate((wcol, [bias_w]))
            fl = np.concatenate((np.zeros(x.shape, bool), [True]))
            o2 = np.argsort(xa, kind="stable")
            xs, ws, is_bias = xa[o2], wa[o2], fl[o2]
    if xs.size == 0:
        return max_time, -1, 0.0
    S = np.cumsum(ws) - theta
    with np.errstate(divide="ignore", invalid="ignore"):
        y = np.cumsum(xs * ws) / S
    nxt = np.concatenate((xs[1:], [max_time]))
    valid = (y > xs) & (y <= nxt) & (xs <= max_time - 0.1)
    # a candidate equal to max_time or beyond is clamped to "never fires" by the kernels
    valid &= y < max_time
    hit = np.flatnonzero(valid)
    if hit.size == 0:
        return max_time, -1, 0.0
    p = hit[0]
    k = int(p + 1 - np.count_nonzero(is_bias[:p + 1]))
    return float(y[p]), k, float(S[p])


def fc_forward_closed_form(x, w, params):
    """Dense layer through ``neuron_closed_form`` (bias first).  Returns y[B,J], k[B,J], S[B,J]."""
    x = np.asarray(x); w = np.asarray(w)
    max_time, theta, biasvolt = float(params[0]), float(params[2]), float(params[5])
    B, I = x.shape
    J = w.shape[1]
    bias = biasvolt > 1e-8
    y = np.empty((B, J)); k = np.empty((B, J), np.int64); S = np.empty((B, J))
    for b in range(B):
        for j in range(J):
            y[b, j], k[b, j], S[b, j] = neuron_closed_form(
                x[b], w[:I, j], w[I, j] if bias else None, biasvolt, theta, max_time)
    return y, k, S


def fc_forward_pyref(x, w, bias, max_time=MAX_TIME):
    """The reference's pure-TF dense forward (snntc/SNN_TC_pyref.py:28-53) in numpy float64.
    Bias = an extra input of value 1.0 sorted with the rest; descending top_k of -x puts the lower
    index first among equal values."""
    x = np.asarray(x, np.float64); w = np.asarray(w, np.float64)
    B = x.shape[0]
    if bias:
        x = np.concatenate((x, np.ones((B, 1))), axis=1)
    order = np.argsort(x, axis=1, kind="stable")
    xs = np.take_along_axis(x, order, axis=1)[:, :, None]            # [B,I,1]
    wsort = w[order]                                                   # [B,I,J]
    wsum = np.cumsum(wsort, axis=1)
    ysum = np.cumsum(wsort * xs, axis=1)
    cand = ysum / np.clip(wsum - 1.0, 1e-10, 1e10)
    cand = np.where(wsum < 1.0, max_time, cand)
    cand = np.where(cand < xs, max_time, cand)
    nxt = np.concatenate((xs[:, 1:], np.full((B, 1, 1), max_time)), axis=1)
    cand = np.where(cand > nxt, max_time, cand)
    return cand.min(axis=1)


def im2col(xpad, Kh, Kw, Sh, Sw):
    """patches[B*Nh*Nw, Kh*Kw*C], depth order (kh,kw,c), patch order (b,nh,nw)."""
    B, H, W, C = xpad.shape
    Nh, Nw = (H - Kh) // Sh + 1, (W - Kw) // Sw + 1
    out = np.empty((B, Nh, Nw, Kh, Kw, C), xpad.dtype)
    for nh in range(Nh):
        for nw in range(Nw):
            out[:, nh, nw] = xpad[:, nh * Sh:nh * Sh + Kh, nw * Sw:nw * Sw + Kw, :]
    return out.reshape(B * Nh * Nw, Kh * Kw * C)


def same_pad(size, kernel, stride):
    """(before, after) padding of SNN_conv's SAME mode along one axis
    (SNN_TC_Modules.py:147-161): total = (ceil(size/stride)-1)*stride + kernel - size,
    before = int(total/2), after = total - before."""
    total = int((np.ceil(size / stride) - 1.0) * stride + kernel) - size
    before = int(total / 2)
    return before, total - before


def causal_mask_from_rank(perm, k):
    """mask[b,i,j] = input i of sample b is among the first k[b,j] sorted inputs."""
    B, I = perm.shape
    rank = np.empty_like(perm)
    np.put_along_axis(rank, perm, np.broadcast_to(np.arange(I, dtype=perm.dtype), (B, I)), axis=1)
    return rank[:, :, None] < k[:, None, :]


def analytic_grads(g, x, w, y, S, mask, biasvolt):
    """Derivatives of sum_bj g_bj * y_bj given causal-set membership mask[b,i,j] (float64):
    dy/dx_i = w_i/S, dy/dw_i = (x_i - y)/S, dy/dw_bias = (biasvolt - y)/S."""
    g = np.asarray(g, np.float64); x = np.asarray(x, np.float64); w = np.asarray(w, np.float64)
    I = x.shape[1]
    fired = S != 0
    up = np.where(fired, g / np.where(fired, S, 1.0), 0.0)                 # [B,J]
    m = mask & fired[:, None, :]
    dx = np.einsum("bij,bj,ij->bi", m, up, w[:I])
    dw = np.einsum("bij,bj->ij", m * (x[:, :, None] - y[:, None, :]), up)
    if w.shape[0] > I:
        dwb = np.einsum("bj,bj->j", np.where(fired, biasvolt - y, 0.0), up)
        dw = np.concatenate((dw, dwb[None]), axis=0)
    return dx, dw


def fd_grads(g, x, w, params, h=1e-6, probes=64, seed=0):
    """Central finite differences of L = sum g*y (float64 closed-form forward) at ``probes`` random
    coordinates of x and of w.  Returns lists of (index, value)."""
    rng = np.random.default_rng(seed)
    x = np.asarray(x, np.float64).copy(); w = np.asarray(w, np.float64).copy()
    g = np.asarray(g, np.float64)

    def loss():
        y, k, _ = fc_forward_closed_form(x, w, params)
        return float(np.sum(np.where(k >= 0, g * y, 0.0)))

    out_x, out_w = [], []
    for _ in range(probes):
        b, i = rng.integers(x.shape[0]), rng.integers(x.shape[1])
        x0 = x[b, i]
        x[b, i] = x0 + h; lp = loss(); x[b, i] = x0 - h; lm = loss(); x[b, i] = x0
        out_x.append(((b, i), (lp - lm) / (2 * h)))
        r, c = rng.integers(w.shape[0]), rng.integers(w.shape[1])
        w0 = w[r, c]
        w[r, c] = w0 + h; lp = loss(); w[r, c] = w0 - h; lm = loss(); w[r, c] = w0
        out_w.append(((r, c), (lp - lm) / (2 * h)))
    return out_x, out_w


def softmax_time_loss(times, label):
    """float64 statement of loss_func (SNN_TC_Modules.py:286-288): per-sample cross-entropy of `label`
    against softmax(-times), and the gradient of the batch mean with respect to `times`."""
    t = np.asarray(times, np.float64); y = np.asarray(label, np.float64)
    l = -t
    l = l - l.max(axis=1, keepdims=True)
    lse = np.log(np.exp(l).sum(axis=1, keepdims=True))
    logp = l - lse
    sample = -(y * logp).sum(axis=1)
    grad = (y - np.exp(logp) * y.sum(axis=1, keepdims=True)) / t.shape[0]
    return sample, grad


def min_pool(x, Kh, Kw, Sh, Sw, same=True, pad_value=1e5):
    """SNN_maxpool2d (SNN_TC_Modules.py:215-246) on NHWC x, written as the reference writes it: pad
    with pad_value (SAME split as same_pad), then -maxpool(-xpad) over VALID windows.
    Returns (y[B,Nh,Nw,C], arg[B,Nh,Nw,C], (top, left)); arg = kh*Kw + kw of the first position of the
    padded window, in row-major order, that holds the maximum of -x."""
    x = np.asarray(x, np.float32)
    B, H, W, C = x.shape
    (top, bottom), (left, right) = (same_pad(H, Kh, Sh), same_pad(W, Kw, Sw)) if same else ((0, 0), (0, 0))
    xpad = np.pad(x, ((0, 0), (top, bottom), (left, right), (0, 0)), constant_values=np.float32(pad_value))
    Nh = (xpad.shape[1] - Kh) // Sh + 1
    Nw = (xpad.shape[2] - Kw) // Sw + 1
    neg = -xpad
    best = np.full((B, Nh, Nw, C), -np.inf, np.float32)
    arg = np.zeros((B, Nh, Nw, C), np.int32)
    for kh in range(Kh):
        for kw in range(Kw):
            v = neg[:, kh:kh + (Nh - 1) * Sh + 1:Sh, kw:kw + (Nw - 1) * Sw + 1:Sw, :]
            better = v > best                                  # strictly greater: the first maximum stays
            arg[better] = kh * Kw + kw
            best = np.where(better, v, best)
    return -best, arg, (top, left)


def min_pool_grad(grad_y, arg, in_shape, Kh, Kw, Sh, Sw, pad):
    """Gradient of min_pool: each window's gradient goes to the padded-window position arg names;
    what lands in the padding is dropped.  Contributions to a pixel are added in (kh, kw) order."""
    B, H, W, C = in_shape
    top, left = pad
    gy = np.asarray(grad_y, np.float32)
    Nh, Nw = gy.shape[1], gy.shape[2]
    dx = np.zeros((B, H, W, C), np.float32)
    for kh in range(Kh):
        for kw in range(Kw):
            hit = arg == kh * Kw + kw
            for nh in range(Nh):
                h = nh * Sh - top + kh
                if h < 0 or h >= H:
                    continue
                for nw in range(Nw):
                    w = nw * Sw - left + kw
                    if w < 0 or w >= W:
                        continue
                    dx[:, h, w, :] += np.where(hit[:, nh, nw, :], gy[:, nh, nw, :], np.float32(0))
    return dx

