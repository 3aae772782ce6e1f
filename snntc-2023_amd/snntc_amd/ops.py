"""The four SNN-TC ops over PyTorch-ROCm tensors, each a thin call into the C ABI.

Counterparts of the reference's op handles (SNN_TC_Modules.py:29-33, 89-93):

    snnfc(X, W, Params)                      -> Y[2B, J]
    snnfc_grad(grad, X, W, Params, Y)        -> (dX, dW, dParams)
    snncv(Xpad, W, Params)                   -> Y[2B, Nh, Nw, Kc]
    snncv_grad(grad, Xpad, W, Params, Y)     -> (dXpad, dW, dParams)

``SnnFc`` / ``SnnCv`` are the autograd bindings that replace ``@ops.RegisterGradient``.
Tensors must be float32 on a ROCm device; ``Params`` is the host-side float32 vector the layers
build.  PyTorch only supplies device memory and the current HIP stream.
"""
import ctypes

import numpy as np
import torch

from . import _lib

_workspaces = {}
_giveups_seen = {}


def check_scan_health(device=None):
    """Raises SnntcError if, since the last call for this device, a wavefront of the classifier-head scan
    ran out of its bounded wait (the affected outputs are NaN).  Synchronises with the current stream of
    the device: call it where the program waits for the GPU anyway (after reading a loss, at the end of
    an epoch or of a batch of requests)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(device):
        n = _lib.scan_giveups(torch.cuda.current_stream(device).cuda_stream)
    before = _giveups_seen.get(device.index, 0)
    _giveups_seen[device.index] = n
    if n > before:
        raise _lib.SnntcError(_lib.ERR_HIP, f"{n - before} scan wavefront(s) gave up waiting for partial sums on "
                                            f"{device}: the outputs of their work items are NaN")
    return n


def _params(params, n):
    p = np.ascontiguousarray(np.asarray(params, dtype=np.float32).reshape(-1))
    if p.size != n:
        raise ValueError(f"Params must hold {n} float32 values, got {p.size}")
    return p, p.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _dev_f32(t, name, ndim):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise _lib.SnntcLibraryError(
            f"{name} lives on {t.device}: the SNN-TC ops run on a ROCm GPU only (no CPU fallback)")
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dimensions, got shape {tuple(t.shape)}")
    return t.contiguous()


def _workspace(device, nbytes):
    """Scratch for one op call.  Eager calls share a grow-only buffer per (device, stream), whose
    contents never outlive the call.  While the stream is being captured into a HIP graph the buffer
    is allocated per call instead: its address is baked into the graph, so it has to belong to the
    graph's own memory pool (which keeps it alive exactly as long as the graph) and must not be a
    cached tensor that a later, larger request would replace and free."""
    nbytes = max(int(nbytes), 256)
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _written_behind_autograd(t):
    """A kernel has written into `t` through its raw pointer.  Autograd counts in-place writes per tensor
    and refuses to run a backward pass whose saved tensors have been written since they were saved; the
    count is advanced here so that this protection also covers the padded input buffers the chained
    layers fill (a second forward pass before the backward pass of the first would otherwise silently
    differentiate against the second pass's input)."""
    torch.autograd.graph.increment_version(t)


def release_workspaces():
    """Drops the cached eager scratch buffers (they are re-created on demand)."""
    _workspaces.clear()


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def snnfc(X, W, Params, return_aux=False):
    """Dense forward.  X[B,I], W[I+bias,J] -> Y[2B,J] (spike times ; 1/(sum w - theta)).
    With return_aux=True also returns (sorted_z[B,I], perm[B,I] int32, causal_k[B,J] int32)."""
    lib = _lib.load()
    X = _dev_f32(X, "X", 2)
    W = _dev_f32(W, "W", 2)
    p, pp = _params(Params, 6)
    B, I = X.shape
    w_rows, J = W.shape
    with torch.cuda.device(X.device):
        need = ctypes.c_size_t()
        _lib.check(lib.snntc_fc_forward_workspace_bytes(B, I, J, ctypes.byref(need)))
        ws = _workspace(X.device, need.value)
        out = torch.empty((2 * B, J), dtype=torch.float32, device=X.device)
        if return_aux:
            sz = torch.empty((B, I), dtype=torch.float32, device=X.device)
            perm = torch.empty((B, I), dtype=torch.int32, device=X.device)
            ck = torch.empty((B, J), dtype=torch.int32, device=X.device)
            _lib.check(lib.snntc_fc_forward_ex(_ptr(X), _ptr(W), pp, _ptr(out), _ptr(sz), _ptr(perm), _ptr(ck),
                                               B, I, J, w_rows, _ptr(ws), ws.numel(), _stream(X.device)))
            return out, sz, perm, ck
        _lib.check(lib.snntc_fc_forward(_ptr(X), _ptr(W), pp, _ptr(out), B, I, J, w_rows, _ptr(ws), ws.numel(),
                                        _stream(X.device)))
    return out


def init(device=None):
    """One-time set-up of a device (kernel attributes, the library's static scratch): call it before
    capturing library calls into a HIP graph.  device=None means the current device."""
    lib = _lib.load()
    if device is None:
        index = -1
    else:
        index = torch.device(device).index
        index = torch.cuda.current_device() if index is None else index
    _lib.check(lib.snntc_init(index))


def snnfc_static(X, W, Params, out=None):
    """snnfc through the entry point that allocates nothing: the scratch is a static device array
    inside the library (snntc_static_scratch_bytes()).  `out` may be a preallocated [2B,J] tensor.
    Calls on one GPU share that array: do not overlap them."""
    lib = _lib.load()
    X = _dev_f32(X, "X", 2)
    W = _dev_f32(W, "W", 2)
    p, pp = _params(Params, 6)
    B, I = X.shape
    w_rows, J = W.shape
    with torch.cuda.device(X.device):
        if out is None:
            out = torch.empty((2 * B, J), dtype=torch.float32, device=X.device)
        elif tuple(out.shape) != (2 * B, J) or out.dtype != torch.float32 or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous float32 [{2 * B},{J}] tensor")
        _lib.check(lib.snntc_fc_forward_static(_ptr(X), _ptr(W), pp, _ptr(out), B, I, J, w_rows, _stream(X.device)))
    return out


def snnfc_grad(grad, X, W, Params, Y, want_dparams=True, want_dx=True, want_dw=True, first_half_grad=False):
    """Dense backward.  grad[2B,J], Y[2B,J] = forward output -> (dX[B,I], dW like W, dParams[6]).
    dParams is all zeros (Params is a constant).  A want_* flag set to False skips that gradient
    (None is returned in its place)."""
    lib = _lib.load()
    grad = _dev_f32(grad, "grad", 2)
    X = _dev_f32(X, "X", 2)
    W = _dev_f32(W, "W", 2)
    Y = _dev_f32(Y, "Y", 2)
    p, pp = _params(Params, 6)
    B, I = X.shape
    w_rows, J = W.shape
    if Y.shape[0] != 2 * B or Y.shape[1] != J or grad.shape[1] != J:
        raise ValueError(f"Grad/Oldout batch should be 2 * batch: Y {tuple(Y.shape)}, grad {tuple(grad.shape)}, "
                         f"X {tuple(X.shape)}, W {tuple(W.shape)}")
    with torch.cuda.device(X.device):
        need = ctypes.c_size_t()
        _lib.check(lib.snntc_fc_backward_workspace_bytes(B, I, J, ctypes.byref(need)))
        ws = _workspace(X.device, need.value)
        dX = torch.empty_like(X) if want_dx else None
        dW = torch.empty_like(W) if want_dw else None
        dP = torch.empty(6, dtype=torch.float32, device=X.device) if want_dparams else None
        # the op only ever reads rows [0,B) of grad, so a caller that holds just those rows passes them as is
        grad_rows = 2 * B if (first_half_grad and grad.shape[0] == B) else grad.shape[0]
        _lib.check(lib.snntc_fc_backward(_ptr(grad), _ptr(X), _ptr(W), pp, _ptr(Y), _ptr(dX), _ptr(dW), _ptr(dP),
                                         B, I, J, w_rows, grad_rows, _ptr(ws), ws.numel(), _stream(X.device)))
    return dX, dW, dP


def snncv_output_dims(H, W, Params):
    lib = _lib.load()
    p, pp = _params(Params, 12)
    nh, nw = ctypes.c_int64(), ctypes.c_int64()
    _lib.check(lib.snntc_cv_output_dims(H, W, pp, ctypes.byref(nh), ctypes.byref(nw)))
    return nh.value, nw.value


def snncv(X, W, Params, return_aux=False, next_xpad=None, next_offset=(0, 0)):
    """Conv forward on the already padded / cropped NHWC input X[B,H,W,C]; W[Kh*Kw*C+bias,Kc]
    -> Y[2B,Nh,Nw,Kc].  With return_aux=True also returns per-patch (sorted_z, perm, causal_k).
    next_xpad[B,h,w,Kc], if given, also receives the spike times, output pixel (nh, nw) at its pixel
    (nh + next_offset[0], nw + next_offset[1]): the padded input of the conv layer that follows."""
    lib = _lib.load()
    X = _dev_f32(X, "X", 4)
    W = _dev_f32(W, "W", 2)
    p, pp = _params(Params, 12)
    B, H, Wd, C = X.shape
    w_rows, Kc = W.shape
    Nh, Nw = snncv_output_dims(H, Wd, p)
    with torch.cuda.device(X.device):
        need = ctypes.c_size_t()
        _lib.check(lib.snntc_cv_forward_workspace_bytes(B, H, Wd, C, Kc, pp, ctypes.byref(need)))
        ws = _workspace(X.device, need.value)
        out = torch.empty((2 * B, Nh, Nw, Kc), dtype=torch.float32, device=X.device)
        if return_aux:
            S, P = B * Nh * Nw, int(p[6]) * int(p[7]) * C
            sz = torch.empty((S, P), dtype=torch.float32, device=X.device)
            perm = torch.empty((S, P), dtype=torch.int32, device=X.device)
            ck = torch.empty((S, Kc), dtype=torch.int32, device=X.device)
            _lib.check(lib.snntc_cv_forward_ex(_ptr(X), _ptr(W), pp, _ptr(out), _ptr(sz), _ptr(perm), _ptr(ck),
                                               B, H, Wd, C, Kc, w_rows, _ptr(ws), ws.numel(), _stream(X.device)))
            return out, sz, perm, ck
        if next_xpad is not None:
            nx = _dev_f32(next_xpad, "next_xpad", 4)
            if nx.shape[0] != B or nx.shape[3] != Kc:
                raise ValueError(f"next_xpad {tuple(nx.shape)} does not match batch {B} / channels {Kc}")
            _lib.check(lib.snntc_cv_forward_chained(_ptr(X), _ptr(W), pp, _ptr(out), _ptr(nx), nx.shape[1], nx.shape[2],
                                                    next_offset[0], next_offset[1], B, H, Wd, C, Kc, w_rows, _ptr(ws),
                                                    ws.numel(), _stream(X.device)))
            _written_behind_autograd(next_xpad)
            return out
        _lib.check(lib.snntc_cv_forward(_ptr(X), _ptr(W), pp, _ptr(out), B, H, Wd, C, Kc, w_rows, _ptr(ws),
                                        ws.numel(), _stream(X.device)))
    return out


def snncv_grad(grad, X, W, Params, Y, want_dparams=True, want_dx=True, want_dw=True, first_half_grad=False,
               crop=None):
    """Conv backward -> (dXpad like X, dW like W, dParams[12] of zeros, or None if not wanted).
    crop = (h, w, top, left): dX is only that window of the padded input's gradient, [B,h,w,C] (the
    gradient with respect to the image before its SAME padding)."""
    lib = _lib.load()
    grad = _dev_f32(grad, "grad", 4)
    X = _dev_f32(X, "X", 4)
    W = _dev_f32(W, "W", 2)
    Y = _dev_f32(Y, "Y", 4)
    p, pp = _params(Params, 12)
    B, H, Wd, C = X.shape
    w_rows, Kc = W.shape
    if Y.shape[0] != 2 * B or tuple(grad.shape[1:]) != tuple(Y.shape[1:]) or Y.shape[3] != Kc:
        raise ValueError(f"Grad/Oldout batch should be 2 * batch: Y {tuple(Y.shape)}, grad {tuple(grad.shape)}, "
                         f"X {tuple(X.shape)}, W {tuple(W.shape)}")
    with torch.cuda.device(X.device):
        need = ctypes.c_size_t()
        _lib.check(lib.snntc_cv_backward_workspace_bytes(B, H, Wd, C, Kc, pp, ctypes.byref(need)))
        ws = _workspace(X.device, need.value)
        dW = torch.empty_like(W) if want_dw else None
        dP = torch.empty(12, dtype=torch.float32, device=X.device) if want_dparams else None
        grad_rows = 2 * B if (first_half_grad and grad.shape[0] == B) else grad.shape[0]
        if crop is not None:
            ch, cw, ctop, cleft = crop
            dX = torch.empty((B, ch, cw, C), dtype=torch.float32, device=X.device) if want_dx else None
            _lib.check(lib.snntc_cv_backward_cropped(_ptr(grad), _ptr(X), _ptr(W), pp, _ptr(Y), _ptr(dX), ch, cw, ctop,
                                                     cleft, _ptr(dW), _ptr(dP), B, H, Wd, C, Kc, w_rows, grad_rows,
                                                     _ptr(ws), ws.numel(), _stream(X.device)))
            return dX, dW, dP
        dX = torch.empty_like(X) if want_dx else None
        _lib.check(lib.snntc_cv_backward(_ptr(grad), _ptr(X), _ptr(W), pp, _ptr(Y), _ptr(dX), _ptr(dW), _ptr(dP),
                                         B, H, Wd, C, Kc, w_rows, grad_rows, _ptr(ws), ws.numel(), _stream(X.device)))
    return dX, dW, dP


class SnnFc(torch.autograd.Function):
    """Y = snnfc(X, W, Params) with the gradient the reference registers for "SnnFc"
    (SNN_TC_Modules.py:31-33): the backward op receives the full [2B,J] forward output."""

    @staticmethod
    def forward(ctx, X, W, Params):
        Y = snnfc(X, W, Params)
        ctx.save_for_backward(X, W, Y)
        ctx.params = np.array(Params, dtype=np.float32, copy=True)
        return Y

    @staticmethod
    def backward(ctx, grad):
        X, W, Y = ctx.saved_tensors
        dX, dW, _ = snnfc_grad(grad.contiguous(), X, W, ctx.params, Y, want_dparams=False,
                               want_dx=ctx.needs_input_grad[0], want_dw=ctx.needs_input_grad[1])
        return dX, dW, None


class SnnCv(torch.autograd.Function):
    """Y = snncv(Xpad, W, Params) with the gradient registered for "SnnCv" (SNN_TC_Modules.py:91-93)."""

    @staticmethod
    def forward(ctx, X, W, Params):
        Y = snncv(X, W, Params)
        ctx.save_for_backward(X, W, Y)
        ctx.params = np.array(Params, dtype=np.float32, copy=True)
        return Y

    @staticmethod
    def backward(ctx, grad):
        X, W, Y = ctx.saved_tensors
        dX, dW, _ = snncv_grad(grad.contiguous(), X, W, ctx.params, Y, want_dparams=False,
                               want_dx=ctx.needs_input_grad[0], want_dw=ctx.needs_input_grad[1])
        return dX, dW, None


class SnnFcTimes(torch.autograd.Function):
    """What SNN_dense.call returns (SNN_TC_Modules.py:73-75): the spike times Y[:B] of snnfc.  The full
    [2B,J] output is kept for the backward op, which then takes the [B,J] upstream gradient directly --
    slicing the output of SnnFc instead costs a zero fill and a copy of [2B,J] per backward pass."""

    @staticmethod
    def forward(ctx, X, W, Params):
        Y = snnfc(X, W, Params)
        ctx.save_for_backward(X, W, Y)
        ctx.params = np.array(Params, dtype=np.float32, copy=True)
        return Y[:X.shape[0]]

    @staticmethod
    def backward(ctx, grad):
        X, W, Y = ctx.saved_tensors
        dX, dW, _ = snnfc_grad(grad.contiguous(), X, W, ctx.params, Y, want_dparams=False,
                               want_dx=ctx.needs_input_grad[0], want_dw=ctx.needs_input_grad[1],
                               first_half_grad=True)
        return dX, dW, None


class SnnCvTimes(torch.autograd.Function):
    """Spike times Y[:B] of snncv, as SNN_conv.call returns them (SNN_TC_Modules.py:168-170)."""

    @staticmethod
    def forward(ctx, X, W, Params):
        Y = snncv(X, W, Params)
        ctx.save_for_backward(X, W, Y)
        ctx.params = np.array(Params, dtype=np.float32, copy=True)
        return Y[:X.shape[0]]

    @staticmethod
    def backward(ctx, grad):
        X, W, Y = ctx.saved_tensors
        dX, dW, _ = snncv_grad(grad.contiguous(), X, W, ctx.params, Y, want_dparams=False,
                               want_dx=ctx.needs_input_grad[0], want_dw=ctx.needs_input_grad[1],
                               first_half_grad=True)
        return dX, dW, None


class SnnCvSame(torch.autograd.Function):
    """SNN_conv with SAME padding as one differentiable step on the un-padded image x[B,H,W,C]: pad with
    MAX_SPIKE_TIME, snncv, and in the backward pass the gradient with respect to x itself (the op stores
    only that window of the padded gradient, so no separate crop runs).
      xpad      None: the padded tensor is made here (one pass).  Otherwise the layer's padded input
                buffer, already holding x in its interior (written there by the layer before, see
                next_xpad) and MAX_SPIKE_TIME on its border.
      next_xpad None, or the padded input buffer of the conv layer that follows: the spike times are
                written there as well, at pixel offset next_offset."""

    @staticmethod
    def forward(ctx, x, W, Params, pads, xpad, next_xpad, next_offset):
        top, bottom, left, right = pads
        B, H, Wd, C = x.shape
        if xpad is None:
            xpad = pad_time(x, top, bottom, left, right, float(Params[0])) if (top or bottom or left or right) else x
        elif tuple(xpad.shape) != (B, top + H + bottom, left + Wd + right, C):
            raise ValueError(f"padded buffer {tuple(xpad.shape)} does not match input {tuple(x.shape)} and pads {pads}")
        Y = snncv(xpad, W, Params, next_xpad=next_xpad, next_offset=next_offset)
        ctx.save_for_backward(xpad, W, Y)
        ctx.params = np.array(Params, dtype=np.float32, copy=True)
        ctx.crop = (H, Wd, top, left)
        return Y[:B]

    @staticmethod
    def backward(ctx, grad):
        X, W, Y = ctx.saved_tensors
        dX, dW, _ = snncv_grad(grad.contiguous(), X, W, ctx.params, Y, want_dparams=False,
                               want_dx=ctx.needs_input_grad[0], want_dw=ctx.needs_input_grad[1],
                               first_half_grad=True, crop=ctx.crop)
        return dX, dW, None, None, None, None, None


def softmax_time_loss(times, label, want_loss=True, want_grad=True):
    """Per-sample cross-entropy of label[B,J] against softmax(-times[B,J]) and the gradient of its batch
    mean with respect to times, in one kernel (loss_func, SNN_TC_Modules.py:286-288).
    Returns (sample_loss[B] or None, dtimes[B,J] or None)."""
    lib = _lib.load()
    times = _dev_f32(times, "times", 2)
    label = _dev_f32(label, "label", 2)
    if tuple(times.shape) != tuple(label.shape):
        raise ValueError(f"loss: times {tuple(times.shape)} and label {tuple(label.shape)} differ in shape")
    B, J = times.shape
    with torch.cuda.device(times.device):
        loss = torch.empty(B, dtype=torch.float32, device=times.device) if want_loss else None
        grad = torch.empty_like(times) if want_grad else None
        _lib.check(lib.snntc_softmax_time_loss(_ptr(times), _ptr(label), _ptr(loss), _ptr(grad), B, J,
                                               _stream(times.device)))
    return loss, grad


def sgd_update(params, grads, lr):
    """In place ``w -= lr * dw`` for every (w, dw) pair, all tensors in one launch: the SGD update of
    a training step (the reference hands it to the framework's optimizer, snntc/snntc-mnist.py:70)."""
    lib = _lib.load()
    params, grads = list(params), list(grads)
    if len(params) != len(grads):
        raise ValueError(f"sgd_update: {len(params)} weight tensors but {len(grads)} gradients")
    if not params:
        return
    ws, gs = [], []
    for i, (w, g) in enumerate(zip(params, grads)):
        w = w.data if isinstance(w, torch.nn.Parameter) else w
        if not (isinstance(w, torch.Tensor) and w.is_cuda and w.dtype == torch.float32 and w.is_contiguous()):
            raise _lib.SnntcLibraryError(f"sgd_update: weight {i} must be a contiguous float32 tensor on a ROCm GPU")
        if tuple(g.shape) != tuple(w.shape) or g.dtype != torch.float32 or g.device != w.device:
            raise ValueError(f"sgd_update: gradient {i} does not match its weight tensor")
        ws.append(w)
        gs.append(g.detach().contiguous())
    k = len(ws)
    vp = ctypes.c_void_p
    w_arr = (vp * k)(*[w.data_ptr() for w in ws])
    g_arr = (vp * k)(*[g.data_ptr() for g in gs])
    n_arr = (ctypes.c_int64 * k)(*[w.numel() for w in ws])
    with torch.cuda.device(ws[0].device):
        _lib.check(lib.snntc_sgd_update(w_arr, g_arr, n_arr, k, float(lr), _stream(ws[0].device)))


class SoftmaxTimeLoss(torch.autograd.Function):
    """mean_b CE(label_b, softmax(-times_b)); the gradient is produced by the forward kernel."""

    @staticmethod
    def forward(ctx, times, label):
        loss, grad = softmax_time_loss(times, label, want_grad=times.requires_grad)
        if grad is not None:
            ctx.save_for_backward(grad)
        ctx.has_grad = grad is not None
        return loss.mean()

    @staticmethod
    def backward(ctx, upstream):
        if not ctx.has_grad:
            return None, None
        (grad,) = ctx.saved_tensors
        return grad * upstream, None


def min_pool(x, kernel, stride, pad, out_hw, pad_value=1e5, want_arg=True, next_xpad=None, next_offset=(0, 0)):
    """Earliest-spike pooling of NHWC spike times x[B,H,W,C] -> (y[B,Nh,Nw,C], arg or None).
    kernel = (Kh, Kw), stride = (Sh, Sw), pad = (top, left), out_hw = (Nh, Nw); pixels outside the
    image count as pad_value.  arg records, per output, the window position that attained the minimum.
    next_xpad[B,h,w,C], if given, also receives y at pixel offset next_offset (the padded input of the
    conv layer that follows)."""
    lib = _lib.load()
    x = _dev_f32(x, "x", 4)
    B, H, W, C = x.shape
    with torch.cuda.device(x.device):
        y = torch.empty((B, out_hw[0], out_hw[1], C), dtype=torch.float32, device=x.device)
        arg = torch.empty(y.shape, dtype=torch.int32, device=x.device) if want_arg else None
        if next_xpad is not None:
            nx = _dev_f32(next_xpad, "next_xpad", 4)
            if nx.shape[0] != B or nx.shape[3] != C:
                raise ValueError(f"next_xpad {tuple(nx.shape)} does not match batch {B} / channels {C}")
            _lib.check(lib.snntc_min_pool_forward_chained(_ptr(x), _ptr(y), _ptr(arg), _ptr(nx), nx.shape[1], nx.shape[2],
                                                          next_offset[0], next_offset[1], B, H, W, C, kernel[0],
                                                          kernel[1], stride[0], stride[1], pad[0], pad[1], out_hw[0],
                                                          out_hw[1], float(pad_value), _stream(x.device)))
            _written_behind_autograd(next_xpad)
            return y, arg
        _lib.check(lib.snntc_min_pool_forward(_ptr(x), _ptr(y), _ptr(arg), B, H, W, C, kernel[0], kernel[1], stride[0],
                                              stride[1], pad[0], pad[1], out_hw[0], out_hw[1], float(pad_value),
                                              _stream(x.device)))
    return y, arg


def min_pool_grad(grad_y, arg, in_shape, kernel, stride, pad):
    """Gradient of min_pool with respect to its input: every pixel adds the gradients of the windows
    that recorded it."""
    lib = _lib.load()
    grad_y = _dev_f32(grad_y, "grad_y", 4)
    B, H, W, C = in_shape
    Nh, Nw = grad_y.shape[1], grad_y.shape[2]
    if tuple(arg.shape) != tuple(grad_y.shape) or arg.dtype != torch.int32 or not arg.is_contiguous():
        raise ValueError("arg must be the contiguous int32 tensor min_pool returned")
    with torch.cuda.device(grad_y.device):
        dx = torch.empty((B, H, W, C), dtype=torch.float32, device=grad_y.device)
        _lib.check(lib.snntc_min_pool_backward(_ptr(grad_y), _ptr(arg), _ptr(dx), B, H, W, C, kernel[0], kernel[1],
                                               stride[0], stride[1], pad[0], pad[1], Nh, Nw, _stream(grad_y.device)))
    return dx


class SnnMinPool(torch.autograd.Function):
    """SNN_maxpool2d on device tensors: min over the (implicitly padded) window, gradient to the
    position that attained it."""

    @staticmethod
    def forward(ctx, x, kernel, stride, pad, out_hw, pad_value, next_xpad=None, next_offset=(0, 0)):
        y, arg = min_pool(x, kernel, stride, pad, out_hw, pad_value, want_arg=x.requires_grad, next_xpad=next_xpad,
                          next_offset=next_offset)
        ctx.geom = (tuple(x.shape), tuple(kernel), tuple(stride), tuple(pad))
        if arg is not None:
            ctx.save_for_backward(arg)
        ctx.has_arg = arg is not None
        return y

    @staticmethod
    def backward(ctx, grad_y):
        if not ctx.has_arg:
            return (None,) * 8
        (arg,) = ctx.saved_tensors
        in_shape, kernel, stride, pad = ctx.geom
        return (min_pool_grad(grad_y.contiguous(), arg, in_shape, kernel, stride, pad),) + (None,) * 7


def pad_time(x, top, bottom, left, right, value):
    """x[B,H,W,C] -> [B, top+H+bottom, left+W+right, C], the border filled with `value` (one pass)."""
    lib = _lib.load()
    x = _dev_f32(x, "x", 4)
    B, H, W, C = x.shape
    Hp, Wp = top + H + bottom, left + W + right
    with torch.cuda.device(x.device):
        xpad = torch.empty((B, Hp, Wp, C), dtype=torch.float32, device=x.device)
        _lib.check(lib.snntc_pad_time_forward(_ptr(x), _ptr(xpad), B, H, W, C, top, left, Hp, Wp, float(value),
                                              _stream(x.device)))
    return xpad


def pad_time_grad(dxpad, in_shape, top, left):
    """The gradient of pad_time: the H x W interior of dxpad."""
    lib = _lib.load()
    dxpad = _dev_f32(dxpad, "dxpad", 4)
    B, H, W, C = in_shape
    with torch.cuda.device(dxpad.device):
        dx = torch.empty((B, H, W, C), dtype=torch.float32, device=dxpad.device)
        _lib.check(lib.snntc_pad_time_backward(_ptr(dxpad), _ptr(dx), B, H, W, C, top, left, dxpad.shape[1],
                                               dxpad.shape[2], _stream(dxpad.device)))
    return dx


class SnnPadTime(torch.autograd.Function):
    """SAME padding of a conv layer's input with MAX_SPIKE_TIME, one kernel each way."""

    @staticmethod
    def forward(ctx, x, top, bottom, left, right, value):
        ctx.geom = (tuple(x.shape), top, left)
        return pad_time(x, top, bottom, left, right, value)

    @staticmethod
    def backward(ctx, dxpad):
        in_shape, top, left = ctx.geom
        return (pad_time_grad(dxpad.contiguous(), in_shape, top, left),) + (None,) * 5

