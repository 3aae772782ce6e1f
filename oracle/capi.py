"""ctypes/numpy binding of ``libsnntc_oracle.so`` (the C restatement in ``snntc_oracle.c``).

Test infrastructure only.  Every function takes and returns C-contiguous numpy arrays (float32 /
int32) with the tensor contracts of the reference ops:

* dense  : x[B,I], w[I+bias,J], params[6]  -> out[2B,J]
* conv   : xpad[B,H,W,C], w[Kh*Kw*C+bias,Kc], params[12] -> out[2B,Nh,Nw,Kc]

``*_dev`` = semantics of the reference's GPU kernels (the op contract), ``*_host`` = semantics of
the reference's single-threaded CPU functors (the timed CPU baseline).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsnntc_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64 = ctypes.c_int64


def build(force=False):
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _f(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _i(a):
    return None if a is None else a.ctypes.data_as(_i32p)


def _c32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _check(rc, name):
    if rc != 0:
        raise MemoryError(f"oracle {name} failed with code {rc}")


def sort_segments(x):
    """Stable ascending sort of every row of x[S,I] -> (sorted[S,I], perm[S,I] int32)."""
    x = _c32(x)
    S, I = x.shape
    sorted_ = np.empty((S, I), np.float32)
    perm = np.empty((S, I), np.int32)
    _check(lib().snntc_oracle_sort_segments(_f(x), _i64(S), _i64(I), _f(sorted_), _i(perm)), "sort")
    return sorted_, perm


def fc_forward_dev(x, w, params, want_aux=False):
    x, w, params = _c32(x), _c32(w), _c32(params)
    B, I = x.shape
    J = w.shape[1]
    out = np.empty((2 * B, J), np.float32)
    k = np.empty((B, J), np.int32) if want_aux else None
    sorted_ = np.empty((B, I), np.float32) if want_aux else None
    perm = np.empty((B, I), np.int32) if want_aux else None
    _check(lib().snntc_oracle_fc_forward_dev(_f(x), _f(w), _f(params), _f(out), _i(k), _f(sorted_),
                                             _i(perm), _i64(B), _i64(I), _i64(J)), "fc_forward_dev")
    return (out, k, sorted_, perm) if want_aux else out


def fc_forward_host(x, w, params):
    x, w, params = _c32(x), _c32(w), _c32(params)
    B, I = x.shape
    J = w.shape[1]
    out = np.empty((2 * B, J), np.float32)
    _check(lib().snntc_oracle_fc_forward_host(_f(x), _f(w), _f(params), _f(out), _i64(B), _i64(I),
                                              _i64(J)), "fc_forward_host")
    return out


def fc_backward_dev(grad, x, w, params, oldout, wide=False):
    grad, x, w, params, oldout = map(_c32, (grad, x, w, params, oldout))
    B, I = x.shape
    J = w.shape[1]
    dx = np.empty((B, I), np.float32)
    dw = np.zeros_like(w)
    dp = np.empty(6, np.float32)
    _check(lib().snntc_oracle_fc_backward_dev(_f(grad), _f(x), _f(w), _f(params), _f(oldout), _f(dx),
                                              _f(dw), _f(dp), _i64(B), _i64(I), _i64(J),
                                              ctypes.c_int(int(wide))), "fc_backward_dev")
    return dx, dw, dp


def fc_backward_host(grad, x, w, params, oldout):
    grad, x, w, params, oldout = map(_c32, (grad, x, w, params, oldout))
    B, I = x.shape
    J = w.shape[1]
    dx = np.empty((B, I), np.float32)
    dw = np.zeros_like(w)
    dp = np.zeros(6, np.float32)
    _check(lib().snntc_oracle_fc_backward_host(_f(grad), _f(x), _f(w), _f(params), _f(oldout), _f(dx),
                                               _f(dw), _f(dp), _i64(B), _i64(I), _i64(J)),
           "fc_backward_host")
    return dx, dw, dp


def cv_dims(xshape, params):
    B, H, W, C = xshape
    Kh, Kw, Sh, Sw = (int(params[t]) for t in (6, 7, 8, 9))
    return (H - Kh) // Sh + 1, (W - Kw) // Sw + 1, Kh * Kw * C


def im2col(xpad, params):
    xpad, params = _c32(xpad), _c32(params)
    B, H, W, C = xpad.shape
    Nh, Nw, P = cv_dims(xpad.shape, params)
    patches = np.empty((B * Nh * Nw, P), np.float32)
    _check(lib().snntc_oracle_im2col(_f(xpad), _f(params), _f(patches), _i64(B), _i64(H), _i64(W),
                                     _i64(C)), "im2col")
    return patches


def cv_forward_dev(xpad, w, params, want_aux=False):
    xpad, w, params = _c32(xpad), _c32(w), _c32(params)
    B, H, W, C = xpad.shape
    Kc = w.shape[1]
    Nh, Nw, P = cv_dims(xpad.shape, params)
    S = B * Nh * Nw
    out = np.empty((2 * B, Nh, Nw, Kc), np.float32)
    k = np.empty((S, Kc), np.int32) if want_aux else None
    sorted_ = np.empty((S, P), np.float32) if want_aux else None
    perm = np.empty((S, P), np.int32) if want_aux else None
    _check(lib().snntc_oracle_cv_forward_dev(_f(xpad), _f(w), _f(params), _f(out), _i(k), _f(sorted_),
                                             _i(perm), _i64(B), _i64(H), _i64(W), _i64(C), _i64(Kc)),
           "cv_forward_dev")
    return (out, k, sorted_, perm) if want_aux else out


def cv_forward_host(xpad, w, params):
    """Returns only the first half [B,Nh,Nw,Kc]: the reference's CPU functor never writes the rest."""
    xpad, w, params = _c32(xpad), _c32(w), _c32(params)
    B, H, W, C = xpad.shape
    Kc = w.shape[1]
    Nh, Nw, _ = cv_dims(xpad.shape, params)
    out = np.empty((B, Nh, Nw, Kc), np.float32)
    _check(lib().snntc_oracle_cv_forward_host(_f(xpad), _f(w), _f(params), _f(out), _i64(B), _i64(H),
                                              _i64(W), _i64(C), _i64(Kc)), "cv_forward_host")
    return out


def cv_backward_dev(grad, xpad, w, params, oldout, wide=False):
    grad, xpad, w, params, oldout = map(_c32, (grad, xpad, w, params, oldout))
    B, H, W, C = xpad.shape
    Kc = w.shape[1]
    dx = np.empty_like(xpad)
    dw = np.zeros_like(w)
    dp = np.empty(12, np.float32)
    _check(lib().snntc_oracle_cv_backward_dev(_f(grad), _f(xpad), _f(w), _f(params), _f(oldout),
                                              _f(dx), _f(dw), _f(dp), _i64(B), _i64(H), _i64(W),
                                              _i64(C), _i64(Kc), ctypes.c_int(int(wide))),
           "cv_backward_dev")
    return dx, dw, dp


def cv_backward_host(grad, xpad, w, params, oldout):
    grad, xpad, w, params, oldout = map(_c32, (grad, xpad, w, params, oldout))
    B, H, W, C = xpad.shape
    Kc = w.shape[1]
    dx = np.empty_like(xpad)
    dw = np.zeros_like(w)
    dp = np.zeros(12, np.float32)
    _check(lib().snntc_oracle_cv_backward_host(_f(grad), _f(xpad), _f(w), _f(params), _f(oldout),
                                               _f(dx), _f(dw), _f(dp), _i64(B), _i64(H), _i64(W),
                                               _i64(C), _i64(Kc)), "cv_backward_host")
    return dx, dw, dp


def fc_params(biasvolt=1.0, max_time=1e5, eps=1e-10, theta=1.0, tpb=0, blocks=0):
    """Params vector of the dense op (SNN_TC_Modules.py:48-49)."""
    return np.array([max_time, eps, theta, tpb, blocks, biasvolt], np.float32)


def cv_params(Kh, Kw, Sh, Sw, same=True, biasvolt=1.0, max_time=1e5, eps=1e-10, theta=1.0,
              tpb=0, blocks=0):
    """Params vector of the conv op (SNN_TC_Modules.py:121-123)."""
    return np.array([max_time, tpb, blocks, eps, theta, 0, Kh, Kw, Sh, Sw, float(bool(same)),
                     biasvolt], np.float32)
