"""The allocation-free dense forward entry point, snntc_fc_forward_static, called through the C ABI
(ctypes) and compared bit for bit with snntc_fc_forward: two calls in a row on the same GPU, the
second with a smaller input (the static scratch keeps the first call's contents), then a call at
the size limit and one past it."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import dense_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _forward_both(lib, x, w, p):
    """(static entry point, workspace entry point) outputs for the same inputs, raw C-ABI calls."""
    from snntc_amd import _lib
    X, W = t(x), t(w)
    B, I = x.shape
    rows, J = w.shape
    pp = p.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out_static = torch.full((2 * B, J), float("nan"), device=DEV)
    out_ws = torch.full((2 * B, J), float("nan"), device=DEV)
    _lib.check(lib.snntc_fc_forward_static(X.data_ptr(), W.data_ptr(), pp, out_static.data_ptr(), B, I, J, rows,
                                           stream))
    need = ctypes.c_size_t()
    _lib.check(lib.snntc_fc_forward_workspace_bytes(B, I, J, ctypes.byref(need)))
    ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=DEV)
    _lib.check(lib.snntc_fc_forward(X.data_ptr(), W.data_ptr(), pp, out_ws.data_ptr(), B, I, J, rows, ws.data_ptr(),
                                    ws.numel(), stream))
    torch.cuda.synchronize()
    return out_static.cpu().numpy(), out_ws.cpu().numpy()


def test_static_scratch_forward_matches_the_workspace_entry_point():
    from snntc_amd import _lib
    lib = _lib.load()
    limit = lib.snntc_static_scratch_bytes()
    assert limit == 8 << 20
    _lib.check(lib.snntc_init(-1))
    cases = [(0, 256, 784, 800, True),      # the north-star dense layer
             (1, 37, 150, 45, True),        # smaller rows and fewer of them: stale scratch beyond them
             (2, 64, 800, 10, False),       # classifier head (split scan kernel), no bias row
             (3, 5, 1, 3, True)]
    for seed, B, I, J, bias in cases:
        x, w, p, _ = dense_case(seed, B, I, J, bias, "baseline")
        got, want = _forward_both(lib, x, w, p)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"case {seed}: outputs differ"
        assert not np.isnan(got).any()
    # against the oracle too, on the second (smaller) call's shape
    from oracle import capi
    x, w, p, _ = dense_case(1, 37, 150, 45, True, "baseline")
    got, _ = _forward_both(lib, x, w, p)
    assert np.array_equal(got.view(np.uint32), capi.fc_forward_dev(x, w, p).view(np.uint32))


def test_static_scratch_forward_rejects_sizes_beyond_the_array():
    from snntc_amd import _lib
    lib = _lib.load()
    limit = lib.snntc_static_scratch_bytes()
    I = 784
    need = ctypes.c_size_t()
    B = 1
    while True:                               # largest batch whose workspace still fits
        _lib.check(lib.snntc_fc_forward_workspace_bytes(B + 1, I, 16, ctypes.byref(need)))
        if need.value > limit:
            break
        B += 1
    x, w, p, _ = dense_case(7, B, I, 16, True, "baseline")
    got, want = _forward_both(lib, x, w, p)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    x2 = np.concatenate((x, x[:1]))
    pp = p.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
    out = torch.empty((2 * (B + 1), 16), device=DEV)
    rc = lib.snntc_fc_forward_static(t(x2).data_ptr(), t(w).data_ptr(), pp, out.data_ptr(), B + 1, I, 16, I + 1, None)
    assert rc == _lib.ERR_WORKSPACE
    assert b"scratch" in lib.snntc_last_error()
