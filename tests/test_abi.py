"""The C-ABI library without a GPU: it loads, exports every symbol include/snntc.h declares, and its
argument checks (which run before any device work) return the codes that mirror the reference
OpKernels' InvalidArgument conditions."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from snntc_amd import _lib
    return _lib.load()


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "snntc.h")).read()
    return re.findall(r"SNNTC_API\s+(?:const\s+char\s*\*|int|size_t)\s+(snntc_\w+)\s*\(", text)


def test_header_and_loader_list_the_same_symbols():
    from snntc_amd import _lib
    declared = _declared_symbols()
    assert len(declared) >= 14
    assert sorted(declared) == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol(lib):
    for name in _declared_symbols():
        assert hasattr(lib, name), name
    assert lib.snntc_version().startswith(b"snntc-hip gfx950")
    assert lib.snntc_status_string(0) == b"ok"


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from snntc_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("SNNTC_HIP_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.SnntcLibraryError, match="no CPU fallback"):
        _lib.load()


def _fp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


FAKE = ctypes.c_void_p(0x1000)      # never dereferenced: every call below fails validation first


def test_fc_forward_argument_errors(lib):
    from snntc_amd import _lib
    p1 = np.array([1e5, 1e-10, 1, 0, 0, 1.0], np.float32)
    p0 = np.array([1e5, 1e-10, 1, 0, 0, 0.0], np.float32)
    # weight rows must be I or I+1 (snntc/snnfc_kernels.cc:171-172)
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p1), FAKE, 4, 10, 5, 12, FAKE, 1 << 20, None) == _lib.ERR_DIM_MISMATCH
    assert b"inner-dim mismatch" in lib.snntc_last_error()
    # rows must agree with the bias flag
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p1), FAKE, 4, 10, 5, 10, FAKE, 1 << 20, None) == _lib.ERR_DIM_MISMATCH
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 11, FAKE, 1 << 20, None) == _lib.ERR_DIM_MISMATCH
    # element counts beyond INT32_MAX (snntc/snnfc_kernels.cc:194-203)
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 1 << 22, 1024, 8, 1024, FAKE, 1 << 20, None) == _lib.ERR_TOO_LARGE
    assert b"input tensor" in lib.snntc_last_error()
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 1 << 21, 8, 1024, 8, FAKE, 1 << 20, None) == _lib.ERR_TOO_LARGE
    assert b"output tensor" in lib.snntc_last_error()
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 1, 8192, 1 << 19, 8192, FAKE, 1 << 20, None) == _lib.ERR_TOO_LARGE
    assert b"weight tensor" in lib.snntc_last_error()
    # segments longer than the largest supported one (2^24 inputs)
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 2, (1 << 24) + 1, 4, (1 << 24) + 1, FAKE, 1 << 20, None) == _lib.ERR_UNSUPPORTED
    # segments longer than one sorting network (8192) need room for the merge passes as well
    need_short, need_long = ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.snntc_fc_forward_workspace_bytes(2, 8192, 4, ctypes.byref(need_short)) == _lib.OK
    assert lib.snntc_fc_forward_workspace_bytes(2, 9000, 4, ctypes.byref(need_long)) == _lib.OK
    assert need_long.value >= need_short.value + 2 * 2 * 16384 * 8
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 2, 9000, 4, 9000, FAKE, need_short.value, None) == _lib.ERR_WORKSPACE
    # workspace: missing, misaligned, too small
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 10, None, 0, None) == _lib.ERR_WORKSPACE
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 10, ctypes.c_void_p(0x1010), 1 << 20, None) == _lib.ERR_WORKSPACE
    assert lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 10, FAKE, 16, None) == _lib.ERR_WORKSPACE
    assert lib.snntc_fc_forward(None, FAKE, _fp(p0), FAKE, 4, 10, 5, 10, FAKE, 1 << 20, None) == _lib.ERR_BAD_ARGUMENT
    assert lib.snntc_fc_forward(FAKE, FAKE, None, FAKE, 4, 10, 5, 10, FAKE, 1 << 20, None) == _lib.ERR_BAD_ARGUMENT


def test_fc_backward_argument_errors(lib):
    from snntc_amd import _lib
    p0 = np.array([1e5, 1e-10, 1, 0, 0, 0.0], np.float32)
    # grad must hold 2*B rows (snntc/snnfcgrad_kernels.cc:119-120)
    rc = lib.snntc_fc_backward(FAKE, FAKE, FAKE, _fp(p0), FAKE, FAKE, FAKE, None, 4, 10, 5, 10, 4, FAKE, 1 << 20, None)
    assert rc == _lib.ERR_DIM_MISMATCH and b"2 * batch" in lib.snntc_last_error()
    rc = lib.snntc_fc_backward(FAKE, FAKE, FAKE, _fp(p0), FAKE, FAKE, FAKE, None, 4, 10, 5, 9, 8, FAKE, 1 << 20, None)
    assert rc == _lib.ERR_DIM_MISMATCH


def test_cv_argument_errors_and_dims(lib):
    from snntc_amd import _lib
    p = np.array([1e5, 0, 0, 1e-10, 1, 0, 3, 3, 2, 2, 1, 1.0], np.float32)
    nh, nw = ctypes.c_int64(), ctypes.c_int64()
    assert lib.snntc_cv_output_dims(9, 11, _fp(p), ctypes.byref(nh), ctypes.byref(nw)) == 0
    assert (nh.value, nw.value) == ((9 - 3) // 2 + 1, (11 - 3) // 2 + 1)      # snntc/snncv_kernels.cc:215
    # weight rows must be Kh*Kw*C + bias (snntc/snncv_kernels.cc:218)
    rc = lib.snntc_cv_forward(FAKE, FAKE, _fp(p), FAKE, 2, 9, 11, 4, 8, 36, FAKE, 1 << 20, None)
    assert rc == _lib.ERR_DIM_MISMATCH and b"(bias)" in lib.snntc_last_error()
    # patch matrix beyond INT32_MAX (snntc/snncv_kernels.cc:237-238)
    p1 = p.copy(); p1[8] = p1[9] = 1
    rc = lib.snntc_cv_forward(FAKE, FAKE, _fp(p1), FAKE, 64, 258, 258, 64, 8, 577, FAKE, 1 << 20, None)
    assert rc == _lib.ERR_TOO_LARGE and b"patched tensor" in lib.snntc_last_error()
    # kernel larger than the image
    assert lib.snntc_cv_forward(FAKE, FAKE, _fp(p), FAKE, 2, 2, 11, 4, 8, 37, FAKE, 1 << 20, None) == _lib.ERR_BAD_ARGUMENT
    rc = lib.snntc_cv_backward(FAKE, FAKE, FAKE, _fp(p), FAKE, FAKE, FAKE, None, 2, 9, 11, 4, 8, 37, 2, FAKE, 1 << 20, None)
    assert rc == _lib.ERR_DIM_MISMATCH


def test_workspace_queries(lib):
    n = ctypes.c_size_t()
    assert lib.snntc_fc_forward_workspace_bytes(256, 784, 800, ctypes.byref(n)) == 0
    assert n.value >= 256 * 784 * 8 and n.value % 256 == 0
    assert lib.snntc_fc_backward_workspace_bytes(256, 784, 800, ctypes.byref(n)) == 0
    assert n.value >= (256 * 800 + 785 * 800) * 4      # the masked upstream gradient and the transposed weights
    p = np.array([1e5, 0, 0, 1e-10, 1, 0, 3, 3, 1, 1, 1, 1.0], np.float32)
    assert lib.snntc_cv_forward_workspace_bytes(64, 34, 34, 64, 64, _fp(p), ctypes.byref(n)) == 0
    assert n.value >= 64 * 32 * 32 * 576 * 8


def test_python_ops_map_status_to_exceptions():
    from snntc_amd import _lib
    lib = _lib.load()
    p0 = np.array([1e5, 1e-10, 1, 0, 0, 0.0], np.float32)
    rc = lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 12, FAKE, 1 << 20, None)
    with pytest.raises(ValueError, match="mismatch"):
        _lib.check(rc)
    rc = lib.snntc_fc_forward(FAKE, FAKE, _fp(p0), FAKE, 4, 10, 5, 10, None, 0, None)
    with pytest.raises(_lib.SnntcError):
        _lib.check(rc)


def test_loss_argument_errors(lib):
    one = ctypes.c_void_p(256)                     # never dereferenced: the checks come first
    assert lib.snntc_softmax_time_loss(one, one, one, one, -1, 4, None) == 3
    assert lib.snntc_softmax_time_loss(None, one, one, one, 2, 4, None) == 3
    assert lib.snntc_softmax_time_loss(one, one, None, None, 2, 4, None) == 3
    assert lib.snntc_softmax_time_loss(one, one, one, one, 1 << 20, 1 << 20, None) == 2
    assert lib.snntc_softmax_time_loss(one, one, one, one, 0, 4, None) == 0      # empty batch: nothing to do


def test_sgd_update_argument_errors(lib):
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    one = (vp * 2)(256, 256)                       # never dereferenced: the checks come first
    null_in = (vp * 2)(256, None)
    n = (i64 * 2)(4, 4)
    assert lib.snntc_sgd_update(one, one, n, -1, 0.1, None) == 3
    assert lib.snntc_sgd_update(None, one, n, 2, 0.1, None) == 3
    assert lib.snntc_sgd_update(one, one, None, 2, 0.1, None) == 3
    assert lib.snntc_sgd_update(one, one, (i64 * 2)(4, -4), 2, 0.1, None) == 3
    assert lib.snntc_sgd_update(null_in, one, n, 2, 0.1, None) == 3
    assert lib.snntc_sgd_update(one, null_in, n, 2, 0.1, None) == 3
    assert lib.snntc_sgd_update(None, None, None, 0, 0.1, None) == 0            # no tensors: nothing to do
    assert lib.snntc_sgd_update(null_in, null_in, (i64 * 2)(0, 0), 2, 0.1, None) == 0   # empty tensors are skipped


def test_chained_entry_points_check_their_windows(lib):
    from snntc_amd import _lib
    p = np.array([1e5, 0, 0, 1e-10, 1, 0, 3, 3, 1, 1, 1, 1.0], np.float32)      # 3x3, stride 1, SAME, bias
    # 6x6 padded input -> 4x4 output; a 5x5 destination at offset (1, 1) holds it, (2, 2) does not
    args = (2, 6, 6, 8, 16, 73, FAKE, 1 << 30, None)
    assert lib.snntc_cv_forward_chained(FAKE, FAKE, _fp(p), FAKE, None, 5, 5, 1, 1, *args) == _lib.ERR_BAD_ARGUMENT
    assert lib.snntc_cv_forward_chained(FAKE, FAKE, _fp(p), FAKE, FAKE, 5, 5, 2, 2, *args) == _lib.ERR_BAD_ARGUMENT
    assert b"does not fit" in lib.snntc_last_error()
    assert lib.snntc_cv_forward_chained(FAKE, FAKE, _fp(p), FAKE, FAKE, 5, 5, -1, 0, *args) == _lib.ERR_BAD_ARGUMENT
    # the gradient window has to lie inside the 6x6 padded image
    bargs = (FAKE, FAKE, 2, 6, 6, 8, 16, 73, 4, FAKE, 1 << 30, None)
    assert lib.snntc_cv_backward_cropped(FAKE, FAKE, FAKE, _fp(p), FAKE, FAKE, 4, 4, 3, 1, *bargs) == _lib.ERR_BAD_ARGUMENT
    assert b"does not lie inside" in lib.snntc_last_error()
    assert lib.snntc_cv_backward_cropped(FAKE, FAKE, FAKE, _fp(p), FAKE, FAKE, 4, 7, 0, 0, *bargs) == _lib.ERR_BAD_ARGUMENT
    # a window that fits passes on to the op's own checks (here: grad rows must be 2 * batch)
    bad_rows = (FAKE, FAKE, 2, 6, 6, 8, 16, 73, 3, FAKE, 1 << 30, None)
    assert lib.snntc_cv_backward_cropped(FAKE, FAKE, FAKE, _fp(p), FAKE, FAKE, 4, 4, 1, 1, *bad_rows) == _lib.ERR_DIM_MISMATCH
    # pooling: 4x4 image, 2x2/2 windows -> 2x2 output, which a 3x3 destination holds at (1, 1) only
    pool = (2, 4, 4, 8, 2, 2, 2, 2, 0, 0, 2, 2, ctypes.c_float(1e5), None)
    assert lib.snntc_min_pool_forward_chained(FAKE, FAKE, None, None, 3, 3, 1, 1, *pool) == _lib.ERR_BAD_ARGUMENT
    assert lib.snntc_min_pool_forward_chained(FAKE, FAKE, None, FAKE, 3, 3, 2, 1, *pool) == _lib.ERR_BAD_ARGUMENT
