"""Loader and raw bindings of ``libsnntc_hip.so`` (C ABI declared in ``include/snntc.h``).

The library is looked up next to the HIP sources (``snntc-2023_amd/csrc/libsnntc_hip.so``, built
in-tree by ``make -C snntc-2023_amd/csrc``) or at ``$SNNTC_HIP_LIB``.  There is no CPU fallback:
if the library is missing, loading raises ``SnntcLibraryError``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "csrc"))
DEFAULT_LIB = os.path.join(CSRC_DIR, "libsnntc_hip.so")

OK = 0
ERR_DIM_MISMATCH = 1
ERR_TOO_LARGE = 2
ERR_BAD_ARGUMENT = 3
ERR_WORKSPACE = 4
ERR_UNSUPPORTED = 5
ERR_HIP = 6

#: every symbol include/snntc.h declares
EXPORTS = (
    "snntc_version", "snntc_last_error", "snntc_status_string", "snntc_init",
    "snntc_static_scratch_bytes", "snntc_fc_forward_static",
    "snntc_fc_forward_workspace_bytes", "snntc_fc_backward_workspace_bytes",
    "snntc_fc_forward", "snntc_fc_forward_ex", "snntc_fc_backward",
    "snntc_cv_output_dims", "snntc_cv_forward_workspace_bytes", "snntc_cv_backward_workspace_bytes",
    "snntc_cv_forward", "snntc_cv_forward_ex", "snntc_cv_forward_chained", "snntc_cv_backward",
    "snntc_cv_backward_cropped", "snntc_min_pool_forward_chained",
    "snntc_softmax_time_loss", "snntc_sgd_update",
    "snntc_min_pool_forward", "snntc_min_pool_backward",
    "snntc_pad_time_forward", "snntc_pad_time_backward",
    "snntc_scan_status", "snntc_debug_set_scan_wait_polls",
    "snntc_profile_enable", "snntc_profile_collect", "snntc_profile_entry",
)


class SnntcLibraryError(RuntimeError):
    """The HIP library is missing or does not export the expected ABI."""


class SnntcError(RuntimeError):
    """A library call failed with a non-argument error (workspace, HIP runtime, unsupported size)."""

    def __init__(self, status, message):
        super().__init__(f"snntc status {status}: {message}")
        self.status = status


_lib = None


def lib_path():
    return os.environ.get("SNNTC_HIP_LIB", DEFAULT_LIB)


def load():
    """Returns the ctypes handle, loading and prototyping the library on first use."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise SnntcLibraryError(
            f"{path} not found: build it with `make -C {CSRC_DIR}` (hipcc, --offload-arch=gfx950). "
            "There is no CPU fallback for the SNN-TC ops.")
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:  # missing ROCm runtime etc.
        raise SnntcLibraryError(f"cannot load {path}: {e}") from e
    missing = [s for s in EXPORTS if not hasattr(lib, s)]
    if missing:
        raise SnntcLibraryError(f"{path} lacks symbols {missing}")

    c = ctypes
    vp, i64, sz = c.c_void_p, c.c_int64, c.c_size_t
    fparams = c.POINTER(c.c_float)
    lib.snntc_version.restype = c.c_char_p
    lib.snntc_last_error.restype = c.c_char_p
    lib.snntc_status_string.restype = c.c_char_p
    lib.snntc_status_string.argtypes = [c.c_int]
    lib.snntc_init.argtypes = [c.c_int]
    lib.snntc_static_scratch_bytes.argtypes = []
    lib.snntc_fc_forward_static.argtypes = [vp, vp, fparams, vp, i64, i64, i64, i64, vp]
    lib.snntc_fc_forward_workspace_bytes.argtypes = [i64, i64, i64, c.POINTER(sz)]
    lib.snntc_fc_backward_workspace_bytes.argtypes = [i64, i64, i64, c.POINTER(sz)]
    lib.snntc_fc_forward.argtypes = [vp, vp, fparams, vp, i64, i64, i64, i64, vp, sz, vp]
    lib.snntc_fc_forward_ex.argtypes = [vp, vp, fparams, vp, vp, vp, vp, i64, i64, i64, i64, vp, sz, vp]
    lib.snntc_fc_backward.argtypes = [vp, vp, vp, fparams, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, sz, vp]
    lib.snntc_cv_output_dims.argtypes = [i64, i64, fparams, c.POINTER(i64), c.POINTER(i64)]
    lib.snntc_cv_forward_workspace_bytes.argtypes = [i64, i64, i64, i64, i64, fparams, c.POINTER(sz)]
    lib.snntc_cv_backward_workspace_bytes.argtypes = [i64, i64, i64, i64, i64, fparams, c.POINTER(sz)]
    lib.snntc_cv_forward.argtypes = [vp, vp, fparams, vp, i64, i64, i64, i64, i64, i64, vp, sz, vp]
    lib.snntc_cv_forward_ex.argtypes = [vp, vp, fparams, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, sz, vp]
    lib.snntc_cv_backward.argtypes = [vp, vp, vp, fparams, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64,
                                      vp, sz, vp]
    lib.snntc_cv_forward_chained.argtypes = [vp, vp, fparams, vp, vp] + [i64] * 10 + [vp, sz, vp]
    lib.snntc_cv_backward_cropped.argtypes = [vp, vp, vp, fparams, vp, vp, i64, i64, i64, i64, vp, vp] + [i64] * 7 + [
        vp, sz, vp]
    lib.snntc_min_pool_forward_chained.argtypes = [vp, vp, vp, vp] + [i64] * 16 + [c.c_float, vp]
    lib.snntc_softmax_time_loss.argtypes = [vp, vp, vp, vp, i64, i64, vp]
    lib.snntc_sgd_update.argtypes = [c.POINTER(vp), c.POINTER(vp), c.POINTER(i64), i64, c.c_float, vp]
    lib.snntc_min_pool_forward.argtypes = [vp, vp, vp] + [i64] * 12 + [c.c_float, vp]
    lib.snntc_min_pool_backward.argtypes = [vp, vp, vp] + [i64] * 12 + [vp]
    lib.snntc_pad_time_forward.argtypes = [vp, vp] + [i64] * 8 + [c.c_float, vp]
    lib.snntc_pad_time_backward.argtypes = [vp, vp] + [i64] * 8 + [vp]
    lib.snntc_scan_status.argtypes = [c.POINTER(i64), vp]
    lib.snntc_debug_set_scan_wait_polls.argtypes = [c.c_int]
    lib.snntc_profile_enable.argtypes = [c.c_int]
    lib.snntc_profile_collect.argtypes = []
    lib.snntc_profile_entry.argtypes = [c.c_int, c.POINTER(c.c_char_p), c.POINTER(i64), c.POINTER(c.c_double)]
    for name in EXPORTS:
        if name not in ("snntc_version", "snntc_last_error", "snntc_status_string", "snntc_static_scratch_bytes"):
            getattr(lib, name).restype = c.c_int
    lib.snntc_static_scratch_bytes.restype = sz
    _lib = lib
    return lib


def check(status):
    """Maps a status code to the exception the reference's Python caller would see:
    InvalidArgument conditions -> ValueError, everything else -> SnntcError."""
    if status == OK:
        return
    msg = load().snntc_last_error().decode("utf-8", "replace")
    if status in (ERR_DIM_MISMATCH, ERR_TOO_LARGE, ERR_BAD_ARGUMENT):
        raise ValueError(msg)
    raise SnntcError(status, msg)


def profile_enable(on=True):
    """Switches the library's per-kernel event timing on (clearing the totals) or off."""
    check(load().snntc_profile_enable(1 if on else 0))


def profile_collect():
    """Waits for the timed launches and returns {kernel name: (launches, total milliseconds)}."""
    lib = load()
    n = lib.snntc_profile_collect()
    out = {}
    for i in range(n):
        name, cnt, ms = ctypes.c_char_p(), ctypes.c_int64(), ctypes.c_double()
        check(lib.snntc_profile_entry(i, ctypes.byref(name), ctypes.byref(cnt), ctypes.byref(ms)))
        out[name.value.decode()] = (cnt.value, ms.value)
    return out


def scan_giveups(stream=None):
    """Wavefronts of the classifier-head scan whose bounded wait ran out on the current device since the
    process started (each leaves NaN in the outputs of its work item).  Waits for `stream`."""
    n = ctypes.c_int64()
    check(load().snntc_scan_status(ctypes.byref(n), ctypes.c_void_p(stream or 0)))
    return n.value


def set_scan_wait_polls(polls):
    """Test hook: polls a waiting scan wavefront spends from the next launch on (< 0: the default)."""
    check(load().snntc_debug_set_scan_wait_polls(int(polls)))
