"""ctypes binding of ``libteletron_op.so`` (the C ABI declared in ``include/teletron_op.h``).

The library is loaded from inside the package directory, where
``python -m teletron_amd.build`` puts it.  There is no fallback: if it is missing,
or an entry point returns a non-zero status, a Python exception is raised.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p, POINTER
from pathlib import Path

LIB_NAME = "libteletron_op.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

TT_OK = 0
TT_ERR_INVALID_ARGUMENT = 1
TT_ERR_UNSUPPORTED = 2
TT_ERR_WORKSPACE = 3
TT_ERR_HIP = 4
TT_ERR_STATIC_LIMIT = 5
TT_STATIC_WORKSPACE_BYTES = 16 << 20


class TeletronOpError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""

    def __init__(self, func: str, code: int, message: str, hip_error: int = 0):
        self.func, self.code, self.hip_error = func, code, hip_error
        extra = f", hipError_t={hip_error}" if code == TT_ERR_HIP else ""
        super().__init__(f"{func} failed with status {code} ({message}{extra})")


# name -> (restype, argtypes); mirrors include/teletron_op.h declaration by declaration.
PROTOTYPES = {
    "tt_version": (c_int, []),
    "tt_error_string": (c_char_p, [c_int]),
    "tt_last_hip_error": (c_int, []),
    "tt_adaln_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_adaln_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_size_t, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_adaln_backward_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_adaln_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "tt_rmsnorm_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_size_t, c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_backward_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "tt_adaln_backward_partials": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_size_t, POINTER(c_int),
                                           c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_backward_partials": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_size_t, POINTER(c_int),
                                             c_int64, c_int64, c_float, c_void_p]),
    "tt_reduce_partials": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_void_p]),
    "tt_rmsnorm_rope_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_rope_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                         c_int64, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_rope_heads_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_int64, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_rmsnorm_rope_heads_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_size_t, c_int64, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_gate_residual_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "tt_gate_residual_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                          c_int64, c_int64, c_int64, c_void_p]),
    "tt_gate_residual_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "tt_residual_norm_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                         c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p,
                                         c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_residual_norm_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int64, c_void_p, c_int64, c_int,
                                          c_void_p, c_size_t, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "tt_residual_norm_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "tt_stream_probe": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tt_stream_probe_two_outputs": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "tt_launch_adaln_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int64, c_double, c_void_p, c_void_p]),
    "tt_launch_adaln_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "tt_launch_rms_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_double, c_void_p, c_void_p]),
    "tt_launch_rms_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
}

_lib = None
_lock = threading.Lock()


def load() -> ctypes.CDLL:
    """Load the shared library (once) and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: the HIP library has not been built. "
                "Run `python -m teletron_amd.build` (needs hipcc); there is no CPU fallback.")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(func: str, status: int) -> None:
    if status != TT_OK:
        lib = load()
        msg = lib.tt_error_string(status).decode()
        raise TeletronOpError(func, status, msg, lib.tt_last_hip_error())


def call(func: str, *args) -> None:
    """Call a status-returning entry point and raise on failure."""
    check(func, getattr(load(), func)(*args))
