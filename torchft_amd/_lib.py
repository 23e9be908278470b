"""ctypes binding of ``libtftq.so`` (the C ABI declared in ``include/tftq.h``)."""

from __future__ import annotations

import ctypes
import os
import threading

from . import _build

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None

ERR_NAMES = {
    -1: "TFTQ_E_ARG", -2: "TFTQ_E_DTYPE", -3: "TFTQ_E_SHAPE", -4: "TFTQ_E_SIZE",
    -5: "TFTQ_E_NOMEM", -6: "TFTQ_E_NOTABLE", -7: "TFTQ_E_ARCH",
}

# every symbol that include/tftq.h declares: (name, restype, argtypes)
_c = ctypes
SYMBOLS = [
    ("tftq_version", _c.c_int, []),
    ("tftq_strerror", _c.c_char_p, [_c.c_int]),
    ("tftq_check_device", _c.c_int, []),
    ("tftq_layout", _c.c_int, [_c.c_int, _c.POINTER(_c.c_int64), _c.c_int,
                               _c.POINTER(_c.c_int64), _c.POINTER(_c.c_int64),
                               _c.POINTER(_c.c_int64)]),
    ("tftq_plan_create", _c.c_int, [_c.c_int, _c.c_int, _c.POINTER(_c.c_void_p),
                                    _c.POINTER(_c.c_int64), _c.POINTER(_c.c_int64), _c.c_int,
                                    _c.POINTER(_c.c_void_p)]),
    ("tftq_plan_destroy", None, [_c.c_void_p]),
    ("tftq_plan_output_size", _c.c_int64, [_c.c_void_p]),
    ("tftq_plan_slot_size", _c.c_int64, [_c.c_void_p]),
    ("tftq_plan_max_rows", _c.c_int64, [_c.c_void_p]),
    ("tftq_plan_table_bytes", _c.c_int64, [_c.c_void_p]),
    ("tftq_plan_table_host", _c.c_void_p, [_c.c_void_p]),
    ("tftq_plan_set_device_table", _c.c_int, [_c.c_void_p, _c.c_void_p]),
    ("tftq_quantize", _c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p]),
    ("tftq_reduce", _c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_int,
                               _c.c_void_p]),
    ("tftq_dequantize", _c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p]),
    ("tftq_dequantize_scaled", _c.c_int,
     [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_float, _c.c_void_p]),
]


def lib_path() -> str:
    """Path of the shared library; ``TFTQ_LIB`` overrides the in-tree build."""
    return os.environ.get("TFTQ_LIB") or _build.LIB_PATH


def load() -> ctypes.CDLL:
    """Load the built library; build it first only if no build exists.

    Raises if the library can be neither found nor built: there is no fallback
    implementation.
    """
    global _lib
    with _lock:
        if _lib is None:
            path = lib_path()
            if not os.path.exists(path):
                _build.build_library()
            L = ctypes.CDLL(path)
            for name, restype, argtypes in SYMBOLS:
                fn = getattr(L, name)  # AttributeError if the export is missing
                fn.restype = restype
                fn.argtypes = argtypes
            if L.tftq_version() != 1:
                raise RuntimeError(f"libtftq.so version {L.tftq_version()} != 1")
            _lib = L
        return _lib


def strerror(code: int) -> str:
    if code > 0:
        return f"hipError_t {code}"
    return f"{ERR_NAMES.get(code, code)}: {load().tftq_strerror(code).decode()}"
