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
    -5: "TFTQ_E_NOMEM", -6: "TFTQ_E_NOTABLE", -7: "TFTQ_E_ARCH", -8: "TFTQ_E_TOOBIG", -9: "TFTQ_E_BUSY",
}

# every symbol that include/tftq.h declares: (name, restype, argtypes)
_c = ctypes
_P = _c.c_void_p
SYMBOLS = [
    ("tftq_version", _c.c_int, []),
    ("tftq_build_id", _c.c_char_p, []),
    ("tftq_strerror", _c.c_char_p, [_c.c_int]),
    ("tftq_check_device", _c.c_int, [_c.c_int]),
    ("tftq_layout", _c.c_int, [_c.c_int, _c.POINTER(_c.c_int64), _c.c_int,
                               _c.POINTER(_c.c_int64), _c.POINTER(_c.c_int64),
                               _c.POINTER(_c.c_int64)]),
    ("tftq_plan_create", _c.c_int, [_c.c_int, _c.c_int, _c.POINTER(_c.c_int64), _c.POINTER(_c.c_int64),
                                    _c.c_int, _c.POINTER(_P)]),
    ("tftq_plan_destroy", None, [_P]),
    ("tftq_plan_output_size", _c.c_int64, [_P]),
    ("tftq_plan_slot_size", _c.c_int64, [_P]),
    ("tftq_plan_max_rows", _c.c_int64, [_P]),
    ("tftq_plan_n_tensors", _c.c_int, [_P]),
    ("tftq_plan_table_bytes", _c.c_int64, [_P]),
    ("tftq_plan_table_host", _P, [_P]),
    ("tftq_upload_pointers", _c.c_int, [_P, _P, _P, _c.c_int, _P]),
    # plan, tensors, table, pointers, packed, packed_bytes, device, stream
    ("tftq_quantize", _c.c_int, [_P, _P, _P, _P, _P, _c.c_int64, _c.c_int, _P]),
    # plan, table, packed, packed_bytes, rank, is_avg, device, stream
    ("tftq_reduce", _c.c_int, [_P, _P, _P, _c.c_int64, _c.c_int, _c.c_int, _c.c_int, _P]),
    ("tftq_dequantize", _c.c_int, [_P, _P, _P, _P, _P, _c.c_int64, _c.c_int, _P]),
    ("tftq_dequantize_scaled", _c.c_int, [_P, _P, _P, _P, _P, _c.c_int64, _c.c_float, _c.c_int, _P]),
    # plan, packed, packed_bytes, rank, is_avg, device, stream
    ("tftq_reduce_static", _c.c_int, [_P, _P, _c.c_int64, _c.c_int, _c.c_int, _c.c_int, _P]),
]
ABI_VERSION = 2


def lib_path() -> str:
    """Path of the shared library; ``TFTQ_LIB`` overrides the in-tree build."""
    return os.environ.get("TFTQ_LIB") or _build.LIB_PATH


def load() -> ctypes.CDLL:
    """Load the built library; build it first only if no build exists.

    Raises if the library can be neither found nor built, or if the in-tree
    library was built from other sources than the ones beside it (its build id is
    a hash of them; rebuild with ``python -m torchft_amd._build``): there is no
    fallback implementation, and a stale library is not used silently.
    ``TFTQ_LIB`` names a library to load as it is.
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
            if L.tftq_version() != ABI_VERSION:
                raise RuntimeError(f"libtftq.so version {L.tftq_version()} != {ABI_VERSION}")
            if path == _build.LIB_PATH and not os.environ.get("TFTQ_ALLOW_STALE"):
                built_from, here = L.tftq_build_id().decode(), _build.source_hash()
                if built_from != here:
                    raise RuntimeError(
                        f"{path} was built from other sources (build id {built_from}, sources {here}); "
                        "rebuild it with `python -m torchft_amd._build` (TFTQ_ALLOW_STALE=1 loads it anyway)")
            _lib = L
        return _lib


_checked_devices: set[int] = set()


def check_device(index: int) -> None:
    """Raises unless device `index` is a gfx950 GPU (checked once per device)."""
    if index in _checked_devices:
        return
    rc = load().tftq_check_device(int(index))
    if rc != 0:
        raise RuntimeError(f"cuda:{index} cannot run the tftq kernels: {strerror(rc)}")
    _checked_devices.add(index)


def strerror(code: int) -> str:
    if code > 0:
        return f"hipError_t {code}"
    return f"{ERR_NAMES.get(code, code)}: {load().tftq_strerror(code).decode()}"
