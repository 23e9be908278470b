"""ctypes front end of the CPU checker in ``tftq_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The shipped package
(``torchft_amd``) never imports this module.

The functions take and return CPU torch tensors and mirror the signatures of
``torchft/quantization.py:531-686`` so that tests read like the reference's.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtftq_oracle.so")

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def build(force: bool = False) -> str:
    """Compile the checker with gcc (always when ``force``)."""
    src = os.path.join(_HERE, "tftq_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libtftq_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.tftq_oracle_scale.restype = ctypes.c_float
        L.tftq_oracle_scale.argtypes = [ctypes.c_float]
        L.tftq_oracle_e4m3_to_f32.restype = ctypes.c_float
        L.tftq_oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.tftq_oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.tftq_oracle_f32_to_e4m3.argtypes = [ctypes.c_float]
        L.tftq_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.tftq_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.tftq_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.tftq_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.tftq_oracle_f16_to_f32.restype = ctypes.c_float
        L.tftq_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.tftq_oracle_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def max_threads() -> int:
    return int(lib().tftq_oracle_max_threads())


def _as_2d(inputs: list[torch.Tensor]) -> None:
    # quantization.py:487-488 -- the caller's list is updated in place
    for i in range(len(inputs)):
        if inputs[i].dim() == 1:
            inputs[i] = inputs[i].unsqueeze(1)
        assert inputs[i].dim() == 2, "Only 2D tensors are supported"


def _tables(inputs: Sequence[torch.Tensor]):
    T = len(inputs)
    shapes = (ctypes.c_int64 * (2 * T))()
    strides = (ctypes.c_int64 * (2 * T))()
    ptrs = (ctypes.c_void_p * T)()
    for i, t in enumerate(inputs):
        assert t.device.type == "cpu"
        shapes[2 * i], shapes[2 * i + 1] = t.shape
        strides[2 * i], strides[2 * i + 1] = t.stride()
        ptrs[i] = t.data_ptr()
    return T, ptrs, shapes, strides


def layout(shapes2d: Sequence[tuple[int, int]], ws: int):
    """-> (slot_offsets, slot_size, output_size)."""
    T = len(shapes2d)
    sh = (ctypes.c_int64 * (2 * T))()
    for i, (m, n) in enumerate(shapes2d):
        sh[2 * i], sh[2 * i + 1] = m, n
    off = (ctypes.c_int64 * T)()
    slot = ctypes.c_int64()
    total = ctypes.c_int64()
    rc = lib().tftq_oracle_layout(T, sh, ws, off, ctypes.byref(slot), ctypes.byref(total))
    assert rc == 0
    return list(off), slot.value, total.value


def fused_quantize_into_fp8(inputs: list[torch.Tensor], all_reduce_group_size: int,
                            nthreads: int = 1) -> torch.Tensor:
    assert len(inputs) > 0, "At least one input tensor is required"
    _as_2d(inputs)
    dtype = inputs[0].dtype
    T, ptrs, shapes, strides = _tables(inputs)
    _, _, total = layout([tuple(t.shape) for t in inputs], all_reduce_group_size)
    out = torch.empty(total, dtype=torch.uint8)
    rc = lib().tftq_oracle_quantize(DTYPE_CODE[dtype], T, ptrs, shapes, strides,
                                    all_reduce_group_size,
                                    ctypes.c_void_p(out.data_ptr()), nthreads)
    assert rc == 0
    return out


def fused_reduce_fp8(inputs: list[torch.Tensor], output: torch.Tensor,
                     all_reduce_group_size: int, all_reduce_rank: int,
                     reduce_op=None, nthreads: int = 1) -> None:
    from torch.distributed import ReduceOp

    _as_2d(inputs)
    T, _, shapes, _ = _tables(inputs)
    _, _, total = layout([tuple(t.shape) for t in inputs], all_reduce_group_size)
    assert output.shape[0] == total, "Output size does not match"
    assert output.dtype == torch.uint8 and output.is_contiguous()
    is_avg = 0 if (reduce_op is None or reduce_op == ReduceOp.SUM) else 1
    rc = lib().tftq_oracle_reduce(T, shapes, all_reduce_group_size, all_reduce_rank, is_avg,
                                  ctypes.c_void_p(output.data_ptr()), nthreads)
    assert rc == 0


def fused_dequantize_from_fp8(inputs: list[torch.Tensor], output: torch.Tensor,
                              all_reduce_group_size: int, nthreads: int = 1) -> None:
    _as_2d(inputs)
    dtype = inputs[0].dtype
    T, ptrs, shapes, strides = _tables(inputs)
    _, _, total = layout([tuple(t.shape) for t in inputs], all_reduce_group_size)
    assert output.shape[0] == total, "Output size does not match"
    assert output.dtype == torch.uint8 and output.is_contiguous()
    rc = lib().tftq_oracle_dequantize(DTYPE_CODE[dtype], T, ptrs, shapes, strides,
                                      all_reduce_group_size,
                                      ctypes.c_void_p(output.data_ptr()), nthreads)
    assert rc == 0
