"""CPU-side checks of libtftq.so: it loads, exports every symbol that
include/tftq.h declares, and its host-only entry points (layout, plan) agree
with the closed forms and with the CPU checker.  No kernel is launched."""

import ctypes
import os
import re

import pytest
import torch

from torchft_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_exported():
    hdr = open(os.path.join(ROOT, "include", "tftq.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(tftq_[a-z_0-9]+)\s*\(", hdr))
    assert len(declared) >= 14
    L = _lib.load()
    for name in declared:
        assert hasattr(L, name), f"{name} declared in tftq.h but not exported"
    assert declared == {n for n, _, _ in _lib.SYMBOLS}
    assert L.tftq_version() == 2
    assert re.fullmatch(r"[0-9a-f]{16}|unknown", L.tftq_build_id().decode())


def _layout(shapes, ws):
    L = _lib.load()
    T = len(shapes)
    sh = (ctypes.c_int64 * (2 * T))(*[v for s in shapes for v in s])
    off = (ctypes.c_int64 * T)()
    slot, total = ctypes.c_int64(), ctypes.c_int64()
    rc = L.tftq_layout(T, sh, ws, off, ctypes.byref(slot), ctypes.byref(total))
    return rc, list(off), slot.value, total.value


def test_layout_closed_forms(oracle):
    assert _layout([(256, 512), (1024, 1)], 2) == (0, [0, 66048], 70144, 140288)
    assert _layout([(5, 3), (1, 7)], 4) == (0, [0, 16], 28, 112)
    g = torch.Generator().manual_seed(0)
    for _ in range(100):
        T = int(torch.randint(1, 8, (1,), generator=g))
        ws = int(torch.randint(1, 17, (1,), generator=g))
        shapes = [(int(torch.randint(0, 5000, (1,), generator=g)),
                   int(torch.randint(0, 5000, (1,), generator=g))) for _ in range(T)]
        rc, off, slot, total = _layout(shapes, ws)
        assert rc == 0 and (off, slot, total) == oracle.layout(shapes, ws)


def test_layout_errors():
    assert _layout([(1, 1)], 0)[0] == -1
    assert _layout([(-1, 1)], 2)[0] == -3
    assert _layout([(1, 2 ** 31)], 2)[0] == -3


def _plan(dtype, shapes, strides, ws):
    L = _lib.load()
    T = len(shapes)
    sh = (ctypes.c_int64 * (2 * T))(*[v for s in shapes for v in s])
    st = (ctypes.c_int64 * (2 * T))(*[v for s in strides for v in s])
    h = ctypes.c_void_p()
    rc = L.tftq_plan_create(dtype, T, sh, st, ws, ctypes.byref(h))
    return rc, h


def test_plan_sizes_and_table():
    L = _lib.load()
    rc, h = _plan(2, [(4096, 4096)], [(4096, 1)], 8)
    assert rc == 0
    assert L.tftq_plan_output_size(h) == 16793600
    assert L.tftq_plan_slot_size(h) == 2099200
    assert L.tftq_plan_max_rows(h) == 4096
    assert L.tftq_plan_table_bytes(h) == 0  # short lists travel in the kernel arguments
    L.tftq_plan_destroy(h)
    shapes = [(3, 5)] * 40
    rc, h = _plan(0, shapes, [(5, 1)] * 40, 4)
    assert rc == 0
    # 40 descriptors of 64 bytes, then the per-stage lookup tables
    assert L.tftq_plan_table_bytes(h) > 40 * 64 and L.tftq_plan_table_bytes(h) % 8 == 0
    assert L.tftq_plan_table_host(h)
    assert L.tftq_plan_max_rows(h) == 4
    assert L.tftq_plan_n_tensors(h) == 40
    # the image holds no address: the first descriptor's pointer field is zero
    assert ctypes.cast(L.tftq_plan_table_host(h), ctypes.POINTER(ctypes.c_uint64))[0] == 0
    # without the device table the compute entry points refuse instead of launching
    buf = (ctypes.c_uint8 * L.tftq_plan_output_size(h))()
    assert L.tftq_quantize(h, None, None, None, buf, len(buf), -1, None) == -6
    assert L.tftq_reduce(h, None, buf, len(buf), 0, 0, -1, None) == -6
    assert L.tftq_quantize(h, None, None, None, buf, len(buf) - 4, -1, None) == -4
    L.tftq_plan_destroy(h)
    # a short list needs its tensors' addresses
    rc, h = _plan(2, [(8, 64)], [(64, 1)], 2)
    buf = (ctypes.c_uint8 * L.tftq_plan_output_size(h))()
    assert L.tftq_quantize(h, None, None, None, buf, len(buf), -1, None) == -1
    assert L.tftq_quantize(h, (ctypes.c_void_p * 1)(None), None, None, buf, len(buf), -1, None) == -1
    L.tftq_plan_destroy(h)


def test_plan_errors():
    assert _plan(3, [(1, 1)], [(1, 1)], 2)[0] == -2
    assert _plan(0, [(1, 1)], [(1, 1)], 0)[0] == -1
    assert b"fp32, fp16 and bf16" in _lib.load().tftq_strerror(-2)
    assert b"Output size does not match" == _lib.load().tftq_strerror(-4)


def test_plan_rejects_grids_the_hardware_cannot_launch():
    """A grid has fewer than 2^32 threads = 2^24 workgroups of 256.  Rows of 640 fp32
    columns are quantized and dequantized by 32 lanes each, eight to a workgroup."""
    rc, h = _plan(0, [(8 * (2 ** 24 - 64), 640)], [(640, 1)], 1)
    assert rc == 0
    _lib.load().tftq_plan_destroy(h)
    assert _plan(0, [(8 * 2 ** 24 + 64, 640)], [(640, 1)], 1)[0] == -3
    # the same rows spread over 20 tensors (device table): rejected as well
    assert _plan(0, [((8 * 2 ** 24) // 20 + 64, 640)] * 20, [(640, 1)] * 20, 1)[0] == -3
    # rows of 600 columns do not end on 64-byte boundaries: dequantize takes four to a workgroup
    assert _plan(0, [(4 * 2 ** 24 + 64, 600)], [(600, 1)], 1)[0] == -3


def test_host_wrapper_validation_messages():
    """Same assertion texts as torchft/quantization.py:463-489."""
    from torchft_amd import quantization as q
    with pytest.raises(AssertionError, match="At least one input tensor is required"):
        q.fused_quantize_into_fp8([], 2)
    with pytest.raises(AssertionError, match="same dtype"):
        q.fused_quantize_into_fp8([torch.zeros(2, 2), torch.zeros(2, 2, dtype=torch.bfloat16)], 2)
    with pytest.raises(AssertionError, match="Only fp32, fp16 and bf16 are supported"):
        q.fused_quantize_into_fp8([torch.zeros(2, 2, dtype=torch.float64)], 2)
    with pytest.raises(AssertionError, match="Only 2D tensors are supported"):
        q.fused_quantize_into_fp8([torch.zeros(2, 2, 2)], 2)
    ins = [torch.zeros(6)]
    with pytest.raises(RuntimeError, match="no CPU path"):
        q.fused_quantize_into_fp8(ins, 2)
    assert ins[0].shape == (6, 1)  # the caller's list is updated like the reference does
