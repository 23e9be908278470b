"""FP8 quantized-collective kernels: host side.

Drop-in for ``torchft/quantization.py``: the same three public functions with
the same positional signatures, the same packed-buffer layout and the same
assertion messages (quantization.py:463-489, 621, 672), backed by hand-written
gfx950 kernels in ``libtftq.so`` instead of Triton.  Differences a caller can
observe:

* only the fp8-e4m3fn / 448 branch exists (quantization.py:30-41; gfx950 reports
  capability (9, 5)); the int8 / 127 branch for older GPUs is not built;
* the packed buffer is allocated uninitialised and every byte of it is written
  by the quantize kernel, instead of ``torch.zeros`` plus a kernel
  (quantization.py:567-571); the bytes are identical;
* the per-call host work of ``_prepare_quantize_fp8`` (four device tables and
  five allocations per call, quantization.py:505-517) is replaced by a cached
  plan; lists of up to 16 tensors need no device metadata at all.

There is no CPU or eager fallback: without the HIP library and a gfx950 device
the functions raise.
"""

from __future__ import annotations

import ctypes
import gc
import math
import operator
import threading
from collections import OrderedDict

import torch
from torch.distributed import ReduceOp

from . import _lib

SCALE_DTYPE: torch.dtype = torch.float32
SCALE_DTYPE_BYTES: int = 4

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_TENSOR = torch.Tensor
_DTYPE_OF = operator.attrgetter("dtype")
# Plans are cached by (device, dtype, group size, addresses, shapes, strides).  The
# per-parameter all-reduce of a model has one single-tensor plan per parameter, so the
# cache holds thousands of small plans; long lists are bounded by their total length.
_PLAN_CACHE_SIZE = 4096
_PLAN_CACHE_TENSORS = 1 << 18


class _Plan:
    """Owns a ``tftq_plan`` and, for long tensor lists, its device table."""

    __slots__ = ("handle", "output_size", "slot_size", "max_rows", "table", "n_tensors", "_lib")

    def __init__(self, lib, handle, table, n_tensors):
        self._lib = lib
        self.handle = handle
        self.table = table
        self.n_tensors = n_tensors
        self.output_size = lib.tftq_plan_output_size(handle)
        self.slot_size = lib.tftq_plan_slot_size(handle)
        self.max_rows = lib.tftq_plan_max_rows(handle)

    def __del__(self):
        try:
            if self.handle:
                self._lib.tftq_plan_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


_cache_lock = threading.Lock()
_plan_cache: "OrderedDict[tuple, _Plan]" = OrderedDict()
_plan_cache_tensors = 0


def _check(rc: int, what: str) -> None:
    if rc == 0:
        return
    if rc == -4:  # TFTQ_E_SIZE
        raise AssertionError("Output size does not match")
    raise RuntimeError(f"{what} failed: {_lib.strerror(rc)}")


def _validate(inputs: list[torch.Tensor]) -> tuple[torch.device, torch.dtype]:
    # quantization.py:462-489, same checks and messages; written with map() so that a
    # list of 10 000 tensors costs a few milliseconds rather than tens
    i_num = len(inputs)
    assert i_num > 0, "At least one input tensor is required"
    device = inputs[0].device
    dtype = inputs[0].dtype
    if i_num > 1:
        same_dev = len(set(map(_TENSOR.get_device, inputs))) == 1  # -1 for every CPU tensor
        assert same_dev, "All inputs must be on the same device"
        assert len(set(map(_DTYPE_OF, inputs))) == 1, "All inputs must be on the same dtype"
    assert dtype in _DTYPE_CODE, "Only fp32, fp16 and bf16 are supported"
    dims = list(map(_TENSOR.dim, inputs))
    if dims.count(2) != i_num:
        for i, d in enumerate(dims):
            # 1-D tensors become [k, 1] in the caller's list (quantization.py:487-488)
            if d == 1:
                inputs[i] = inputs[i].unsqueeze(1)
            assert inputs[i].dim() == 2, "Only 2D tensors are supported"
    return device, dtype


def _prepare(inputs: list[torch.Tensor], all_reduce_group_size: int) -> tuple[_Plan, torch.device]:
    """Counterpart of ``_prepare_quantize_fp8`` (quantization.py:431-528)."""
    device, dtype = _validate(inputs)
    if device.type != "cuda":
        raise RuntimeError(
            "torchft_amd.quantization needs tensors on a gfx950 GPU; there is no CPU path")
    ws = int(all_reduce_group_size)
    # The key holds tens of thousands of small tuples for long lists; keep the cyclic
    # garbage collector from walking them while they are being built.
    pause_gc = len(inputs) > 256 and gc.isenabled()
    if pause_gc:
        gc.disable()
    try:
        ptrs_key = tuple(map(_TENSOR.data_ptr, inputs))
        sizes_key = tuple(map(_TENSOR.size, inputs))
        strides_key = tuple(map(_TENSOR.stride, inputs))
        key = (device.index, dtype, ws, ptrs_key, sizes_key, strides_key)
    finally:
        if pause_gc:
            gc.enable()
    with _cache_lock:
        plan = _plan_cache.get(key)
        if plan is not None:
            _plan_cache.move_to_end(key)
            return plan, device

    lib = _lib.load()
    T = len(inputs)
    ptrs = (ctypes.c_void_p * T)()
    shapes = (ctypes.c_int64 * (2 * T))()
    strides = (ctypes.c_int64 * (2 * T))()
    ptrs[:] = ptrs_key
    shapes[:] = [d for sz in sizes_key for d in sz]
    strides[:] = [d for st in strides_key for d in st]
    handle = ctypes.c_void_p()
    _check(lib.tftq_plan_create(_DTYPE_CODE[dtype], T, ptrs, shapes, strides, ws,
                                ctypes.byref(handle)), "tftq_plan_create")
    table = None
    nbytes = lib.tftq_plan_table_bytes(handle)
    if nbytes > 0:
        host = (ctypes.c_uint8 * nbytes).from_address(lib.tftq_plan_table_host(handle))
        # synchronous copy: the plan may be used from any stream afterwards
        table = torch.frombuffer(host, dtype=torch.uint8).to(device)
        _check(lib.tftq_plan_set_device_table(handle, ctypes.c_void_p(table.data_ptr())),
               "tftq_plan_set_device_table")
    plan = _Plan(lib, handle, table, T)
    global _plan_cache_tensors
    with _cache_lock:
        old = _plan_cache.pop(key, None)  # another thread may have built the same plan
        if old is not None:
            _plan_cache_tensors -= old.n_tensors
        _plan_cache[key] = plan
        _plan_cache_tensors += T
        while len(_plan_cache) > 1 and (len(_plan_cache) > _PLAN_CACHE_SIZE
                                        or _plan_cache_tensors > _PLAN_CACHE_TENSORS):
            _, gone = _plan_cache.popitem(last=False)
            _plan_cache_tensors -= gone.n_tensors
    return plan, device


# Per-call host cost matters for the per-parameter all-reduce (thousands of small
# calls): the raw current stream and the current device come from torch's C
# bindings where they exist (0.3 us instead of 4 us for a Stream object and
# 2 us for a device context that changes nothing).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_ptr(device: torch.device) -> ctypes.c_void_p:
    if _raw_stream is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device: torch.device):
    """Context in which ``device`` is the current device."""
    if _raw_device is not None and device.index is not None and _raw_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


def _keep_table(plan: _Plan, device: torch.device) -> None:
    """A plan can be evicted from the cache while its kernel is still queued: tell the
    allocator on which stream the device table is in use."""
    if plan.table is not None:
        plan.table.record_stream(torch.cuda.current_stream(device))


def _check_packed(output: torch.Tensor, plan: _Plan, device: torch.device) -> None:
    assert output.shape[0] == plan.output_size, "Output size does not match"
    if output.dtype != torch.uint8 or not output.is_contiguous():
        raise RuntimeError("the packed buffer must be a contiguous uint8 tensor")
    if output.device != device:
        # its address would be handed to a kernel on `device`
        raise RuntimeError(f"the packed buffer is on {output.device}, the tensors are on {device}")


# The three stages on a prepared plan.  The public functions below prepare and
# call these; torchft_amd.collectives prepares once per collective and calls
# all three, which saves two walks over the tensor list.
def _quantize(plan: _Plan, device: torch.device) -> torch.Tensor:
    with _on_device(device):
        # float32 storage like the reference (:567-571) so that scales are aligned
        output = torch.empty(plan.output_size // SCALE_DTYPE_BYTES, device=device,
                             dtype=SCALE_DTYPE).view(torch.uint8)
        _check(plan._lib.tftq_quantize(plan.handle, ctypes.c_void_p(output.data_ptr()),
                                       plan.output_size, _stream_ptr(device)), "tftq_quantize")
        _keep_table(plan, device)
    return output


def _reduce(plan: _Plan, device: torch.device, output: torch.Tensor, rank: int,
            reduce_op: ReduceOp) -> None:
    _check_packed(output, plan, device)
    is_avg = 0 if reduce_op == ReduceOp.SUM else 1  # anything but SUM averages (:682)
    with _on_device(device):
        _check(plan._lib.tftq_reduce(plan.handle, ctypes.c_void_p(output.data_ptr()),
                                     plan.output_size, int(rank), is_avg,
                                     _stream_ptr(device)), "tftq_reduce")
        _keep_table(plan, device)


def _dequantize(plan: _Plan, device: torch.device, output: torch.Tensor,
                divide_by: float | None = None) -> None:
    _check_packed(output, plan, device)
    with _on_device(device):
        if divide_by is None:
            _check(plan._lib.tftq_dequantize(plan.handle, ctypes.c_void_p(output.data_ptr()),
                                             plan.output_size, _stream_ptr(device)),
                   "tftq_dequantize")
        else:
            # torch divides a GPU tensor by a host scalar as a multiplication by the
            # reciprocal, computed in double and rounded to fp32
            divisor = float(divide_by)
            factor = 1.0 / divisor if divisor != 0.0 else math.copysign(math.inf, divisor)
            _check(plan._lib.tftq_dequantize_scaled(plan.handle, ctypes.c_void_p(output.data_ptr()),
                                                    plan.output_size, factor,
                                                    _stream_ptr(device)),
                   "tftq_dequantize_scaled")
        _keep_table(plan, device)


def fused_quantize_into_fp8(
    inputs: list[torch.Tensor], all_reduce_group_size: int
) -> torch.Tensor:
    """
    Quantizes every row of every input tensor to fp8-e4m3fn with its own fp32
    scale and packs ``[scale][codes][pad]`` rows into one uint8 tensor laid out
    as ``all_reduce_group_size`` equal slots (quantization.py:531-588).

    Args:
        inputs: tensors to quantize (1-D or 2-D, one dtype, one device)
        all_reduce_group_size: size of the all-reduce group

    Returns:
        the packed uint8 tensor (``numel() % all_reduce_group_size == 0``)
    """
    plan, device = _prepare(inputs, all_reduce_group_size)
    return _quantize(plan, device)


def fused_dequantize_from_fp8(
    inputs: list[torch.Tensor], output: torch.Tensor, all_reduce_group_size: int,
    *, divide_by: float | None = None,
) -> None:
    """
    Dequantizes the packed tensor ``output`` into ``inputs`` in place
    (quantization.py:591-635).  The tensors must have the shapes that were
    quantized.

    ``divide_by`` (no counterpart in the reference's function) folds the caller's
    ``tensor /= divide_by`` (manager.py:450-452) into the same pass: the tensors end
    up with the bytes that dequantizing and then dividing each of them by that
    Python number on the GPU gives.
    """
    plan, device = _prepare(inputs, all_reduce_group_size)
    _dequantize(plan, device, output, divide_by)


def fused_reduce_fp8(
    inputs: list[torch.Tensor],
    output: torch.Tensor,
    all_reduce_group_size: int,
    all_reduce_rank: int,
    reduce_op: ReduceOp = ReduceOp.SUM,
) -> None:
    """
    Sums the ``all_reduce_group_size`` slots of ``output`` in fp32, requantizes
    and stores the result in slot ``all_reduce_rank`` (quantization.py:638-686).
    Any ``reduce_op`` other than SUM averages (quantization.py:682).
    ``inputs`` only supplies the shapes.
    """
    plan, device = _prepare(inputs, all_reduce_group_size)
    _reduce(plan, device, output, all_reduce_rank, reduce_op)
