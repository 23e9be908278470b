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
  five allocations per call, quantization.py:505-517) is replaced by a plan that
  depends on shapes, strides, dtype and group size only and is cached; the
  tensors' addresses travel with each call.  Lists of up to 16 tensors need no
  device metadata at all; longer lists use one cached descriptor table per
  device and 8 bytes per tensor for the addresses.

:func:`prepare` (no counterpart in the reference) does the walk over a tensor
list once and returns a :class:`PreparedBucket` whose ``quantize`` / ``reduce`` /
``dequantize`` cost the same few microseconds whatever the length of the list:
the thing to hold on to for a bucket that is reduced every step.

Lists of more than 16 tensors that come back call after call (the same shapes,
strides, dtype and device; the tensors themselves may be new or may have moved)
are recognised by one C++ walk over the list (``_pylist.scan``, about 10 ns per
tensor), which checks every tensor against the plan of an earlier call and
collects the addresses (on this path 1-D tensors are taken as their ``[k, 1]``
views without being replaced in the caller's list); the three functions then cost a fraction of a
millisecond on 10 000 tensors instead of the 5 ms of the walk in Python, which
stays as the path of every first call and of every list that does not match.

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

from . import _build, _lib

_pylist = _build.load_pylist()  # None when the helper cannot be built: the Python walk does everything

SCALE_DTYPE: torch.dtype = torch.float32
SCALE_DTYPE_BYTES: int = 4

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_TENSOR = torch.Tensor
_DTYPE_OF = operator.attrgetter("dtype")
_N_INLINE = 16  # TFTQ_N_INLINE
# Plans are cached by (dtype, group size, shapes, strides).  The per-parameter all-reduce of a
# model has one single-tensor plan per distinct shape; long lists are bounded by their total
# length.
_PLAN_CACHE_SIZE = 4096
_PLAN_CACHE_TENSORS = 1 << 18


class _Ready:
    """An upload that kernels on other streams must wait for until it has completed."""

    __slots__ = ("event", "stream_id")

    def __init__(self, stream: torch.cuda.Stream) -> None:
        self.event: torch.cuda.Event | None = torch.cuda.Event()
        self.event.record(stream)
        self.stream_id = stream.cuda_stream

    def wait(self, stream: torch.cuda.Stream, raw_stream: int) -> None:
        ev = self.event
        if ev is None or raw_stream == self.stream_id:  # done, or ordered by the stream itself
            return
        if torch.cuda.is_current_stream_capturing():
            stream.wait_event(ev)  # a capture may wait for an outside event, but not ask about it
        elif ev.query():
            self.event = None
        else:
            stream.wait_event(ev)


class _Plan:
    """Owns a ``tftq_plan`` and, for long tensor lists, its descriptor table on every
    device it has been used on.  Holds no tensor and no address."""

    __slots__ = ("handle", "output_size", "slot_size", "max_rows", "n_tensors", "table_bytes",
                 "tables", "_lib", "_lock", "dtype_code", "ws", "shapes", "strides", "a_shapes",
                 "a_strides", "streams")

    def __init__(self, lib, handle, n_tensors, dtype_code, ws, shapes, strides):
        self._lib = lib
        self.handle = handle
        self.n_tensors = n_tensors
        self.dtype_code = dtype_code
        self.ws = ws
        # what the plan was built from, [n_tensors][2] int64 each: _pylist.scan compares a list with them
        self.shapes = shapes
        self.strides = strides
        self.a_shapes = ctypes.addressof(shapes)
        self.a_strides = ctypes.addressof(strides)
        # long lists through the named functions: (device index, raw stream) -> _StreamPointers
        self.streams: "OrderedDict[tuple, _StreamPointers]" = OrderedDict()
        self.output_size = lib.tftq_plan_output_size(handle)
        self.slot_size = lib.tftq_plan_slot_size(handle)
        self.max_rows = lib.tftq_plan_max_rows(handle)
        self.table_bytes = lib.tftq_plan_table_bytes(handle)
        self.tables: dict = {}  # device index -> (device tensor, _Ready)
        self._lock = threading.Lock()

    def table_on(self, device: torch.device):
        """The descriptor table on ``device`` (None for short lists).  The first use on a
        device copies the image from pinned staging memory on the current stream; nothing
        blocks, and users on other streams wait for the copy's event."""
        if self.table_bytes == 0:
            return None
        entry = self.tables.get(device.index)
        if entry is None:
            with self._lock:
                entry = self.tables.get(device.index)
                if entry is None:
                    host = (ctypes.c_uint8 * self.table_bytes).from_address(
                        self._lib.tftq_plan_table_host(self.handle))
                    staged = torch.empty(self.table_bytes, dtype=torch.uint8, pin_memory=True)
                    staged.copy_(torch.frombuffer(host, dtype=torch.uint8))
                    with torch.cuda.device(device):
                        table = torch.empty(self.table_bytes, dtype=torch.uint8, device=device)
                        table.copy_(staged, non_blocking=True)  # the pinned allocator keeps `staged` until then
                        entry = (table, _Ready(torch.cuda.current_stream(device)))
                    self.tables[device.index] = entry
        return entry

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


def _plan_for(dtype: torch.dtype, ws: int, sizes_key: tuple, strides_key: tuple) -> _Plan:
    key = (dtype, ws, sizes_key, strides_key)
    with _cache_lock:
        plan = _plan_cache.get(key)
        if plan is not None:
            _plan_cache.move_to_end(key)
            return plan
    lib = _lib.load()
    T = len(sizes_key)
    shapes = (ctypes.c_int64 * (2 * T))()
    strides = (ctypes.c_int64 * (2 * T))()
    shapes[:] = [d for sz in sizes_key for d in sz]
    strides[:] = [d for st in strides_key for d in st]
    handle = ctypes.c_void_p()
    _check(lib.tftq_plan_create(_DTYPE_CODE[dtype], T, shapes, strides, ws, ctypes.byref(handle)),
           "tftq_plan_create")
    plan = _Plan(lib, handle, T, _DTYPE_CODE[dtype], ws, shapes, strides)
    global _plan_cache_tensors
    with _cache_lock:
        old = _plan_cache.pop(key, None)  # another thread may have built the same plan
        if old is not None:
            _plan_cache_tensors -= old.n_tensors
            _forget_long_plan(old)
        _plan_cache[key] = plan
        _plan_cache_tensors += T
        if T > _N_INLINE:
            _long_plans.setdefault((T, ws), []).insert(0, plan)
        while len(_plan_cache) > 1 and (len(_plan_cache) > _PLAN_CACHE_SIZE
                                        or _plan_cache_tensors > _PLAN_CACHE_TENSORS):
            _, gone = _plan_cache.popitem(last=False)
            _plan_cache_tensors -= gone.n_tensors
            _forget_long_plan(gone)
    return plan


# ---------------------------------------------------------------------------------------------
# long lists through the three named functions
# ---------------------------------------------------------------------------------------------
# Plans of more than 16 tensors by (number of tensors, group size), newest first: the plans a
# list of that length is compared with by _pylist.scan before the Python walk is tried.
_long_plans: "dict[tuple, list[_Plan]]" = {}
_LONG_CANDIDATES = 4    # plans of one length and group size that a call compares its list with
_STREAMS_PER_PLAN = 8   # address buffers (one per device and stream) that a plan keeps


def _forget_long_plan(plan: _Plan) -> None:  # called with _cache_lock held
    peers = _long_plans.get((plan.n_tensors, plan.ws))
    if peers is not None and plan in peers:
        peers.remove(plan)
        if not peers:
            del _long_plans[(plan.n_tensors, plan.ws)]


class _StreamPointers:
    """What a plan keeps for calls on one stream of one device: the device copy of a long
    list's addresses and what it holds, so that a call whose list has the addresses of the
    last one uploads nothing."""

    __slots__ = ("dev", "held", "lock")

    def __init__(self, plan: _Plan, device: torch.device, table: torch.Tensor) -> None:
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream(device)
            self.dev = torch.empty(plan.n_tensors, dtype=torch.int64, device=device)
            # both are read by kernels on this stream, which need not be the one they were allocated on
            self.dev.record_stream(stream)
            table.record_stream(stream)
        self.held = None   # host array of the addresses that `dev` holds (or will, in stream order)
        self.lock = threading.Lock()


_memcmp = ctypes.CDLL(None).memcmp
_memcmp.restype = ctypes.c_int
_memcmp.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]


def _match_long_list(inputs, ws: int, want_pointers: bool):
    """(plan, device, addresses) when `inputs` is a list of more than 16 tensors that fits a
    plan of an earlier call as it is (same length, group size, dtype, sizes and strides, every
    tensor 2-D, or 1-D and taken as its [k, 1] view, and on one GPU), found with one C++ walk
    per candidate plan; else None, and
    the caller takes the Python walk.  addresses: a fresh host array, or None when not wanted."""
    if _pylist is None or type(inputs) is not list:
        return None
    T = len(inputs)
    if T <= _N_INLINE:
        return None
    peers = _long_plans.get((T, ws))
    if not peers:
        return None
    first = inputs[0]
    if not isinstance(first, _TENSOR):
        return None
    device = first.device
    if device.type != "cuda":
        return None
    ptrs = (ctypes.c_void_p * T)() if want_pointers else None
    a_ptrs = ctypes.addressof(ptrs) if want_pointers else 0
    for plan in peers[:_LONG_CANDIDATES]:
        if _pylist.scan(inputs, plan.dtype_code, device.index, plan.a_shapes, plan.a_strides, a_ptrs, T) == T:
            return plan, device, ptrs
    return None


def _long_list_args(plan: _Plan, device: torch.device, raw_stream: int, ptrs):
    """(table, pointers, lock to hold until the kernel is queued) for a compute call on a
    matched long list.  The addresses are uploaded on the call's stream unless the buffer
    of this device and stream holds them already (ptrs None: no addresses wanted, no lock)."""
    table, ready = plan.table_on(device)
    if ready.event is not None:
        ready.wait(torch.cuda.current_stream(device), raw_stream)
    key = (device.index, raw_stream)
    sp = plan.streams.get(key)
    if sp is None:
        with plan._lock:
            sp = plan.streams.get(key)
            if sp is None:
                sp = _StreamPointers(plan, device, table)
                plan.streams[key] = sp
                while len(plan.streams) > _STREAMS_PER_PLAN:
                    plan.streams.popitem(last=False)
    if ptrs is None:
        return table.data_ptr(), None, None
    sp.lock.acquire()
    try:
        capturing = torch.cuda.is_current_stream_capturing()
        if capturing or sp.held is None or _memcmp(sp.held, ptrs, 8 * plan.n_tensors) != 0:
            _check(plan._lib.tftq_upload_pointers(plan.handle, ptrs, sp.dev.data_ptr(), device.index, raw_stream),
                   "tftq_upload_pointers")
            # an upload that a stream capture records has not run: the next call uploads again
            sp.held = None if capturing else ptrs
    except BaseException:
        sp.lock.release()
        raise
    return table.data_ptr(), sp.dev.data_ptr(), sp.lock


# Per-call host cost matters for the per-parameter all-reduce (thousands of small
# calls): the raw current stream comes from torch's C bindings where they exist
# (0.3 us instead of 4 us for a Stream object).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_of(device: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class PreparedBucket:
    """One list of tensors, ready for the three kernels: the result of :func:`prepare`.

    Holds the plan, the tensors (so that their memory outlives every kernel queued on
    their addresses) and, for lists of more than 16 tensors, the device copy of their
    addresses.  The methods launch on the current stream of the tensors' device and cost
    a few microseconds of host time whatever the length of the list.

    The bucket is bound to the storage the tensors had when it was prepared: prepare again
    after ``tensor.data = ...``, ``resize_`` or anything else that moves a tensor.  One
    bucket may be used from several threads and streams.  A HIP graph that captures these
    calls must be kept together with the bucket: it pins the plan's table and the
    addresses that the captured kernels read.
    """

    __slots__ = ("plan", "device", "tensors", "ws", "_ptrs", "_ptrs_dev", "_ptrs_ready", "_table",
                 "_table_ready", "_lib", "_handle", "_dev_index", "_lock")

    def __init__(self, plan: _Plan, device: torch.device, tensors: list, ws: int, ptrs) -> None:
        self.plan = plan
        self.device = device
        self.tensors = tensors
        self.ws = ws
        self._lib = plan._lib
        self._handle = plan.handle
        self._dev_index = device.index
        self._ptrs = ptrs                # host array of addresses (ctypes)
        self._ptrs_dev = None            # long lists: their device copy, written by the first call
        self._ptrs_ready: _Ready | None = None
        self._table = None
        self._table_ready: _Ready | None = None
        self._lock = threading.Lock()
        if plan.table_bytes:
            table, ready = plan.table_on(device)
            self._table = table
            self._table_ready = ready
            with torch.cuda.device(device):
                self._ptrs_dev = torch.empty(plan.n_tensors, dtype=torch.int64, device=device)

    # -- properties of the layout ------------------------------------------------------
    @property
    def output_size(self) -> int:
        """Bytes of the packed buffer (``numel()`` of what :meth:`quantize` returns)."""
        return self.plan.output_size

    @property
    def slot_size(self) -> int:
        return self.plan.slot_size

    def matches(self, tensors) -> bool:
        """True when ``tensors`` are what this bucket was prepared for: as many tensors, of the
        plan's dtype, sizes and strides (a 1-D tensor of k elements counts as ``[k, 1]``,
        quantization.py:487-488), on the bucket's device, at the addresses the bucket has bound."""
        plan = self.plan
        n = plan.n_tensors
        if len(tensors) != n:
            return False
        if _pylist is not None and type(tensors) is list:
            got = (ctypes.c_void_p * n)()
            if _pylist.scan(tensors, plan.dtype_code, self._dev_index, plan.a_shapes, plan.a_strides,
                            ctypes.addressof(got), n) == n:
                return _memcmp(got, self._ptrs, 8 * n) == 0
        shapes, strides, ptrs = plan.shapes, plan.strides, self._ptrs
        for i, t in enumerate(tensors):
            if not isinstance(t, _TENSOR) or _DTYPE_CODE.get(t.dtype) != plan.dtype_code or t.device != self.device:
                return False
            if t.dim() == 2:
                size, stride = tuple(t.shape), t.stride()
            elif t.dim() == 1:
                size, stride = (t.shape[0], 1), (t.stride(0), 1)
            else:
                return False
            if (size[0] != shapes[2 * i] or size[1] != shapes[2 * i + 1] or stride[0] != strides[2 * i]
                    or stride[1] != strides[2 * i + 1] or t.data_ptr() != (ptrs[i] or 0)):
                return False
        return True

    # -- launches ------------------------------------------------------------------------
    def _long_list_args(self, raw_stream: int, needs_pointers: bool):
        """(table, pointers) arguments of a compute call on a long list, both current for
        kernels on the current stream, and protected against being freed while in use there."""
        stream = torch.cuda.current_stream(self.device)
        self._table_ready.wait(stream, raw_stream)
        self._table.record_stream(stream)
        if not needs_pointers:
            return self._table.data_ptr(), None
        self._ptrs_dev.record_stream(stream)
        ready = self._ptrs_ready
        if ready is None:
            with self._lock:
                ready = self._ptrs_ready
                if ready is None:
                    # the first call on this bucket writes the addresses; later calls reuse them
                    _check(self._lib.tftq_upload_pointers(self._handle, self._ptrs, self._ptrs_dev.data_ptr(),
                                                          self._dev_index, raw_stream), "tftq_upload_pointers")
                    # Under a stream capture the upload has only been recorded (it runs with the
                    # graph, before the kernel recorded behind it): nothing is ready, and the
                    # next call uploads again.
                    if not torch.cuda.is_current_stream_capturing():
                        self._ptrs_ready = _Ready(stream)
                    return self._table.data_ptr(), self._ptrs_dev.data_ptr()
        ready.wait(stream, raw_stream)
        return self._table.data_ptr(), self._ptrs_dev.data_ptr()

    def quantize(self, out: torch.Tensor | None = None) -> torch.Tensor:
        """Quantizes the tensors into ``out`` (allocated when None) and returns it."""
        plan = self.plan
        if out is None:
            out = torch.empty(plan.output_size, dtype=torch.uint8, device=self.device)
        else:
            _check_packed(out, plan, self.device)
        raw = _stream_of(self.device)
        if self._table is None:
            rc = self._lib.tftq_quantize(self._handle, self._ptrs, None, None, out.data_ptr(),
                                         plan.output_size, self._dev_index, raw)
        else:
            table, pointers = self._long_list_args(raw, True)
            rc = self._lib.tftq_quantize(self._handle, None, table, pointers, out.data_ptr(),
                                         plan.output_size, self._dev_index, raw)
        _check(rc, "tftq_quantize")
        return out

    def reduce(self, packed: torch.Tensor, rank: int, reduce_op: ReduceOp = ReduceOp.SUM) -> None:
        """Reduces the ``ws`` slots of ``packed`` into slot ``rank`` in place."""
        plan = self.plan
        _check_packed(packed, plan, self.device)
        is_avg = 0 if reduce_op == ReduceOp.SUM else 1  # anything but SUM averages (:682)
        raw = _stream_of(self.device)
        table = None
        if self._table is not None:
            table, _ = self._long_list_args(raw, False)
        _check(self._lib.tftq_reduce(self._handle, table, packed.data_ptr(), plan.output_size, int(rank), is_avg,
                                     self._dev_index, raw), "tftq_reduce")

    def dequantize(self, packed: torch.Tensor, divide_by: float | None = None) -> None:
        """Dequantizes ``packed`` into the tensors; with ``divide_by`` they end up with the
        bytes of dequantizing and then dividing each of them by that Python number."""
        plan = self.plan
        _check_packed(packed, plan, self.device)
        raw = _stream_of(self.device)
        tensors, table, pointers = self._ptrs, None, None
        if self._table is not None:
            tensors = None
            table, pointers = self._long_list_args(raw, True)
        if divide_by is None:
            _check(self._lib.tftq_dequantize(self._handle, tensors, table, pointers, packed.data_ptr(),
                                             plan.output_size, self._dev_index, raw), "tftq_dequantize")
        else:
            _check(self._lib.tftq_dequantize_scaled(self._handle, tensors, table, pointers, packed.data_ptr(),
                                                    plan.output_size, _post_scale(divide_by), self._dev_index, raw),
                   "tftq_dequantize_scaled")


def _post_scale(divide_by: float) -> float:
    # torch divides a GPU tensor by a host scalar as a multiplication by the reciprocal,
    # computed in double and rounded to fp32
    divisor = float(divide_by)
    return 1.0 / divisor if divisor != 0.0 else math.copysign(math.inf, divisor)


def _check_packed(output: torch.Tensor, plan: _Plan, device: torch.device) -> None:
    assert output.shape[0] == plan.output_size, "Output size does not match"
    if output.dtype != torch.uint8 or not output.is_contiguous():
        raise RuntimeError("the packed buffer must be a contiguous uint8 tensor")
    if output.device != device:
        # its address would be handed to a kernel on `device`
        raise RuntimeError(f"the packed buffer is on {output.device}, the tensors are on {device}")


def prepare(inputs: list[torch.Tensor], all_reduce_group_size: int) -> PreparedBucket:
    """Counterpart of ``_prepare_quantize_fp8`` (quantization.py:431-528): validates the
    list, turns 1-D tensors into ``[k, 1]`` in the caller's list (:487-488), finds or
    builds the plan for these shapes and binds the tensors' addresses to it.  This is the
    only walk over the list; the returned bucket can be used any number of times."""
    device, dtype = _validate(inputs)
    if device.type != "cuda":
        raise RuntimeError(
            "torchft_amd.quantization needs tensors on a gfx950 GPU; there is no CPU path")
    _lib.check_device(device.index)
    ws = int(all_reduce_group_size)
    T = len(inputs)
    # The key holds tens of thousands of small tuples for long lists; keep the cyclic
    # garbage collector from walking them while they are being built.
    pause_gc = T > 256 and gc.isenabled()
    if pause_gc:
        gc.disable()
    try:
        sizes_key = tuple(map(_TENSOR.size, inputs))
        strides_key = tuple(map(_TENSOR.stride, inputs))
        plan = _plan_for(dtype, ws, sizes_key, strides_key)
        ptrs = (ctypes.c_void_p * T)()
        ptrs[:] = list(map(_TENSOR.data_ptr, inputs))
    finally:
        if pause_gc:
            gc.enable()
    return PreparedBucket(plan, device, list(inputs), ws, ptrs)


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
    hit = _match_long_list(inputs, all_reduce_group_size, True)
    if hit is None:
        return prepare(inputs, all_reduce_group_size).quantize()
    plan, device, ptrs = hit
    out = torch.empty(plan.output_size, dtype=torch.uint8, device=device)
    raw = _stream_of(device)
    table, pointers, lock = _long_list_args(plan, device, raw, ptrs)
    try:
        rc = plan._lib.tftq_quantize(plan.handle, None, table, pointers, out.data_ptr(), plan.output_size,
                                     device.index, raw)
    finally:
        lock.release()
    _check(rc, "tftq_quantize")
    return out


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
    hit = _match_long_list(inputs, all_reduce_group_size, True)
    if hit is None:
        prepare(inputs, all_reduce_group_size).dequantize(output, divide_by)
        return
    plan, device, ptrs = hit
    _check_packed(output, plan, device)
    raw = _stream_of(device)
    table, pointers, lock = _long_list_args(plan, device, raw, ptrs)
    try:
        if divide_by is None:
            rc = plan._lib.tftq_dequantize(plan.handle, None, table, pointers, output.data_ptr(),
                                           plan.output_size, device.index, raw)
        else:
            rc = plan._lib.tftq_dequantize_scaled(plan.handle, None, table, pointers, output.data_ptr(),
                                                  plan.output_size, _post_scale(divide_by), device.index, raw)
    finally:
        lock.release()
    _check(rc, "tftq_dequantize")


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
    hit = _match_long_list(inputs, all_reduce_group_size, False)
    if hit is None:
        prepare(inputs, all_reduce_group_size).reduce(output, all_reduce_rank, reduce_op)
        return
    plan, device, _ = hit
    _check_packed(output, plan, device)
    is_avg = 0 if reduce_op == ReduceOp.SUM else 1  # anything but SUM averages (:682)
    raw = _stream_of(device)
    table, _, _ = _long_list_args(plan, device, raw, None)
    _check(plan._lib.tftq_reduce(plan.handle, table, output.data_ptr(), plan.output_size, int(all_reduce_rank),
                                 is_avg, device.index, raw), "tftq_reduce")
