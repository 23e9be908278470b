"""The callers of the quantized all-reduce: one managed all-reduce of a tensor and
DiLoCo's bucketised averaging of pseudo-gradients.

Data path of ``Manager.allreduce`` (torchft/manager.py:386-467) and of
``_StreamingDiLoCoFragment._bucketize_and_allreduce`` /
``_allreduce_per_param`` (torchft/local_sgd.py:489-567), without the manager's
quorum, error tracking and healing: what is left is which tensors go through
:func:`torchft_amd.collectives.allreduce_quantized`, with which reduce op, on
which stream, and what is done to the result.

* ``allreduce`` zeroes the tensor of a replica that is not participating, turns
  AVG into SUM for the collective and divides by the number of participants in
  a continuation of the collective's future (manager.py:419-456); on the
  quantized path the division is done by the dequantize kernel as it stores
  (same bytes, one read and one write of the tensor less).  With
  ``should_quantize`` the list ``[tensor]`` goes to ``allreduce_quantized`` on
  the current stream (manager.py:432-439); a 1-D tensor is quantized as rows of
  one column (quantization.py:487-488), 8 packed bytes per element.
* ``bucketize_and_allreduce`` packs the tensors into flat zero-initialised
  buffers of at most ``bucket_size_bytes``, reduces each buffer and copies the
  result back in the continuation (local_sgd.py:499-556).

``row_width`` is an addition with no counterpart in the reference: the flat
bucket is handed to the all-reduce as a 2-D view ``[rows, row_width]``, so that
quantization keeps one scale per ``row_width`` elements (``row_width + 4`` packed
bytes per row) instead of one per element.  It changes the quantization
granularity, hence the values, and is off by default.
"""

from __future__ import annotations

from typing import Any, Callable

import torch
from torch.distributed import ReduceOp
from torch.distributed.distributed_c10d import AllreduceOptions

from . import quantization as _q
from .collectives import allreduce_quantized


class _Completed:
    """What a continuation is called with: the value the chain has reached."""

    def __init__(self, value: Any) -> None:
        self._value = value

    def wait(self) -> Any:
        return self._value

    def value(self) -> Any:
        return self._value


class _ChainFuture:
    """The future of a :class:`_ChainedWork`: ``then`` appends to the work's chain,
    so that the continuation runs on the work's stream like the ones before it."""

    def __init__(self, work: "_ChainedWork") -> None:
        self._work = work

    def then(self, callback: Callable[[Any], Any]) -> "_ChainFuture":
        self._work._then(lambda value: callback(_Completed(value)))
        return self

    def wait(self) -> Any:
        return self._work._tail.wait()

    def value(self) -> Any:
        return self._work._tail.value()


class _ChainedWork:
    """The collective's work plus the continuations that finish the tensor.

    Every continuation runs with the stream that was current when the work was
    created, after a dependency on the collective (manager.py:1214-1227), in
    the order in which it was added."""

    def __init__(self, work: Any, value: Any) -> None:
        self._work = work
        self._stream = torch.cuda.current_stream() if torch.cuda.is_available() else None
        self._tail: torch.futures.Future = work.get_future().then(lambda fut: value)

    def _then(self, callback: Callable[[Any], Any]) -> None:
        stream = self._stream

        def run(fut: torch.futures.Future) -> Any:
            if stream is None:
                return callback(fut.wait())
            with torch.cuda.stream(stream):
                return callback(fut.wait())

        self._tail = self._tail.then(run)

    def wait(self, timeout=None) -> bool:
        self._work.wait()
        self._tail.wait()
        return True

    def get_future(self) -> _ChainFuture:
        return _ChainFuture(self)


def allreduce(
    tensor: torch.Tensor,
    process_group: Any,
    num_participants: int,
    is_participating: bool = True,
    should_quantize: bool = False,
    reduce_op: ReduceOp = ReduceOp.AVG,
    fold_normalization: bool = True,
    prepared: "_q.PreparedBucket | None" = None,
):
    """
    All-reduce ``tensor`` in place over ``process_group`` and scale it by
    ``1 / num_participants`` when ``reduce_op`` is AVG (manager.py:386-456).
    With ``should_quantize`` the scaling is part of the dequantize kernel unless
    ``fold_normalization`` is False (then it is a separate in-place division in
    the continuation, as in the reference); the resulting bytes are the same.

    ``prepared``: ``torchft_amd.quantization.prepare([tensor], process_group.size())`` made
    once for a tensor that is reduced every step (see :class:`BucketizedAllreduce`).

    Returns a work whose future completes with the tensor.  The result is in
    ``tensor`` once the work has been waited on, in stream order of the stream
    that was current at the call.
    """
    if not is_participating:
        tensor.zero_()  # manager.py:419-420

    pg_reduce_op = reduce_op
    if reduce_op == ReduceOp.AVG:
        if not torch.is_floating_point(tensor):
            raise ValueError("average reduce op is only supported for floating point tensors")
        pg_reduce_op = ReduceOp.SUM  # manager.py:422-429

    normalized = False
    if should_quantize:
        # the division by the number of participants (manager.py:450-452) happens in the
        # dequantize kernel: same bytes, one pass over the tensor less
        divide_by = num_participants if reduce_op == ReduceOp.AVG and fold_normalization else None
        normalized = divide_by is not None
        work = allreduce_quantized([tensor], pg_reduce_op, process_group, torch.cuda.current_stream(),
                                   divide_by=divide_by, prepared=prepared)
    else:
        opts = AllreduceOptions()
        opts.reduceOp = pg_reduce_op
        work = process_group.allreduce([tensor], opts)

    chained = _ChainedWork(work, tensor)

    def normalize(value: torch.Tensor) -> torch.Tensor:
        if reduce_op == ReduceOp.AVG and not normalized:
            value /= num_participants  # manager.py:450-452
        return value

    chained._then(normalize)
    return chained


def allreduce_per_param(grads: dict, allreduce_fn: Callable[[torch.Tensor], Any]) -> list:
    """One all-reduce per pseudo-gradient (local_sgd.py:489-497)."""
    return [allreduce_fn(g) for g in grads.values()]


def plan_buckets(sizes: list, capacity: int) -> list:
    """Which tensors share a flat buffer: ``[(buffer length, [tensor indices]), ...]``.

    The reference's walk (local_sgd.py:519-553): a buffer has ``capacity`` elements, or
    what is left of the total if that is less; tensors are taken in order while they fit;
    the walk ends when the buffer lengths add up to the total element count.  Because the
    lengths, not the packed elements, are added up, a tensor that does not fit the rest of
    a buffer can leave the last tensors in no buffer at all.
    """
    total = sum(sizes)
    plan, covered, nxt = [], 0, 0
    while covered < total:
        length = min(capacity, total - covered)
        members, used = [], 0
        while nxt < len(sizes) and used + sizes[nxt] <= length:
            members.append(nxt)
            used += sizes[nxt]
            nxt += 1
        plan.append((length, members))
        covered += length
    return plan


def _copy_all(dst: list, src: list) -> None:
    """dst[i].copy_(src[i]) for all i: a few batched kernels instead of one launch per
    tensor (200 tensors: 0.8 ms of launches -> 0.05 ms)."""
    if not dst:
        return
    foreach = getattr(torch, "_foreach_copy_", None)
    if foreach is not None:
        foreach(dst, src)
    else:
        for d, s in zip(dst, src):
            d.copy_(s)


class BucketizedAllreduce:
    """DiLoCo's bucket packing (local_sgd.py:499-556) with everything that does not change
    from step to step built once: the flat buffers, the views of the tensors inside them and,
    on the quantized path, one prepared bucket per flat buffer, so that a step costs the
    copies and a few microseconds of host time per bucket.

    The packing is the reference's (:func:`plan_buckets`), including its corner: tensors that
    end up in no buffer keep their local values.  A bucket capacity that is a multiple of
    every tensor's size, or larger than the whole list, avoids it.

    One instance serves one list of tensors; steps on the same instance must not overlap
    (wait for the works of a step before starting the next one: they share the flat buffers).
    """

    def __init__(self, tensors: list, bucket_size_bytes: int, row_width: int | None = None) -> None:
        self.tensors = list(tensors)
        self.row_width = row_width
        self.buckets: list = []
        if not self.tensors:
            return
        first = self.tensors[0]
        capacity = bucket_size_bytes // first.element_size()
        assert capacity > 0, "bucket_size_bytes is smaller than one element"
        for length, members in plan_buckets([t.numel() for t in self.tensors], capacity):
            padded = length
            if row_width:
                padded = -(-length // row_width) * row_width  # whole rows; the tail stays zero
            flat = torch.zeros(padded, dtype=first.dtype, device=first.device)  # zero-filled (:527-529)
            owners, pieces, at = [], [], 0
            for i in members:
                n = self.tensors[i].numel()
                owners.append(self.tensors[i])
                pieces.append(flat[at:at + n].view_as(self.tensors[i]))
                at += n
            self.buckets.append({"flat": flat, "view": flat.view(-1, row_width) if row_width else flat,
                                 "owners": owners, "pieces": pieces, "used": at, "prepared": {}, "fresh": True})

    def _pack(self, bucket: dict) -> None:
        if not bucket["fresh"] and bucket["used"] < bucket["flat"].numel():
            bucket["flat"][bucket["used"]:].zero_()  # what no tensor covers is zero in every step (:527-529)
        bucket["fresh"] = False
        _copy_all(bucket["pieces"], bucket["owners"])  # :534-537

    @staticmethod
    def _unpack_later(work: Any, bucket: dict) -> None:
        owners, pieces = bucket["owners"], bucket["pieces"]

        def unpack(fut):
            _copy_all(owners, pieces)  # :546-551
            return []

        work.get_future().then(unpack)

    def __call__(self, allreduce_fn: Callable[[torch.Tensor], Any]) -> list:
        """Packs, calls ``allreduce_fn(flat)`` for every bucket and returns the works; each
        tensor holds its reduced values once its bucket's work has been waited on."""
        works = []
        for bucket in self.buckets:
            self._pack(bucket)
            work = allreduce_fn(bucket["view"])
            self._unpack_later(work, bucket)
            works.append(work)
        return works

    def allreduce(self, process_group: Any, num_participants: int, is_participating: bool = True,
                  should_quantize: bool = True, reduce_op: ReduceOp = ReduceOp.AVG) -> list:
        """One managed all-reduce (:func:`allreduce`) per bucket; the quantized path reuses the
        buckets' prepared tensor lists."""
        works = []
        ws = process_group.size()
        for bucket in self.buckets:
            self._pack(bucket)
            prepared = None
            if should_quantize:
                prepared = bucket["prepared"].get(ws)
                if prepared is None:
                    prepared = bucket["prepared"][ws] = _q.prepare([bucket["view"]], ws)
            work = allreduce(bucket["view"], process_group, num_participants, is_participating,
                             should_quantize, reduce_op, prepared=prepared)
            self._unpack_later(work, bucket)
            works.append(work)
        return works


def bucketize_and_allreduce(
    tensors: list,
    bucket_size_bytes: int,
    allreduce_fn: Callable[[torch.Tensor], Any],
    row_width: int | None = None,
) -> list:
    """
    All-reduce ``tensors`` through flat buffers of at most ``bucket_size_bytes``
    (local_sgd.py:499-556) and return the works; each tensor holds its reduced
    values once its bucket's work has been waited on.  The flat buffers are allocated
    for this call, as in the reference; :class:`BucketizedAllreduce` keeps them from
    step to step.

    ``allreduce_fn(flat)`` is, for example,
    ``lambda t: allreduce(t, pg, n, should_quantize=True)``.
    """
    return BucketizedAllreduce(tensors, bucket_size_bytes, row_width)(allreduce_fn)
