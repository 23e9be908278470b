"""Quantized all-reduce and reduce-scatter: host orchestration on ROCm.

Same public surface as ``torchft/collectives.py`` (``get_padded_sizes``,
``allocate_reduce_scatter_output``, ``reduce_scatter_quantized``,
``allreduce_quantized``; same arguments, return values and errors), built on the
gfx950 kernels of :mod:`torchft_amd.quantization`.

``process_group`` is anything with ``rank()``, ``size()``,
``alltoall_base(out, in, [], [], opts)`` and
``allgather_into_tensor_coalesced(outs, ins, opts)`` whose results offer
``wait()`` and ``get_future()``: torchft's process-group wrappers over RCCL
(backend ``"nccl"`` on ROCm) in production, the one-process simulation of
``tests/sim_pg.py`` in this repository.

Data flow of both collectives (collectives.py:159-294, 297-415):

    quantize(tensors)  --all-to-all of slots-->  reduce(own slot)
        all-reduce:      --all-gather of reduced slots-->  dequantize(tensors)
        reduce-scatter:  dequantize(own slot) into ``output``

Everything is queued on ``sync_stream`` after a dependency on the caller's
current stream; the host never blocks.  The last stage runs in the done-callback
of the last collective's future, as in the reference.  The receive buffer of the
all-to-all is allocated uninitialised: the exchange overwrites every byte of it
(the reference zero-fills it, collectives.py:243, 367).
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any

import torch
from torch import cuda
from torch.distributed import ReduceOp
from torch.distributed.distributed_c10d import (
    AllgatherOptions,
    AllreduceOptions,
    AllToAllOptions,
    ReduceScatterOptions,
)

from . import quantization as _q

_SUPPORTED_OPS = (ReduceOp.AVG, ReduceOp.SUM)


def get_padded_sizes(tensors: list[torch.Tensor], world_size: int) -> list[torch.Size]:
    """Sizes of ``tensors`` with dim 0 rounded up to a multiple of ``world_size``;
    a 1-D tensor counts as ``[k, 1]`` (collectives.py:51-84)."""
    out = []
    for t in tensors:
        dims = tuple(t.size())
        if len(dims) == 1:
            dims = (dims[0], 1)
        rows = math.ceil(dims[0] / world_size) * world_size
        out.append(torch.Size((rows,) + dims[1:]))
    return out


def allocate_reduce_scatter_output(
    tensors: list[torch.Tensor], world_size: int
) -> tuple[torch.Tensor, list[torch.Size]]:
    """A flat tensor for this rank's share of a reduce-scatter of ``tensors`` and
    the padded input sizes (collectives.py:87-136)."""
    first = tensors[0]
    for prev, cur in zip(tensors, tensors[1:]):
        assert cur.device == prev.device, "All inputs must be on the same device"
        assert cur.dtype == prev.dtype, "All inputs must be on the same dtype"
    padded = get_padded_sizes(tensors, world_size)
    share = sum(p.numel() // world_size for p in padded)
    return torch.empty((share,), device=first.device, dtype=first.dtype), padded


@dataclass
class _Exchange:
    """One quantized collective in flight: who we are, what op, which stream."""

    pg: Any
    reduce_op: ReduceOp
    timeout: Any
    stream: cuda.Stream

    @property
    def rank(self) -> int:
        return self.pg.rank()

    @property
    def world_size(self) -> int:
        return self.pg.size()

    def scatter_slots(self, packed: torch.Tensor):
        """All-to-all of the ``world_size`` slots of ``packed``; returns the buffer
        of received slots and the work object."""
        ws = self.world_size
        received = torch.empty_like(packed)
        opts = AllToAllOptions()
        opts.timeout = self.timeout
        work = self.pg.alltoall_base(received.view(ws, -1), packed.view(ws, -1), [], [], opts)
        return received, work

    def gather_slots(self, into: torch.Tensor, received: torch.Tensor):
        """All-gather of every rank's reduced slot into ``into``."""
        ws = self.world_size
        opts = AllgatherOptions()
        opts.timeout = self.timeout
        mine = torch.split(received.view(ws, -1), 1)[self.rank]
        return self.pg.allgather_into_tensor_coalesced([into.view(ws, -1)], [mine], opts)

    def finish_on_stream(self, work, stage) -> None:
        """Run ``stage()`` on the exchange's stream once ``work`` has completed."""
        fut = work.get_future()
        stream = self.stream

        def _done(f) -> None:
            with cuda.stream(stream):
                f.wait()
                stage()

        fut.add_done_callback(_done)


def _begin(opts, default_opts, what: str, process_group, sync_stream) -> _Exchange:
    if isinstance(opts, ReduceOp):
        full = default_opts()
        full.reduceOp = opts
    else:
        full = opts
    if full.reduceOp not in {ReduceOp(op) for op in _SUPPORTED_OPS}:
        raise NotImplementedError(
            f"ReduceOp {full.reduceOp} is not supported "
            f"for quantized {what}, only AVG and SUM are supported"
        )
    stream = sync_stream if sync_stream is not None else cuda.Stream()
    # whatever the caller queued so far happens before the collective
    stream.wait_stream(cuda.current_stream())
    return _Exchange(process_group, full.reduceOp, full.timeout, stream)


def reduce_scatter_quantized(
    output: torch.Tensor,
    inputs: list[torch.Tensor],
    opts: ReduceScatterOptions | ReduceOp,
    process_group: Any,
    sync_stream: cuda.Stream | None = None,
):
    """
    Quantized reduce-scatter of ``inputs`` into ``output`` (a tensor from
    :func:`allocate_reduce_scatter_output`).  Only AVG and SUM are supported
    (``NotImplementedError`` otherwise).  Returns the all-to-all work; the result
    is complete once the work's future has run its callbacks and
    ``sync_stream`` has been waited on (collectives.py:159-294).
    """
    ex = _begin(opts, ReduceScatterOptions, "reduce-scatter", process_group, sync_stream)
    ws, rank = ex.world_size, ex.rank

    # views of `output`, one per input, shaped [m_pad / ws, n]
    shares = [torch.Size((p[0] // ws,) + tuple(p[1:])) for p in get_padded_sizes(inputs, ws)]
    share_views = [
        flat.view(shape)
        for flat, shape in zip(output.split([s.numel() for s in shares]), shares)
    ]

    with cuda.stream(ex.stream):
        bucket = _q.prepare(inputs, ws)  # one walk over the list for both kernels
        packed = bucket.quantize()
        received, work = ex.scatter_slots(packed)
        work.wait()

        def reduce_then_dequantize() -> None:
            # `bucket` keeps the inputs alive, `share_views` the output, until this has been queued
            bucket.reduce(received, rank, ex.reduce_op)
            own = received.view(ws, -1).split(1)[rank].squeeze(0)
            # one slot has the layout of a group of one over the [m_pad / ws, n] shares
            _q.fused_dequantize_from_fp8(share_views, own, 1)

        ex.finish_on_stream(work, reduce_then_dequantize)
    return work


def allreduce_quantized(
    tensors: list[torch.Tensor],
    opts: AllreduceOptions | ReduceOp,
    process_group: Any,
    sync_stream: cuda.Stream | None = None,
    *,
    divide_by: float | None = None,
    prepared: "_q.PreparedBucket | None" = None,
):
    """
    Quantized all-reduce of ``tensors`` in place.  Only AVG and SUM are
    supported (``NotImplementedError`` otherwise).  Returns the all-gather work;
    the tensors hold the result once the work's future has run its callbacks
    and ``sync_stream`` has been waited on (collectives.py:297-415).

    ``divide_by`` (no counterpart in the reference's function): the tensors are
    left as if each had then been divided by that Python number on the GPU, as
    ``Manager.allreduce`` does with the number of participants
    (manager.py:450-452), at no extra pass over them.

    ``prepared`` (no counterpart either): the result of
    :func:`torchft_amd.quantization.prepare` for these very tensors and this group size.
    A bucket that is reduced every step prepares once and passes it in, which takes the walk
    over the tensor list out of every step.
    """
    ex = _begin(opts, AllreduceOptions, "allreduce", process_group, sync_stream)
    ws, rank = ex.world_size, ex.rank

    # the bucket's kernels read and write the addresses bound by prepare(): tensors that are not
    # those, or have moved since, would be left untouched without a word
    if prepared is not None and (prepared.ws != ws or not prepared.matches(tensors)):
        raise ValueError("`prepared` was made for another group size or for other tensors than these "
                         "(other shapes, strides, dtype, device, or storage that has moved since): prepare again")

    with cuda.stream(ex.stream):
        # one walk over the list for all three kernels; the bucket holds the tensors, so the
        # memory behind the addresses it has bound outlives the dequantize kernel queued below
        bucket = prepared if prepared is not None else _q.prepare(tensors, ws)
        packed = bucket.quantize()
        received, a2a = ex.scatter_slots(packed)
        a2a.wait()
        bucket.reduce(received, rank, ex.reduce_op)
        # the reduced slots of all ranks land in the first buffer
        work = ex.gather_slots(packed, received)
        work.wait()  # a stream dependency with RCCL, not a host block
        ex.finish_on_stream(work, lambda: bucket.dequantize(packed, divide_by))
    return work
