"""A process group simulated inside one process, for testing and timing the host
orchestration of the quantized collectives on a single GPU.

Every rank is a thread (as in the reference's own collective tests,
torchft/process_group_test.py:863-898) and all ranks share the one device.  Only
the two collectives the quantized path needs are provided, with the semantics
pinned by process_group_test.py:175-215 (all-gather) and :255-296 (all-to-all),
plus a SUM all-reduce for the unquantized branch of the managed all-reduce:

    alltoall_base(out, inp):                      out[p] on rank r  =  inp[r] of rank p
    allgather_into_tensor_coalesced([out], [inp]): out[p] on rank r =  inp of rank p
    allreduce([t]):                               t on every rank  =  sum_p t of rank p, p ascending

The copies are queued on each rank's current stream behind events of the
producers, so nothing blocks the host except the thread barrier that publishes
the buffers.  A rank's stream also waits until every peer has finished reading
its buffer before the collective is considered complete on that rank.
"""

from __future__ import annotations

import threading

import torch


class _DoneWork:
    """Work whose effects are already ordered on the caller's stream."""

    def wait(self, timeout=None) -> bool:
        return True

    def get_future(self) -> torch.futures.Future:
        fut: torch.futures.Future = torch.futures.Future()
        fut.set_result(None)
        return fut


class SimGroup:
    def __init__(self, world_size: int) -> None:
        self.world_size = world_size
        self.barrier = threading.Barrier(world_size)
        self.posted = [None] * world_size
        self.read_done = [None] * world_size

    def rank(self, r: int) -> "SimProcessGroup":
        return SimProcessGroup(self, r)


class SimProcessGroup:
    def __init__(self, group: SimGroup, rank: int) -> None:
        self._g = group
        self._rank = rank

    def rank(self) -> int:
        return self._rank

    def size(self) -> int:
        return self._g.world_size

    def _exchange(self, mine: torch.Tensor, pull) -> _DoneWork:
        g, r = self._g, self._rank
        stream = torch.cuda.current_stream()
        ready = torch.cuda.Event()
        ready.record(stream)
        g.posted[r] = (mine, ready)
        g.barrier.wait()
        for p in range(g.world_size):
            src, ev = g.posted[p]
            stream.wait_event(ev)
            pull(p, src)
        done = torch.cuda.Event()
        done.record(stream)
        g.read_done[r] = done
        g.barrier.wait()
        for p in range(g.world_size):
            stream.wait_event(g.read_done[p])
        g.barrier.wait()  # nobody reposts before everybody has picked up the events
        return _DoneWork()

    def alltoall_base(self, output, input, output_split_sizes, input_split_sizes, opts=None):
        assert not output_split_sizes and not input_split_sizes, "equal splits only"
        r = self._rank
        return self._exchange(input, lambda p, src: output[p].copy_(src[r], non_blocking=True))

    def allgather_into_tensor_coalesced(self, output_tensors, input_tensors, opts=None):
        assert len(output_tensors) == 1 and len(input_tensors) == 1
        out = output_tensors[0]
        return self._exchange(
            input_tensors[0], lambda p, src: out[p].copy_(src.reshape(out[p].shape), non_blocking=True))

    def allreduce(self, tensors, opts=None):
        assert len(tensors) == 1
        t = tensors[0]
        acc = torch.zeros_like(t)

        def pull(p, src):
            acc.add_(src)

        work = self._exchange(t.clone(), pull)
        t.copy_(acc)
        return work
