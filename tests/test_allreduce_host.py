"""Bucket packing of torchft_amd.allreduce.bucketize_and_allreduce against a
restatement of torchft/local_sgd.py:499-556, on the CPU with a stand-in
all-reduce (no GPU, no process group), and the argument checks of the managed
all-reduce (manager.py:422-429)."""

import pytest
import torch
from torch.distributed import ReduceOp

from torchft_amd import allreduce as A


class _Done:
    def __init__(self):
        self._f = torch.futures.Future()
        self._f.set_result(None)

    def wait(self, timeout=None):
        return True

    def get_future(self):
        return self._f


class _DoublingGroup:
    """all-reduce of two identical replicas: SUM doubles the tensor"""

    def __init__(self):
        self.calls = []

    def allreduce(self, tensors, opts):
        assert opts.reduceOp == ReduceOp.SUM
        self.calls.append(tensors[0].numel())
        tensors[0].mul_(2)
        return _Done()


def reference_buckets(sizes, per_bucket):
    """(bucket capacity, [tensor indices]) per bucket, local_sgd.py:519-553"""
    total, offset, idx, out = sum(sizes), 0, 0, []
    while offset < total:
        chunk = min(per_bucket, total - offset)
        used, members = 0, []
        for k in range(idx, len(sizes)):
            if used + sizes[k] > chunk:
                break
            members.append(k)
            used += sizes[k]
        idx += len(members)
        out.append((chunk, members))
        offset += chunk
    return out


@pytest.mark.parametrize("sizes,per_bucket", [
    ([3, 5, 4], 8),            # exact fit
    ([10, 10, 10], 1000),      # one bucket for everything
    ([6, 6, 6, 6], 8),         # a tensor does not fit the rest of a bucket: the last one is dropped
    ([2, 9, 2], 8),            # a tensor larger than a bucket stops the packing
    ([1] * 17, 4),
])
def test_bucket_packing_follows_the_reference(sizes, per_bucket):
    pg = _DoublingGroup()
    tensors = [torch.full((n,), float(i + 1)) for i, n in enumerate(sizes)]
    works = A.bucketize_and_allreduce(
        tensors, per_bucket * 4, lambda t: A.allreduce(t, pg, 2, reduce_op=ReduceOp.SUM))
    for w in works:
        assert w.wait()
    want = reference_buckets(sizes, per_bucket)
    assert pg.calls == [c for c, _ in want]
    reduced = {k for _, members in want for k in members}
    for i, t in enumerate(tensors):
        factor = 2.0 if i in reduced else 1.0
        assert torch.equal(t, torch.full((sizes[i],), factor * (i + 1))), i


def test_reference_bucket_walkthroughs():
    # worked by hand from local_sgd.py:519-553; the module's planner and this file's restatement
    for sizes, cap in (([6, 6, 6, 6], 8), ([2, 9, 2], 8), ([3, 5, 4], 8), ([1] * 17, 4), ([10, 10, 10], 1000)):
        assert A.plan_buckets(sizes, cap) == reference_buckets(sizes, cap)
    assert A.plan_buckets([6, 6, 6, 6], 8) == [(8, [0]), (8, [1]), (8, [2])]
    assert A.plan_buckets([2, 9, 2], 8) == [(8, [0]), (5, [])]
    # four tensors of 6 elements, buckets of 8: one tensor per bucket, the offset reaches
    # the total (24) after three buckets, the fourth tensor is never packed
    assert reference_buckets([6, 6, 6, 6], 8) == [(8, [0]), (8, [1]), (8, [2])]
    # a 9-element tensor never fits a bucket of 8: one bucket with the first tensor, one
    # empty bucket of the 5 remaining elements, nothing else
    assert reference_buckets([2, 9, 2], 8) == [(8, [0]), (5, [])]
    assert reference_buckets([3, 5, 4], 8) == [(8, [0, 1]), (4, [2])]


def test_bucket_rows_are_whole_with_row_width():
    seen = []

    def fake(t):
        seen.append(tuple(t.shape))
        t.mul_(3)
        return A._ChainedWork(_Done(), t)

    tensors = [torch.ones(5), torch.ones(6) * 2]
    works = A.bucketize_and_allreduce(tensors, 64, fake, row_width=4)
    for w in works:
        w.wait()
    assert seen == [(3, 4)]  # 11 elements in rows of 4, the last one zero
    assert torch.equal(tensors[0], torch.full((5,), 3.0)) and torch.equal(tensors[1], torch.full((6,), 6.0))


def test_average_and_participation():
    pg = _DoublingGroup()
    t = torch.arange(8.0)
    w = A.allreduce(t, pg, num_participants=4)  # AVG is the default (manager.py:390)
    assert w.wait() and w.get_future().value() is t
    assert torch.equal(t, torch.arange(8.0) * 2 / 4)
    t = torch.arange(8.0)
    A.allreduce(t, pg, 2, is_participating=False).wait()
    assert torch.equal(t, torch.zeros(8))
    with pytest.raises(ValueError, match="average reduce op is only supported for floating point"):
        A.allreduce(torch.arange(8), pg, 2)
    # continuations added by the caller run after the normalisation, in order
    order = []
    t = torch.ones(4)
    w = A.allreduce(t, pg, 2)
    w.get_future().then(lambda f: order.append(("a", f.value()[0].item()))).then(
        lambda f: order.append("b"))
    w.wait()
    assert order == [("a", 1.0), "b"]
