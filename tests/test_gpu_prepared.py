"""The prepared bucket (torchft_amd.quantization.prepare), per-call tensor addresses and the
host cost of the path, on a gfx950 GPU.

A plan holds shapes only; addresses travel with every call.  These tests check that a bucket
prepared once gives the bytes of the three functions the reference names, for short lists
(descriptors in the kernel arguments) and long ones (device table + address buffer), that
calls on the same shapes with new addresses every time neither block the host nor mix up
addresses, and that the persistent DiLoCo buckets equal the per-call ones.
"""

import time

import pytest
import torch
from torch.distributed import ReduceOp

import sim
from sim_pg import SimGroup
from test_gpu_collectives import run_ranks
from test_gpu_parity import q, same_bytes  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu


def make_list(n_tensors, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    shapes = [(37, 4096), (50, 333), (1900,), (64, 64), (9, 1000), (3, 14336), (130, 72)]
    return [(torch.randn(shapes[i % len(shapes)], generator=g) * 0.05 * (1 + i % 3)).to(dtype).cuda()
            for i in range(n_tensors)]


@pytest.mark.parametrize("n_tensors", [1, 7, 16, 17, 40, 600])
@pytest.mark.parametrize("op", [ReduceOp.SUM, ReduceOp.AVG])
def test_prepared_bucket_equals_named_functions(q, n_tensors, op):
    ws, rank = 4, 1
    peers = [make_list(n_tensors, 100 + p) for p in range(ws)]
    by_name = [q.fused_quantize_into_fp8(list(t), ws) for t in peers]
    buckets = [q.prepare(t, ws) for t in peers]
    assert buckets[0].output_size == by_name[0].numel()
    for rep in range(3):  # the same bucket again and again
        for b, want in zip(buckets, by_name):
            same_bytes(b.quantize(), want, f"quantize, use {rep}")
    # into a buffer of the caller's
    mine = torch.full((buckets[0].output_size,), 0xEE, dtype=torch.uint8, device="cuda")
    assert buckets[0].quantize(out=mine) is mine
    same_bytes(mine, by_name[0], "quantize into a given buffer")

    recv = sim.recv_buffer(by_name, rank, ws)
    want = recv.clone()
    q.fused_reduce_fp8(list(peers[0]), want, ws, rank, op)
    for rep in range(2):
        got = recv.clone()
        buckets[0].reduce(got, rank, op)
        same_bytes(got, want, f"reduce, use {rep}")

    outs_named = [torch.full_like(t, 3.0) for t in peers[0]]
    q.fused_dequantize_from_fp8(outs_named, by_name[2], ws)
    outs = [torch.full_like(t, 5.0) for t in peers[0]]
    ob = q.prepare(outs, ws)
    assert ob.plan is buckets[0].plan  # same shapes, same plan, other addresses
    for rep in range(2):
        for o in outs:
            o.fill_(9.0)
        ob.dequantize(by_name[2])
        for i, (a, b) in enumerate(zip(outs, outs_named)):
            same_bytes(a, b, f"dequantize tensor {i}, use {rep}")
    # the scaled form
    q.fused_dequantize_from_fp8(outs_named, by_name[2], ws, divide_by=3)
    ob.dequantize(by_name[2], divide_by=3)
    for i, (a, b) in enumerate(zip(outs, outs_named)):
        same_bytes(a, b, f"scaled dequantize tensor {i}")
    with pytest.raises(AssertionError, match="Output size does not match"):
        ob.dequantize(by_name[2][:-4])


@pytest.mark.parametrize("n_tensors", [3, 24])
def test_new_addresses_every_call_without_blocking(q, oracle, n_tensors):
    """The same shapes at other addresses in every call: one cached plan, the addresses of
    each call reach its kernels, and the host is never synchronised (the calls are queued
    behind a long-running kernel and return long before it ends)."""
    ws, sets = 2, 12
    lists = [make_list(n_tensors, 300 + k) for k in range(sets)]
    want = [oracle.fused_quantize_into_fp8([t.cpu() for t in ts], ws) for ts in lists]
    outs = [[torch.empty_like(t) for t in ts] for ts in lists]
    first = q.fused_quantize_into_fp8(list(lists[0]), ws)  # builds the plan (and uploads its table)
    torch.cuda.synchronize()
    plans_before = len(q._plan_cache)

    # A kernel that keeps the GPU busy for a long time, and the calls queued behind it.  (Few
    # enough of them to fit the hardware queue: a full queue would make the runtime wait.)
    blocker_done = torch.cuda.Event()
    torch.cuda._sleep(int(1.0e9))
    blocker_done.record()
    t0 = time.perf_counter()
    packed = []
    reps = 4
    for rep in range(reps):
        for k in range(sets):
            p = q.fused_quantize_into_fp8(list(lists[k]), ws)
            q.fused_dequantize_from_fp8(outs[k], p, ws)
            if rep == reps - 1:
                packed.append(p)
    enqueue_s = time.perf_counter() - t0
    still_blocked = not blocker_done.query()
    torch.cuda.synchronize()
    total_s = time.perf_counter() - t0
    print(f"{2 * reps * sets} calls queued in {enqueue_s * 1e3:.1f} ms, finished after {total_s * 1e3:.1f} ms")
    assert still_blocked and enqueue_s < 0.5 * total_s, \
        f"{2 * reps * sets} calls took {enqueue_s:.3f} s of host time: something waited for the GPU"
    assert len(q._plan_cache) == plans_before, "new addresses must not make new plans"
    same_bytes(first, want[0], "first call")
    for k in range(sets):
        same_bytes(packed[k], want[k], f"quantize of list {k}")
        ref = [torch.empty_like(t.cpu()) for t in lists[k]]
        oracle.fused_dequantize_from_fp8(ref, want[k], ws)
        for i, (a, b) in enumerate(zip(outs[k], ref)):
            same_bytes(a, b, f"dequantize of list {k} tensor {i}")


def test_prepared_bucket_on_other_streams(q):
    """A bucket prepared on one stream and used on others: the table copy and the address
    upload are waited for by event, not by luck."""
    ws = 2
    ts = make_list(30, 7)
    want = q.fused_quantize_into_fp8(list(make_list(30, 7)), ws)
    torch.cuda.synchronize()
    q._plan_cache.clear()  # the table is uploaded again, on the side stream below
    side, other = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        torch.cuda._sleep(int(2.0e8))  # the upload sits behind this
        bucket = q.prepare(ts, ws)
        a = bucket.quantize()
    with torch.cuda.stream(other):
        b = bucket.quantize()
    c = bucket.quantize()  # the default stream
    torch.cuda.synchronize()
    for got, name in ((a, "side"), (b, "other"), (c, "default")):
        same_bytes(got, want, f"quantize on the {name} stream")


def test_host_cost_of_a_prepared_bucket(q):
    """10 000 tensors: a prepared bucket's calls cost microseconds; the walk over the list is
    paid once, in prepare()."""
    import workloads
    shapes = workloads.cfg5_shapes(10000)
    ts = workloads.cfg5(0, torch.bfloat16, shapes, device="cuda")
    ws = 16
    bucket = q.prepare(ts, ws)
    packed = bucket.quantize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 50
    for _ in range(n):
        bucket.quantize(out=packed)
        bucket.reduce(packed, 3, ReduceOp.SUM)
        bucket.dequantize(packed)
    host_us = (time.perf_counter() - t0) / (3 * n) * 1e6
    torch.cuda.synchronize()
    assert host_us < 200.0, f"{host_us:.0f} us of host time per call on a prepared bucket"
    same_bytes(bucket.quantize(), q.fused_quantize_into_fp8(list(ts), ws), "10 000 tensors")


@pytest.mark.parametrize("row_width", [None, 256])
def test_persistent_buckets_equal_per_call_buckets(q, row_width):
    from torchft_amd import allreduce as ar
    ws = 2
    sizes = [(64, 48), (1000,), (7, 33), (2048,), (300,)]
    per_bucket = 4303
    group = SimGroup(ws)
    steps = 3
    g = torch.Generator().manual_seed(11)
    data = [[[(torch.randn(s, generator=g) * 0.1).to(torch.bfloat16) for s in sizes] for _ in range(ws)]
            for _ in range(steps)]
    results = {}
    for mode in ("per_call", "persistent"):
        on_gpu = [[torch.empty(s, dtype=torch.bfloat16, device="cuda") for s in sizes] for _ in range(ws)]
        keep = [ar.BucketizedAllreduce(on_gpu[r], per_bucket * 2, row_width) for r in range(ws)]
        got = []
        for step in range(steps):
            for r in range(ws):
                for dst, src in zip(on_gpu[r], data[step][r]):
                    dst.copy_(src)

            def rank_fn(r):
                pg = group.rank(r)
                if mode == "per_call":
                    works = ar.bucketize_and_allreduce(
                        on_gpu[r], per_bucket * 2, lambda t: ar.allreduce(t, pg, ws, should_quantize=True),
                        row_width=row_width)
                else:
                    works = keep[r].allreduce(pg, ws, should_quantize=True)
                for w in works:
                    assert w.wait()

            run_ranks(ws, rank_fn, group)
            torch.cuda.synchronize()
            got.append([[t.clone() for t in on_gpu[r]] for r in range(ws)])
        results[mode] = got
    for step in range(steps):
        for r in range(ws):
            for i in range(len(sizes)):
                same_bytes(results["persistent"][step][r][i], results["per_call"][step][r][i],
                           f"step {step} rank {r} tensor {i}")


@pytest.mark.parametrize("n_tensors", [3, 40])
def test_documented_binding(q, n_tensors):
    """The minimal ctypes binding shown to maintainers runs as printed and gives the bytes of
    the shipped wrapper, for a short list and for one that needs the device table; a second
    call on fresh tensors of the same shapes reuses its plan."""
    import os
    import re

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    blocks = [b for b in re.findall(r"```python\n(.*?)```", text, flags=re.S) if "class Plan" in b]
    assert len(blocks) == 1
    code = blocks[0].replace('"torchft_amd/libtftq.so"', repr(os.path.join(root, "torchft_amd", "libtftq.so")))
    scope: dict = {}
    exec(compile(code, "documented_binding", "exec"), scope)
    for seed in (1, 2):
        tensors = make_list(n_tensors, seed)
        got = scope["fused_quantize_into_fp8"](tensors, 4)
        want = q.fused_quantize_into_fp8(tensors, 4)
        torch.cuda.synchronize()
        assert got.dtype == torch.uint8 and torch.equal(got, want)
    assert len(scope["_plans"]) == 1
