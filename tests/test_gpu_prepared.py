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


def _count_prepare(q, monkeypatch):
    calls = []
    real = q.prepare

    def counting(*a, **k):
        calls.append(1)
        return real(*a, **k)

    monkeypatch.setattr(q, "prepare", counting)
    return calls


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_named_functions_recognise_a_long_list(q, oracle, monkeypatch, dtype):
    """From the second call on, a list of more than 16 tensors that fits the plan of an
    earlier call is checked and its addresses collected by one C++ walk: prepare() (the walk
    in Python) is not called again, whatever tensors the list holds, and every call still
    gives the checker's bytes."""
    if q._pylist is None:
        pytest.skip("torchft_amd._pylist is not built")
    ws, rank, n = 4, 2, 40
    lists = [make_list(n, 500 + p, dtype) for p in range(ws)]  # same shapes, other tensors and addresses
    want = [oracle.fused_quantize_into_fp8([t.cpu() for t in ts], ws) for ts in lists]
    same_bytes(q.fused_quantize_into_fp8(list(lists[0]), ws), want[0], "first call")
    calls = _count_prepare(q, monkeypatch)
    packed = [q.fused_quantize_into_fp8(list(ts), ws) for ts in lists]
    packed += [q.fused_quantize_into_fp8(list(lists[1]), ws)]  # the addresses of two calls ago
    assert not calls, "the Python walk ran for a list that fits a cached plan"
    for k, (got, ref) in enumerate(zip(packed, want + [want[1]])):
        same_bytes(got, ref, f"quantize of list {k}")

    recv = sim.recv_buffer(packed[:ws], rank, ws)
    ref = sim.recv_buffer(want, rank, ws)
    for op in (ReduceOp.SUM, ReduceOp.AVG):
        got_r, ref_r = recv.clone(), ref.clone()
        q.fused_reduce_fp8(list(lists[0]), got_r, ws, rank, op)
        oracle.fused_reduce_fp8([t.cpu() for t in lists[0]], ref_r, ws, rank, op)
        same_bytes(got_r, ref_r, f"reduce {op}")

    for k in (0, 3, 0):
        outs = [torch.full_like(t, 7.0) for t in lists[k]]
        outs_ref = [torch.empty_like(t.cpu()) for t in lists[k]]
        q.fused_dequantize_from_fp8(outs, packed[k], ws)
        oracle.fused_dequantize_from_fp8(outs_ref, want[k], ws)
        for i, (a, b) in enumerate(zip(outs, outs_ref)):
            same_bytes(a, b, f"dequantize of list {k}, tensor {i}")
    assert not calls
    with pytest.raises(AssertionError, match="Output size does not match"):
        q.fused_dequantize_from_fp8(list(lists[0]), packed[0][:-4], ws)
    with pytest.raises(AssertionError, match="Output size does not match"):
        q.fused_reduce_fp8(list(lists[0]), packed[0][:-4], ws, rank)


def test_long_list_whose_tensors_move_between_calls(q, oracle, monkeypatch):
    """One list object, called again and again while its tensors change under it: storage
    that moves (`.data =`), an element replaced by a tensor of the same shape, of another
    shape, of another dtype, a 1-D element.  Every call sees the list as it is then."""
    if q._pylist is None:
        pytest.skip("torchft_amd._pylist is not built")
    ws, n = 2, 24
    ts = make_list(n, 900)

    def check(what):
        got = q.fused_quantize_into_fp8(ts, ws)
        same_bytes(got, oracle.fused_quantize_into_fp8([t.cpu() for t in ts], ws), what)
        return got

    check("first call")
    calls = _count_prepare(q, monkeypatch)
    check("same list again")
    old = ts[5]
    ts[5].data = (old.float() * 3).to(old.dtype)  # new storage, same tensor object
    assert ts[5] is old
    check("a tensor whose storage moved")
    ts[7] = (ts[7].float() - 1).to(ts[7].dtype)   # another tensor of the same shape
    packed = check("an element replaced by another tensor")
    assert not calls
    outs = [torch.empty_like(t) for t in ts]
    q.fused_dequantize_from_fp8(outs, packed, ws)
    moved = [torch.empty_like(t) for t in ts]     # all outputs somewhere else, in one call
    q.fused_dequantize_from_fp8(moved, packed, ws)
    for i, (a, b) in enumerate(zip(outs, moved)):
        same_bytes(a, b, f"dequantize into moved tensor {i}")
    assert not calls
    ts[3] = torch.randn(11, 77, device="cuda").to(ts[0].dtype)  # another shape: a new plan
    check("an element of another shape")
    assert len(calls) == 1
    check("the new shapes again")
    assert len(calls) == 1
    ts[4] = ts[4].t().contiguous().t()            # same shape, other strides
    check("an element with other strides")
    assert len(calls) == 2
    ts[6] = torch.randn(50, device="cuda").to(ts[0].dtype)      # 1-D: becomes [50, 1] in the list
    check("a 1-D element")
    assert ts[6].dim() == 2 and len(calls) == 3
    check("after the 1-D element became 2-D")
    assert len(calls) == 3
    ts[2] = ts[2].float()
    with pytest.raises(AssertionError, match="same dtype"):
        q.fused_quantize_into_fp8(ts, ws)
    ts[2] = ts[2].to(ts[0].dtype).cpu()
    with pytest.raises(AssertionError, match="same device"):
        q.fused_quantize_into_fp8(ts, ws)


def test_long_list_on_several_streams_and_under_capture(q, oracle, monkeypatch):
    """The address buffer of the fast path belongs to one device and stream: calls on other
    streams, with other tensors, do not disturb each other; a call recorded by a stream
    capture leaves nothing behind that a later call would trust."""
    if q._pylist is None:
        pytest.skip("torchft_amd._pylist is not built")
    ws, n = 2, 30
    a, b = make_list(n, 41), make_list(n, 42)
    want_a = oracle.fused_quantize_into_fp8([t.cpu() for t in a], ws)
    want_b = oracle.fused_quantize_into_fp8([t.cpu() for t in b], ws)
    q.fused_quantize_into_fp8(list(a), ws)
    torch.cuda.synchronize()
    calls = _count_prepare(q, monkeypatch)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got = []
    for rep in range(3):
        with torch.cuda.stream(s1):
            torch.cuda._sleep(int(5.0e7))
            got.append((q.fused_quantize_into_fp8(list(a), ws), want_a))
        with torch.cuda.stream(s2):
            got.append((q.fused_quantize_into_fp8(list(b), ws), want_b))
        got.append((q.fused_quantize_into_fp8(list(b if rep % 2 else a), ws), want_b if rep % 2 else want_a))
    torch.cuda.synchronize()
    for k, (g, w) in enumerate(got):
        same_bytes(g, w, f"call {k}")
    assert not calls

    # a capture records the upload of b's addresses; the eager call after it must not take
    # the buffer to hold them
    cap = torch.cuda.Stream()
    cap.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    out_b = [torch.empty_like(t) for t in b]
    packed_b = q.fused_quantize_into_fp8(list(b), ws)
    torch.cuda.synchronize()
    with torch.cuda.stream(cap):
        q.fused_dequantize_from_fp8(list(a), q.fused_quantize_into_fp8(list(a), ws), ws)  # warm the stream's state
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=cap):
            q.fused_dequantize_from_fp8(out_b, packed_b, ws)
        out_b2 = [torch.empty_like(t) for t in b]
        q.fused_dequantize_from_fp8(out_b2, packed_b, ws)  # eager, same stream, before any replay
    torch.cuda.synchronize()
    ref = [torch.empty_like(t.cpu()) for t in b]
    oracle.fused_dequantize_from_fp8(ref, want_b, ws)
    for i, (x, r) in enumerate(zip(out_b2, ref)):
        same_bytes(x, r, f"eager call after the capture, tensor {i}")
    for rep in range(2):
        for t in out_b:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for i, (x, r) in enumerate(zip(out_b, ref)):
            same_bytes(x, r, f"replay {rep}, tensor {i}")


def test_host_cost_of_the_named_functions_on_a_long_list(q):
    """10 000 tensors through the three functions the reference names: after the first call
    the host side of a call is a fraction of a millisecond."""
    if q._pylist is None:
        pytest.skip("torchft_amd._pylist is not built")
    import workloads
    shapes = workloads.cfg5_shapes(10000)
    ts = workloads.cfg5(0, torch.bfloat16, shapes, device="cuda")
    ws = 16
    packed = q.fused_quantize_into_fp8(ts, ws)
    want = q.prepare(ts, ws).quantize()
    q.fused_reduce_fp8(ts, packed.clone(), ws, 3)
    q.fused_dequantize_from_fp8(ts, packed, ws)
    torch.cuda.synchronize()
    n = 20
    t0 = time.perf_counter()
    for _ in range(n):
        p = q.fused_quantize_into_fp8(ts, ws)
        q.fused_reduce_fp8(ts, p, ws, 3, ReduceOp.SUM)
        q.fused_dequantize_from_fp8(ts, packed, ws)
    host_ms = (time.perf_counter() - t0) / n * 1e3
    torch.cuda.synchronize()
    print(f"{host_ms:.3f} ms of host time per quantize + reduce + dequantize on 10 000 tensors")
    assert host_ms < 2.0, f"{host_ms:.2f} ms of host time per step through the named functions"
    same_bytes(q.fused_quantize_into_fp8(ts, ws), want, "10 000 tensors")


@pytest.mark.parametrize("n_tensors", [1, 5, 30])
def test_prepared_bucket_is_bound_to_its_tensors(q, n_tensors):
    """`prepared=` of allreduce_quantized must be the bucket of these very tensors: a bucket of
    other tensors, or of tensors that have moved since, is refused instead of reducing the
    old addresses."""
    from torchft_amd import collectives as col
    ws = 2
    ts = make_list(n_tensors, 77)
    bucket = q.prepare(ts, ws)
    assert bucket.matches(ts) and bucket.matches(list(ts)) and bucket.matches(tuple(ts))
    flat = torch.randn(1000, device="cuda")
    one = q.prepare([flat], ws)            # the bucket holds the [1000, 1] view
    assert one.matches([flat]) and one.matches([flat.unsqueeze(1)]) and not one.matches([flat.clone()])
    assert not one.matches([flat[::2]]) and not one.matches([flat.double()])
    others = make_list(n_tensors, 77)      # same values and shapes, other addresses
    assert not bucket.matches(others) and not bucket.matches(ts[:-1]) and not bucket.matches(ts + ts[:1])
    group = SimGroup(1)
    with pytest.raises(ValueError, match="prepare again"):
        col.allreduce_quantized(others, ReduceOp.SUM, group.rank(0), prepared=bucket)
    moved = list(ts)
    moved[0].data = moved[0].clone()
    assert not bucket.matches(moved)
    with pytest.raises(ValueError, match="prepare again"):
        col.allreduce_quantized(moved, ReduceOp.SUM, group.rank(0), prepared=bucket)
    with pytest.raises(ValueError, match="prepare again"):
        col.allreduce_quantized(ts, ReduceOp.SUM, group.rank(0), prepared=q.prepare(ts, 4))


def test_first_use_of_a_bucket_under_capture(q):
    """A bucket of a long list whose first compute call is recorded by a stream capture: the
    capture holds the upload of the addresses, and eager calls after it, on this stream and
    on another, upload them themselves instead of trusting an upload that has not run."""
    ws = 2
    ts = make_list(30, 5)
    want = q.prepare(make_list(30, 5), ws).quantize()
    torch.cuda.synchronize()
    bucket = q.prepare(ts, ws)
    out = torch.empty(bucket.output_size, dtype=torch.uint8, device="cuda")
    cap = torch.cuda.Stream()
    cap.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(cap):
        with torch.cuda.graph(graph, stream=cap):
            bucket.quantize(out=out)
        eager_same = bucket.quantize()
    eager_default = bucket.quantize()
    torch.cuda.synchronize()
    same_bytes(eager_same, want, "eager call on the capture's stream")
    same_bytes(eager_default, want, "eager call on the default stream")
    for rep in range(2):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        same_bytes(out, want, f"replay {rep}")
