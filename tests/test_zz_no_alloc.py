"""tftq_reduce_static: the reduce entry point that takes no device memory for the descriptor
table from its caller and allocates none (it keeps the table in a fixed array inside the
library's code object).  Called through the C ABI and checked byte for byte against
tftq_reduce on the same buffers: two calls in a row, the second on a shorter list, so that
the array still holds the longer table of the first call when the second one starts."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _plan(L, shapes, ws):
    T = len(shapes)
    sh = (ctypes.c_int64 * (2 * T))(*[v for s in shapes for v in s])
    st = (ctypes.c_int64 * (2 * T))(*[v for s in shapes for v in (s[1], 1)])
    h = ctypes.c_void_p()
    assert L.tftq_plan_create(2, T, sh, st, ws, ctypes.byref(h)) == 0
    return h


def _both_ways(L, shapes, ws, rank, is_avg, seed):
    """Random packed buffer of the list's layout, reduced by tftq_reduce (table in a tensor of the
    caller's) and by tftq_reduce_static; returns the two results."""
    h = _plan(L, shapes, ws)
    size = L.tftq_plan_output_size(h)
    g = torch.Generator(device="cuda").manual_seed(seed)
    # valid contents: quantize random tensors of these shapes
    ts = [torch.randn(s, device="cuda", generator=g).to(torch.bfloat16) * (0.01 + 0.1 * (i % 5)) for i, s in enumerate(shapes)]
    T = len(ts)
    ptrs = (ctypes.c_void_p * T)(*[t.data_ptr() for t in ts])
    nbytes = L.tftq_plan_table_bytes(h)
    table = dev_ptrs = None
    if nbytes:
        host = (ctypes.c_uint8 * nbytes).from_address(L.tftq_plan_table_host(h))
        table = torch.frombuffer(host, dtype=torch.uint8).cuda()
        dev_ptrs = torch.empty(T, dtype=torch.int64, device="cuda")
    addr = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    dev = torch.cuda.current_device()
    packed = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert L.tftq_quantize(h, ptrs, addr(table), addr(dev_ptrs), addr(packed), size, dev, stream) == 0
    a, b = packed.clone(), packed.clone()
    assert L.tftq_reduce(h, addr(table), addr(a), size, rank, is_avg, dev, stream) == 0
    # nothing is allocated: neither in torch's allocator nor, as far as the driver's count of
    # free device memory shows, behind its back
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    assert L.tftq_reduce_static(h, addr(b), size, rank, is_avg, dev, stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    # error paths queue nothing
    assert L.tftq_reduce_static(h, addr(b), size - 4, rank, is_avg, dev, stream) == -4
    assert L.tftq_reduce_static(h, addr(b), size, ws, is_avg, dev, stream) == -1
    torch.cuda.synchronize()
    L.tftq_plan_destroy(h)
    return a.cpu(), b.cpu(), packed.cpu()


def test_reduce_static_equals_reduce_twice_in_a_row():
    from torchft_amd import _lib
    L = _lib.load()
    assert torch.cuda.is_available() and L.tftq_check_device(0) == 0
    cols = [72, 4096, 1, 333, 64, 1000, 14336, 17, 256, 5]
    long_list = [(3 + (7 * i) % 50, cols[i % len(cols)]) for i in range(90)]
    short_list = [(5 + (3 * i) % 20, cols[(i + 3) % len(cols)]) for i in range(24)]
    a, b, start = _both_ways(L, long_list, 4, 1, 1, seed=1)
    assert not torch.equal(a, start)
    assert torch.equal(a, b), "first call (90 tensors)"
    a, b, start = _both_ways(L, short_list, 8, 5, 0, seed=2)  # the array still holds the longer table
    assert not torch.equal(a, start)
    assert torch.equal(a, b), "second call (24 tensors)"
    a, b, _ = _both_ways(L, long_list[:9], 3, 2, 1, seed=3)  # a short list: descriptors in the kernel arguments
    assert torch.equal(a, b), "third call (9 tensors)"


def test_reduce_static_refuses_tables_beyond_its_array():
    from torchft_amd import _lib
    L = _lib.load()
    h = _plan(L, [(4, 40)] * 7000, 2)
    assert L.tftq_plan_table_bytes(h) > 512 * 1024
    size = L.tftq_plan_output_size(h)
    buf = torch.zeros(size, dtype=torch.uint8, device="cuda")
    rc = L.tftq_reduce_static(h, ctypes.c_void_p(buf.data_ptr()), size, 0, 0, torch.cuda.current_device(), None)
    assert rc == -8
    assert b"fixed array" in L.tftq_strerror(rc)
    L.tftq_plan_destroy(h)
    h = _plan(L, [(4, 40)] * 2000, 2)  # this one fits
    assert 0 < L.tftq_plan_table_bytes(h) <= 512 * 1024
    L.tftq_plan_destroy(h)


def test_reduce_static_is_busy_for_other_streams_until_its_kernel_has_finished():
    """All calls on a device share one array.  A second call on the same stream is ordered
    behind the first; on another stream, while the first call's kernel has not finished, it
    returns TFTQ_E_BUSY and queues nothing; once the first stream has drained it goes through."""
    from torchft_amd import _lib
    L = _lib.load()
    assert L.tftq_check_device(0) == 0
    shapes = [(5 + i % 9, 40 + 8 * (i % 7)) for i in range(30)]
    ws, rank = 2, 1
    h = _plan(L, shapes, ws)
    size = L.tftq_plan_output_size(h)
    nbytes = L.tftq_plan_table_bytes(h)
    host = (ctypes.c_uint8 * nbytes).from_address(L.tftq_plan_table_host(h))
    table = torch.frombuffer(host, dtype=torch.uint8).cuda()
    ts = [torch.randn(s, device="cuda").to(torch.bfloat16) for s in shapes]
    ptrs = (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    dev_ptrs = torch.empty(len(ts), dtype=torch.int64, device="cuda")
    packed = torch.empty(size, dtype=torch.uint8, device="cuda")
    dev = torch.cuda.current_device()
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    assert L.tftq_quantize(h, ptrs, p(table), p(dev_ptrs), p(packed), size, dev,
                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    want = packed.clone()
    assert L.tftq_reduce(h, p(table), p(want), size, rank, 0, dev,
                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    a, b, c = packed.clone(), packed.clone(), packed.clone()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        torch.cuda._sleep(int(4.0e8))  # the first call's kernels sit behind this
    raw1, raw2 = ctypes.c_void_p(s1.cuda_stream), ctypes.c_void_p(s2.cuda_stream)
    assert L.tftq_reduce_static(h, p(a), size, rank, 0, dev, raw1) == 0
    assert L.tftq_reduce_static(h, p(b), size, rank, 0, dev, raw1) == 0      # same stream: ordered
    rc = L.tftq_reduce_static(h, p(c), size, rank, 0, dev, raw2)               # another stream: refused
    assert rc == -9 and b"still in use" in L.tftq_strerror(rc)
    s1.synchronize()
    assert torch.equal(c, packed), "a refused call must not have touched its buffer"
    assert L.tftq_reduce_static(h, p(c), size, rank, 0, dev, raw2) == 0      # now it goes through
    torch.cuda.synchronize()
    for got, name in ((a, "first"), (b, "second, same stream"), (c, "third, other stream")):
        assert torch.equal(got, want), name
    L.tftq_plan_destroy(h)


def test_reduce_static_under_stream_capture():
    """A stream capture (global mode) is invalidated by any call that allocates or
    synchronises: tftq_reduce_static on a long list is recorded in one, and the graph's
    replays give the bytes of tftq_reduce."""
    from torchft_amd import _lib
    L = _lib.load()
    assert L.tftq_check_device(0) == 0   # looks up the array's address outside the capture
    shapes = [(4 + i % 11, 24 + 4 * (i % 13)) for i in range(40)]
    ws, rank = 4, 3
    h = _plan(L, shapes, ws)
    size = L.tftq_plan_output_size(h)
    nbytes = L.tftq_plan_table_bytes(h)
    host = (ctypes.c_uint8 * nbytes).from_address(L.tftq_plan_table_host(h))
    table = torch.frombuffer(host, dtype=torch.uint8).cuda()
    ts = [torch.randn(s, device="cuda").to(torch.bfloat16) for s in shapes]
    ptrs = (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    dev_ptrs = torch.empty(len(ts), dtype=torch.int64, device="cuda")
    packed = torch.empty(size, dtype=torch.uint8, device="cuda")
    dev = torch.cuda.current_device()
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    cur = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.tftq_quantize(h, ptrs, p(table), p(dev_ptrs), p(packed), size, dev, cur) == 0
    want = packed.clone()
    assert L.tftq_reduce(h, p(table), p(want), size, rank, 1, dev, cur) == 0
    work = packed.clone()
    torch.cuda.synchronize()
    cap = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(cap):
        with torch.cuda.graph(graph, stream=cap):
            rc = L.tftq_reduce_static(h, p(work), size, rank, 1, dev, ctypes.c_void_p(cap.cuda_stream))
    assert rc == 0
    for rep in range(3):
        work.copy_(packed)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(work, want), f"replay {rep}"
    L.tftq_plan_destroy(h)
