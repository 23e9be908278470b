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
    before = torch.cuda.memory_allocated()
    assert L.tftq_reduce_static(h, addr(b), size, rank, is_avg, dev, stream) == 0
    assert torch.cuda.memory_allocated() == before
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
