"""The C++ walk over a list of tensors (torchft_amd/csrc/tftq_pylist.cpp) on host tensors:
what it accepts, where it stops, what it writes."""

import ctypes

import pytest
import torch

from torchft_amd import _build


@pytest.fixture(scope="module")
def pylist():
    mod = _build.load_pylist()
    if mod is None:
        pytest.skip("torchft_amd._pylist cannot be built here")
    return mod


def arrays(ts):
    n = len(ts)
    shapes = (ctypes.c_int64 * (2 * n))(*[d for t in ts for d in t.shape])
    strides = (ctypes.c_int64 * (2 * n))(*[d for t in ts for d in t.stride()])
    ptrs = (ctypes.c_uint64 * n)()
    return shapes, strides, ptrs


def scan(pylist, ts, shapes, strides, ptrs, dtype=0, n=None):
    return pylist.scan(ts, dtype, -1, ctypes.addressof(shapes), ctypes.addressof(strides),
                       ctypes.addressof(ptrs) if ptrs is not None else 0, len(ts) if n is None else n)


def test_build_id(pylist):
    assert pylist.BUILD_ID == _build.pylist_hash()


def test_scan_accepts_and_collects(pylist):
    ts = [torch.empty(3 + i % 5, 7) for i in range(100)]
    ts[10] = torch.empty(7, 5).t()                      # strided
    ts[11] = torch.nn.Parameter(torch.empty(4, 7))      # a subclass torch itself defines
    ts[12] = torch.empty(0, 7)                          # empty
    ts[13] = torch.empty(40, 7)[3:7]                    # a view with a storage offset
    shapes, strides, ptrs = arrays(ts)
    ts[14] = ts[14][:, 0]                               # 1-D: stands for its [k, 1] view ...
    assert scan(pylist, ts, shapes, strides, ptrs) == 14
    ts[14] = torch.empty(40)[::2]
    ts[15] = torch.empty(9)
    shapes, strides, ptrs = arrays([t if t.dim() == 2 else t.unsqueeze(1) for t in ts])  # ... of these sizes and strides
    assert scan(pylist, ts, shapes, strides, ptrs) == len(ts)
    assert list(ptrs) == [t.data_ptr() for t in ts]
    assert scan(pylist, ts, shapes, strides, None) == len(ts)   # no addresses wanted


@pytest.mark.parametrize("what", ["shape", "stride", "dtype", "dim", "none", "int", "device", "subclass"])
def test_scan_stops_at_the_first_mismatch(pylist, what):
    ts = [torch.empty(4, 6) for _ in range(20)]
    shapes, strides, ptrs = arrays(ts)
    k = 13
    ts[k] = {
        "shape": lambda: torch.empty(4, 7),
        "stride": lambda: torch.empty(6, 4).t(),
        "dtype": lambda: torch.empty(4, 6, dtype=torch.float16),
        "dim": lambda: torch.empty(4, 6, 1),
        "none": lambda: None,
        "int": lambda: 5,
        "device": lambda: torch.empty(4, 6, device="meta"),
        "subclass": lambda: _Wrapper(torch.empty(4, 6)),
    }[what]()
    assert scan(pylist, ts, shapes, strides, ptrs) == k
    assert list(ptrs)[:k] == [t.data_ptr() for t in ts[:k]] and list(ptrs)[k:] == [0] * (len(ts) - k)


class _Wrapper(torch.Tensor):
    """A tensor subclass that intercepts operations in Python."""

    @staticmethod
    def __new__(cls, elem):
        return torch.Tensor._make_wrapper_subclass(cls, elem.shape, dtype=elem.dtype, device=elem.device)

    def __init__(self, elem):
        self.elem = elem

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        raise RuntimeError("not meant to be called")


def test_scan_wants_a_list_of_the_right_length(pylist):
    ts = [torch.empty(4, 6) for _ in range(5)]
    shapes, strides, ptrs = arrays(ts)
    assert scan(pylist, tuple(ts), shapes, strides, ptrs) == -1
    assert scan(pylist, ts[:4], shapes, strides, ptrs, n=5) == -1
    assert scan(pylist, ts, shapes, strides, ptrs, dtype=2) == 0   # bfloat16 wanted
    assert scan(pylist, ts, shapes, strides, ptrs, dtype=0) == 5


def test_named_functions_fall_back_without_a_gpu():
    from torchft_amd import quantization as q
    ts = [torch.empty(4, 6) for _ in range(20)]
    assert q._match_long_list(ts, 2, True) is None
    with pytest.raises(RuntimeError, match="no CPU path"):
        q.fused_quantize_into_fp8(ts, 2)
