// _pylist: one walk over a Python list of tensors, in C++.
//
// The three functions of torchft/quantization.py walk their tensor list on every call
// (_prepare_quantize_fp8, quantization.py:462-515: device, dtype, dimensions, shapes,
// strides, addresses).  In Python that walk costs about half a microsecond per tensor and
// check, milliseconds for a list of 10 000 tensors whose kernels take 50 us.  scan() makes
// all the checks against the arrays of a cached plan and collects the addresses in one
// pass of a few nanoseconds per tensor.  It decides nothing on its own: any tensor that
// does not match sends the caller back to the Python walk, which builds a new plan or
// raises the reference's assertion.
//
// Host code only; built with the host compiler against the Python and libtorch headers
// (torchft_amd/_build.py).  Not part of libtftq.so, whose C ABI has no Python or torch
// types.

#include <Python.h>

#include <torch/csrc/autograd/python_variable.h>

#include <ATen/core/Tensor.h>

namespace {

// scan(tensors, dtype, device, shapes, strides, pointers, n) -> int
//   tensors   a list
//   dtype     0 = float32, 1 = float16, 2 = bfloat16 (the TFTQ_* codes of tftq.h)
//   device    ordinal of the GPU every tensor must be on (-1: host memory; the tests of this
//             walk run where there is no GPU)
//   shapes    address of int64[n][2]: the sizes every tensor must have
//   strides   address of int64[n][2]: the strides every tensor must have
//   pointers  address of uint64[n] that receives the tensors' addresses (0: not wanted)
//   n         length the list must have
// Returns n when every element is a plain 2-D tensor of that dtype on that device with
// those sizes and strides (or the 1-D tensor that unsqueeze(1) turns into such a one); the index of the first element that is not, otherwise (the
// addresses before it have then been written); -1 when `tensors` is not a list of n elements.
PyObject *scan(PyObject *, PyObject *args)
{
    PyObject *list = nullptr;
    int dtype_code = 0, device = 0;
    unsigned long long a_shapes = 0, a_strides = 0, a_pointers = 0;
    Py_ssize_t n = 0;
    if (!PyArg_ParseTuple(args, "OiiKKKn", &list, &dtype_code, &device, &a_shapes, &a_strides, &a_pointers, &n))
        return nullptr;
    if (!PyList_CheckExact(list) || PyList_GET_SIZE(list) != n) return PyLong_FromLong(-1);
    const at::ScalarType want = dtype_code == 0   ? at::kFloat
                                : dtype_code == 1 ? at::kHalf
                                                  : at::kBFloat16;
    const int64_t *shapes = reinterpret_cast<const int64_t *>(static_cast<uintptr_t>(a_shapes));
    const int64_t *strides = reinterpret_cast<const int64_t *>(static_cast<uintptr_t>(a_strides));
    uint64_t *pointers = reinterpret_cast<uint64_t *>(static_cast<uintptr_t>(a_pointers));
    Py_ssize_t i = 0;
    try {
        for (; i < n; i++) {
            PyObject *o = PyList_GET_ITEM(list, i);
            if (!THPVariable_CheckExact(o) && !THPVariable_Check(o)) break;
            const at::Tensor &t = THPVariable_Unpack(o);
            // tensor subclasses that intercept operations (fake, functional, distributed
            // tensors) answer for themselves in Python
            if (!t.defined() || t.unsafeGetTensorImpl()->is_python_dispatch()) break;
            const int64_t dim = t.dim();
            if ((dim != 2 && dim != 1) || t.scalar_type() != want) break;
            const c10::Device d = t.device();
            if (device >= 0 ? (!d.is_cuda() || d.index() != device) : !d.is_cpu()) break;
            const c10::IntArrayRef sz = t.sizes(), st = t.strides();
            // a 1-D tensor of k elements stands for its [k, 1] view (quantization.py:487-488)
            if (sz[0] != shapes[2 * i] || (dim == 2 ? sz[1] : 1) != shapes[2 * i + 1]) break;
            if (st[0] != strides[2 * i] || (dim == 2 ? st[1] : 1) != strides[2 * i + 1]) break;
            if (pointers) pointers[i] = static_cast<uint64_t>(reinterpret_cast<uintptr_t>(t.data_ptr()));
        }
    } catch (...) {
        // whatever this tensor is, the Python walk will say it in the reference's words
    }
    return PyLong_FromSsize_t(i);
}

PyMethodDef methods[] = {
    {"scan", scan, METH_VARARGS,
     "scan(tensors, dtype, device, shapes, strides, pointers, n): check a list of tensors against a plan's "
     "arrays and collect their addresses; returns n, the index of the first mismatch, or -1"},
    {nullptr, nullptr, 0, nullptr},
};

PyModuleDef module = {PyModuleDef_HEAD_INIT, "_pylist", "C++ walk over lists of tensors", -1, methods,
                      nullptr, nullptr, nullptr, nullptr};

}  // namespace

#ifndef TFTQ_PYLIST_ID
#define TFTQ_PYLIST_ID "unknown"
#endif

PyMODINIT_FUNC PyInit__pylist(void)
{
    PyObject *m = PyModule_Create(&module);
    // identifies the source the module was built from (a hash that the build passes in)
    if (m && PyModule_AddStringConstant(m, "BUILD_ID", TFTQ_PYLIST_ID) != 0) {
        Py_DECREF(m);
        return nullptr;
    }
    return m;
}
