// Host helper of the Python entry points (no GPU code): the key under which a validated call is remembered.
// tensor_key(tuple[, open_dim0]) packs address, dtype, sizes and strides of every tensor of the tuple (None: a marker) into one
// bytes object -- hashable, compared bytewise -- in a fifth of a microsecond; the same tuple built in Python from
// data_ptr() / shape / stride() / dtype costs six.  A CPython module linked against libtorch_python for
// THPVariable_Unpack; lazy_amd/attention/_launch.py falls back to the Python tuple when it is not built.
#include <Python.h>
#include <torch/csrc/autograd/python_variable.h>
#include <ATen/core/Tensor.h>
#include <string>

static PyObject *tensor_key(PyObject *, PyObject *const *args, Py_ssize_t nargs) {
    if (nargs < 1 || nargs > 2 || !PyTuple_Check(args[0])) {
        PyErr_SetString(PyExc_TypeError, "tensor_key(tuple of tensors or None[, open_dim0: int])");
        return nullptr;
    }
    // bit i set: the first dimension of tensor i is left out of the key (a per-token or per-request count that the
    // caller handles itself)
    unsigned long long open_dim0 = 0;
    if (nargs == 2) {
        open_dim0 = PyLong_AsUnsignedLongLongMask(args[1]);
        if (PyErr_Occurred()) return nullptr;
    }
    PyObject *tup = args[0];
    const Py_ssize_t n = PyTuple_GET_SIZE(tup);
    int64_t buf[512];
    int m = 0;
    try {
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject *o = PyTuple_GET_ITEM(tup, i);
        if (m >= 500) {                              // (every write below stays inside buf: a tensor adds at most 3 + 2 x 64)
            PyErr_SetString(PyExc_ValueError, "tensor_key: too many entries");
            return nullptr;
        }
        if (o == Py_None) { buf[m++] = -1; continue; }
        if (!THPVariable_Check(o)) {
            PyErr_SetString(PyExc_TypeError, "tensor_key: not a tensor");
            return nullptr;
        }
        const at::Tensor &t = THPVariable_Unpack(o);
        const auto sizes = t.sizes();
        const auto strides = t.strides();
        if (m + 2 + 2 * (int)sizes.size() > 512) {
            PyErr_SetString(PyExc_ValueError, "tensor_key: too many dimensions");
            return nullptr;
        }
        buf[m++] = (int64_t)(intptr_t)t.data_ptr();
        buf[m++] = ((int64_t)t.scalar_type() << 8) | (int64_t)sizes.size();
        const bool open = i < 64 && ((open_dim0 >> i) & 1ull) && !sizes.empty();
        for (size_t j = 0; j < sizes.size(); ++j) buf[m++] = (open && j == 0) ? -2 : sizes[j];
        for (auto s : strides) buf[m++] = s;
    }
    } catch (const std::exception &e) {             // (a tensor without storage has no address)
        PyErr_SetString(PyExc_RuntimeError, e.what());
        return nullptr;
    }
    return PyBytes_FromStringAndSize(reinterpret_cast<const char *>(buf), (Py_ssize_t)m * 8);
}

static PyMethodDef methods[] = {
    {"tensor_key", (PyCFunction)(void (*)(void))tensor_key, METH_FASTCALL, "metadata of a tuple of tensors as bytes"},
    {nullptr, nullptr, 0, nullptr}};
static struct PyModuleDef moddef = {PyModuleDef_HEAD_INIT, "_callkey", nullptr, -1, methods};
PyMODINIT_FUNC PyInit__callkey(void) { return PyModule_Create(&moddef); }
