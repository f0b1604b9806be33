// _fo_hostscan: the per-step check of a cached multi-tensor launch plan, as one C++ loop.
//
// Before a cached plan may be launched again, step() has to see that every parameter still owns the storage the
// launch table points at and where its gradient lives now (torch frees and reallocates gradients every iteration).
// In Python that is four attribute reads or calls per parameter, 0.25 us each: 0.9 ms for a list of 4096 tensors,
// during which the device idles at the head of every burst of steps.  This module does the same walk over the
// at::Tensor objects directly (20 ns per parameter).  It is host-side bookkeeping only: no device code, no math; the
// package falls back to the Python loop when the module has not been built (flashoptim_amd/base.py).
//
// same_objects(a, b) -> bool
//   whether the two lists hold the very same objects in the same order (the group's parameter list against the one the
//   plan was built for).
// scan(params, table_address, table_entries) -> None | tuple of (index, new_gradient_address)
//   params         list of the bucket's parameters, in table order
//   table_address  address of the bucket's fo_tensor_desc array (host copy, include/flashoptim_hip.h)
//   table_entries  its length; a list of another length is an error (ValueError)
//   None: some parameter has no gradient, does not require one, moved to other storage, or its gradient changed
//         dtype, device, size or contiguity -- the caller takes the full planning path.  Otherwise the gradients
//         that now live at another address than the table says (empty tuple: the table is current).
//         A tensor object that libtorch cannot answer these questions for (a wrapper subclass without storage)
//         also gives None.
#include <Python.h>

#include <ATen/core/Tensor.h>
#include <torch/csrc/autograd/python_variable.h>

#include <cstdint>

namespace {

struct TensorDesc {  // fo_tensor_desc
    void* param;
    const void* grad;
    void* ecc;
    void* mom;
    void* mom_scales;
    void* var;
    void* var_scales;
    int64_t n;
};
static_assert(sizeof(TensorDesc) == 64, "layout of fo_tensor_desc");

PyObject* scan(PyObject*, PyObject* args) {
    PyObject* params = nullptr;
    unsigned long long address = 0;
    Py_ssize_t entries = 0;
    if (!PyArg_ParseTuple(args, "OKn", &params, &address, &entries)) return nullptr;
    if (!PyList_CheckExact(params)) {
        PyErr_SetString(PyExc_TypeError, "scan(params, table_address, table_entries): params must be a list");
        return nullptr;
    }
    const TensorDesc* table = reinterpret_cast<const TensorDesc*>(static_cast<uintptr_t>(address));
    const Py_ssize_t n = PyList_GET_SIZE(params);
    if (n != entries || (n > 0 && table == nullptr)) {
        PyErr_SetString(PyExc_ValueError, "scan: the parameter list and the launch table differ in length");
        return nullptr;
    }
    PyObject* moved = nullptr;
    try {
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject* obj = PyList_GET_ITEM(params, i);
        bool ok = THPVariable_Check(obj);
        if (ok) {
            const at::Tensor& p = THPVariable_Unpack(obj);
            ok = p.defined() && p.requires_grad() && p.is_leaf();
            if (ok) {
                const at::Tensor& g = p.grad();
                ok = g.defined() && p.data_ptr() == table[i].param;
                if (ok) {
                    const void* ptr = g.data_ptr();
                    if (ptr != table[i].grad) {
                        ok = g.scalar_type() == p.scalar_type() && g.device() == p.device() && g.is_contiguous() &&
                             g.numel() == p.numel() && g.layout() == c10::kStrided;
                        if (ok) {
                            if (!moved) moved = PyList_New(0);
                            PyObject* item = moved ? Py_BuildValue("(nK)", i, (unsigned long long)(uintptr_t)ptr) : nullptr;
                            if (!item || PyList_Append(moved, item) != 0) {
                                Py_XDECREF(item);
                                Py_XDECREF(moved);
                                return nullptr;
                            }
                            Py_DECREF(item);
                        }
                    }
                }
            }
        }
        if (!ok) {
            Py_XDECREF(moved);
            Py_RETURN_NONE;
        }
    }
    } catch (...) {  // libtorch refused a query (e.g. data_ptr() of a tensor without storage): not a plan this walk can vouch for
        Py_XDECREF(moved);
        Py_RETURN_NONE;
    }
    if (!moved) return PyTuple_New(0);
    PyObject* out = PyList_AsTuple(moved);
    Py_DECREF(moved);
    return out;
}

PyObject* same_objects(PyObject*, PyObject* args) {
    PyObject *a = nullptr, *b = nullptr;
    if (!PyArg_ParseTuple(args, "OO", &a, &b)) return nullptr;
    if (!PyList_CheckExact(a) || !PyList_CheckExact(b)) {
        PyErr_SetString(PyExc_TypeError, "same_objects(a, b): both arguments must be lists");
        return nullptr;
    }
    const Py_ssize_t n = PyList_GET_SIZE(a);
    if (n != PyList_GET_SIZE(b)) Py_RETURN_FALSE;
    for (Py_ssize_t i = 0; i < n; ++i)
        if (PyList_GET_ITEM(a, i) != PyList_GET_ITEM(b, i)) Py_RETURN_FALSE;
    Py_RETURN_TRUE;
}

PyMethodDef methods[] = {
    {"same_objects", same_objects, METH_VARARGS, "same_objects(a, b) -> bool: the same objects in the same order"},
    {"scan", scan, METH_VARARGS, "scan(params, table_address, table_entries) -> None | tuple of (index, gradient address)"},
    {nullptr, nullptr, 0, nullptr},
};

PyModuleDef module = {PyModuleDef_HEAD_INIT, "_fo_hostscan", "per-step validation of cached launch plans", -1, methods,
                      nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__fo_hostscan(void) { return PyModule_Create(&module); }
