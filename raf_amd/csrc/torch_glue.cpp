// CPython module `_torch_glue`: walks Python lists of torch tensors at C speed for the operator
// front end (raf_amd/op.py).  RAF's own front end converts a Python argument list into values
// through its FFI on every call (python/raf/optim/lans.py:89-102 builds `tensor_list` per step);
// for lists of thousands of tensors that conversion, done with Python-level calls, costs several
// times the GPU time of the step it precedes.  Here the list is read through torch's C++ object
// layout instead: a tensor's address, dtype, device and shape are a few loads each.
//
//   describe(tensors, descs_addr, shapes_addr, shapes_capacity, ptrs_addr) -> dims used
//       fills rafhip_tensor_desc[len] (include/rafhip_dialect.h), their shapes back to back
//       into int64[shapes_capacity] and the data pointers into uint64[len]
//   same_storage(tensors, ptrs_addr) -> bool
//       whether every tensor's data pointer still equals the recorded one (x.data = ..., set_()
//       and resize_() move it without replacing the Python object)
//   diff_range(a, b) -> (first, end)
//       the smallest index range outside which two equally long lists hold the very same
//       objects; (-1, -1) if they agree everywhere
//   signature(descs_addr, n) -> bytes
//       dtype, device and shape of every descriptor packed into one bytes object: what two
//       lists must share to be served by one OpEnv
//   rebind(tensors, first, end, descs_addr, ptrs_addr) -> bool
//       brings descriptors and recorded pointers of a list described earlier up to date with
//       `tensors`, of which [first, end) are other objects than the ones described: True, and the
//       addresses of that range written, if those have the recorded dtype, device and shape and
//       every tensor outside the range still lives at its recorded address; False, and nothing
//       written, otherwise
//
//   unreferenced(tensors, first, end) -> bool
//       whether the list holds the only Python reference to every object in [first, end): nobody
//       can pass those objects again
//   grads(params) -> (list, missing)
//       the `.grad` of every parameter (None where there is none) and how many are None
//
// torch is used for nothing but this object access; no kernels, no allocator, no dispatcher.
#include <Python.h>

#include <ATen/core/Tensor.h>
#include <torch/csrc/autograd/python_variable.h>

#include <cstdint>
#include <exception>
#include <vector>

#include "rafhip_dialect.h"

namespace {

constexpr int kDevCpu = 1, kDevRocm = 10;  // include/raf/device.h:37-50

bool dtype_of(c10::ScalarType t, int32_t* code, int32_t* bits) {
  switch (t) {
    case c10::ScalarType::Float: *code = 2; *bits = 32; return true;
    case c10::ScalarType::Half: *code = 2; *bits = 16; return true;
    case c10::ScalarType::Double: *code = 2; *bits = 64; return true;
    case c10::ScalarType::BFloat16: *code = 4; *bits = 16; return true;
    case c10::ScalarType::Int: *code = 0; *bits = 32; return true;
    case c10::ScalarType::Long: *code = 0; *bits = 64; return true;
    case c10::ScalarType::Byte: *code = 1; *bits = 8; return true;
    case c10::ScalarType::Char: *code = 0; *bits = 8; return true;
    case c10::ScalarType::Short: *code = 0; *bits = 16; return true;
    default: return false;
  }
}

bool list_arg(PyObject* o, const char* what) {
  if (PyList_CheckExact(o)) return true;
  PyErr_Format(PyExc_TypeError, "%s must be a list", what);
  return false;
}

const at::Tensor* tensor_at(PyObject* list, Py_ssize_t i) {
  PyObject* o = PyList_GET_ITEM(list, i);
  if (!THPVariable_Check(o)) {  // two pointer comparisons for Tensor and Parameter themselves
    PyErr_Format(PyExc_TypeError, "expected a tensor, got %s", Py_TYPE(o)->tp_name);
    return nullptr;
  }
  return &THPVariable_Unpack(o);
}

PyObject* describe_impl(PyObject* args) {
  PyObject* list;
  unsigned long long descs_addr, shapes_addr, ptrs_addr;
  long long shapes_cap;
  if (!PyArg_ParseTuple(args, "OKKLK", &list, &descs_addr, &shapes_addr, &shapes_cap, &ptrs_addr))
    return nullptr;
  if (!list_arg(list, "tensors")) return nullptr;
  auto* descs = reinterpret_cast<rafhip_tensor_desc*>(descs_addr);
  auto* shapes = reinterpret_cast<int64_t*>(shapes_addr);
  auto* ptrs = reinterpret_cast<uint64_t*>(ptrs_addr);
  long long used = 0;
  const Py_ssize_t n = PyList_GET_SIZE(list);
  for (Py_ssize_t i = 0; i < n; ++i) {
    const at::Tensor* t = tensor_at(list, i);
    if (!t) return nullptr;
    if (!t->is_contiguous()) {
      PyErr_SetString(PyExc_ValueError, "tensors must be contiguous");
      return nullptr;
    }
    rafhip_tensor_desc& d = descs[i];
    if (!dtype_of(t->scalar_type(), &d.dtype_code, &d.dtype_bits)) {
      PyErr_Format(PyExc_TypeError, "tensor %zd has a dtype the operators do not take", i);
      return nullptr;
    }
    const auto sizes = t->sizes();
    if (used + (long long)sizes.size() > shapes_cap) {
      PyErr_SetString(PyExc_ValueError, "shape buffer too small");
      return nullptr;
    }
    d.data = t->data_ptr();
    // torch on ROCm reports its devices as "cuda"; they are ROCm devices for RAF's purposes.
    d.device_type = t->is_cuda() ? kDevRocm : kDevCpu;
    d.device_id = t->is_cuda() && t->device().has_index() ? t->device().index() : 0;
    d.ndim = (int32_t)sizes.size();
    d.shape = shapes + used;
    for (int64_t s : sizes) shapes[used++] = s;
    ptrs[i] = reinterpret_cast<uint64_t>(d.data);
  }
  return PyLong_FromLongLong(used);
}

PyObject* same_storage_impl(PyObject* args) {
  PyObject* list;
  unsigned long long ptrs_addr;
  if (!PyArg_ParseTuple(args, "OK", &list, &ptrs_addr)) return nullptr;
  if (!list_arg(list, "tensors")) return nullptr;
  const auto* want = reinterpret_cast<const uint64_t*>(ptrs_addr);
  const Py_ssize_t n = PyList_GET_SIZE(list);
  for (Py_ssize_t i = 0; i < n; ++i) {
    const at::Tensor* t = tensor_at(list, i);
    if (!t) return nullptr;
    if (reinterpret_cast<uint64_t>(t->data_ptr()) != want[i]) Py_RETURN_FALSE;
  }
  Py_RETURN_TRUE;
}

PyObject* diff_range_impl(PyObject* args) {
  PyObject *a, *b;
  if (!PyArg_ParseTuple(args, "OO", &a, &b)) return nullptr;
  if (!list_arg(a, "a") || !list_arg(b, "b")) return nullptr;
  const Py_ssize_t n = PyList_GET_SIZE(a);
  if (PyList_GET_SIZE(b) != n) {
    PyErr_SetString(PyExc_ValueError, "the lists differ in length");
    return nullptr;
  }
  Py_ssize_t first = 0, end = n;
  while (first < n && PyList_GET_ITEM(a, first) == PyList_GET_ITEM(b, first)) ++first;
  if (first == n) return Py_BuildValue("(nn)", (Py_ssize_t)-1, (Py_ssize_t)-1);
  while (end > first && PyList_GET_ITEM(a, end - 1) == PyList_GET_ITEM(b, end - 1)) --end;
  return Py_BuildValue("(nn)", first, end);
}

PyObject* signature_impl(PyObject* args) {
  unsigned long long descs_addr;
  long long n;
  if (!PyArg_ParseTuple(args, "KL", &descs_addr, &n)) return nullptr;
  const auto* descs = reinterpret_cast<const rafhip_tensor_desc*>(descs_addr);
  std::vector<int64_t> words;
  words.reserve((size_t)(n > 0 ? n : 0) * 7 + 1);
  words.push_back(n);
  for (long long i = 0; i < n; ++i) {
    const rafhip_tensor_desc& d = descs[i];
    words.push_back(((int64_t)d.device_type << 32) | (uint32_t)d.device_id);
    words.push_back(((int64_t)d.dtype_code << 40) | ((int64_t)d.dtype_bits << 32) | (uint32_t)d.ndim);
    for (int32_t k = 0; k < d.ndim; ++k) words.push_back(d.shape[k]);
  }
  return PyBytes_FromStringAndSize(reinterpret_cast<const char*>(words.data()),
                                   (Py_ssize_t)(words.size() * sizeof(int64_t)));
}

PyObject* rebind_impl(PyObject* args) {
  PyObject* list;
  long long first, end;
  unsigned long long descs_addr, ptrs_addr;
  if (!PyArg_ParseTuple(args, "OLLKK", &list, &first, &end, &descs_addr, &ptrs_addr)) return nullptr;
  if (!list_arg(list, "tensors")) return nullptr;
  const Py_ssize_t n = PyList_GET_SIZE(list);
  if (first < 0 || end < first || end > (long long)n) {
    PyErr_SetString(PyExc_IndexError, "range outside the list");
    return nullptr;
  }
  auto* descs = reinterpret_cast<rafhip_tensor_desc*>(descs_addr);
  auto* ptrs = reinterpret_cast<uint64_t*>(ptrs_addr);
  for (Py_ssize_t i = 0; i < n; ++i) {
    const at::Tensor* t = tensor_at(list, i);
    if (!t) return nullptr;
    if (i < first || i >= end) {
      if (reinterpret_cast<uint64_t>(t->data_ptr()) != ptrs[i]) Py_RETURN_FALSE;
      continue;
    }
    const rafhip_tensor_desc& d = descs[i];
    int32_t code = 0, bits = 0;
    if (!t->is_contiguous() || !dtype_of(t->scalar_type(), &code, &bits) || code != d.dtype_code ||
        bits != d.dtype_bits || (t->is_cuda() ? kDevRocm : kDevCpu) != d.device_type ||
        (t->is_cuda() && t->device().has_index() ? t->device().index() : 0) != d.device_id)
      Py_RETURN_FALSE;
    const auto sizes = t->sizes();
    if ((int32_t)sizes.size() != d.ndim) Py_RETURN_FALSE;
    for (int32_t k = 0; k < d.ndim; ++k)
      if (sizes[(size_t)k] != d.shape[k]) Py_RETURN_FALSE;
  }
  for (Py_ssize_t i = (Py_ssize_t)first; i < (Py_ssize_t)end; ++i) {
    void* p = THPVariable_Unpack(PyList_GET_ITEM(list, i)).data_ptr();
    descs[i].data = p;
    ptrs[i] = reinterpret_cast<uint64_t>(p);
  }
  Py_RETURN_TRUE;
}

PyObject* unreferenced_impl(PyObject* args) {
  PyObject* list;
  long long first, end;
  if (!PyArg_ParseTuple(args, "OLL", &list, &first, &end)) return nullptr;
  if (!list_arg(list, "tensors")) return nullptr;
  if (first < 0 || end < first || end > (long long)PyList_GET_SIZE(list)) {
    PyErr_SetString(PyExc_IndexError, "range outside the list");
    return nullptr;
  }
  for (Py_ssize_t i = (Py_ssize_t)first; i < (Py_ssize_t)end; ++i)
    if (Py_REFCNT(PyList_GET_ITEM(list, i)) != 1) Py_RETURN_FALSE;
  Py_RETURN_TRUE;
}

PyObject* grads_impl(PyObject* args) {
  PyObject* list;
  if (!PyArg_ParseTuple(args, "O", &list)) return nullptr;
  if (!list_arg(list, "params")) return nullptr;
  static PyObject* const name = PyUnicode_InternFromString("grad");
  const Py_ssize_t n = PyList_GET_SIZE(list);
  PyObject* out = PyList_New(n);
  if (!out) return nullptr;
  Py_ssize_t missing = 0;
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* g = PyObject_GetAttr(PyList_GET_ITEM(list, i), name);  // new reference
    if (!g) {
      Py_DECREF(out);
      return nullptr;
    }
    missing += g == Py_None;
    PyList_SET_ITEM(out, i, g);  // steals it
  }
  return Py_BuildValue("(Nn)", out, missing);
}

// No C++ exception may reach the interpreter: torch raises c10::Error for tensors without storage.
template <PyObject* (*F)(PyObject*)>
PyObject* guarded(PyObject*, PyObject* args) {
  try {
    return F(args);
  } catch (const std::exception& e) {
    PyErr_SetString(PyExc_RuntimeError, e.what());
  } catch (...) {
    PyErr_SetString(PyExc_RuntimeError, "unknown C++ exception");
  }
  return nullptr;
}

PyMethodDef kMethods[] = {
    {"describe", guarded<describe_impl>, METH_VARARGS, "fill descriptors, shapes and data pointers of a tensor list"},
    {"same_storage", guarded<same_storage_impl>, METH_VARARGS, "whether the tensors' data pointers equal the recorded ones"},
    {"diff_range", guarded<diff_range_impl>, METH_VARARGS, "index range outside which two lists hold the same objects"},
    {"rebind", guarded<rebind_impl>, METH_VARARGS, "bring a described list up to date with tensors that replace a range of it"},
    {"unreferenced", guarded<unreferenced_impl>, METH_VARARGS, "whether the list holds the only reference to a range of its objects"},
    {"grads", guarded<grads_impl>, METH_VARARGS, "the .grad of every parameter and the number of missing ones"},
    {"signature", guarded<signature_impl>, METH_VARARGS, "dtype, device and shape of every descriptor as bytes"},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef kModule = {PyModuleDef_HEAD_INIT, "_torch_glue", nullptr, -1, kMethods, nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__torch_glue(void) { return PyModule_Create(&kModule); }
