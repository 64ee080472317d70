// Descriptors of a list of torch tensors without one DLPack capsule per tensor: the per-tensor
// loop of the reference's ExtractDlpackTensor + ExtractTensorMetaFromDlm
// (axon/python/src/dlpack_helpers.cpp:136-156, 696-724) for the case where every producer is a
// plain torch.Tensor.  The fields come from torch's own converter (at::toDLPackNonOwning, the
// code Tensor.__dlpack__ ends in, minus the allocation of a managed tensor and a capsule), so
// dtype codes, device types and the strides of size-1 dimensions are what the capsule would
// carry.
//
// describe(sequence, device_id) -> (descs: bytearray, dims: bytearray, owners: list) | None
//   descs   n * sizeof(axr_tensor_t); shape/strides point into `dims`
//   dims    the copied shapes and strides (int64)
//   owners  the tensors themselves (they own the memory the descriptors name)
// None when any element is not exactly a torch.Tensor, requires grad, carries the conjugate or
// negative bit, is not strided, lives on another GPU than `device_id`, or is refused by the
// converter: the caller then takes the capsule route, which gives Tensor.__dlpack__'s answer.
//
// Built against the torch that is installed; importable only after `import torch`.
#include <torch/csrc/autograd/python_variable.h>
#include <ATen/DLConvertor.h>

#include <Python.h>

#include <cstdint>
#include <cstring>

#include "axon_rocm.h"

static_assert(sizeof(axr_tensor_t) == sizeof(DLTensor), "axr_tensor_t mirrors DLTensor");
static_assert(offsetof(axr_tensor_t, shape) == offsetof(DLTensor, shape), "axr_tensor_t mirrors DLTensor");
static_assert(offsetof(axr_tensor_t, byte_offset) == offsetof(DLTensor, byte_offset), "axr_tensor_t mirrors DLTensor");

namespace {

// The tensor behind `obj` when the capsule route would export it unchanged, else nullptr.
const at::Tensor* exportable(PyObject* obj, long device_id) {
  if (!THPVariable_CheckExact(obj)) return nullptr;
  const at::Tensor& t = THPVariable_Unpack(obj);
  if (!t.defined() || t.layout() != c10::kStrided || t.is_nested() || t.is_quantized() ||
      t.is_conj() || t.is_neg() || t._is_zerotensor() || !t.has_storage() || t.requires_grad()) {
    return nullptr;
  }
  const c10::Device dev = t.device();
  if (dev.is_cuda()) {
    if (dev.index() != device_id) return nullptr;
  } else if (!dev.is_cpu()) {
    return nullptr;
  }
  return &t;
}

PyObject* describe(PyObject*, PyObject* args) {
  PyObject* arg = nullptr;
  long device_id = -1;
  if (!PyArg_ParseTuple(args, "Ol", &arg, &device_id)) return nullptr;
  PyObject* seq = PySequence_Fast(arg, "describe() needs a sequence of tensors");
  if (!seq) return nullptr;
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
  PyObject** items = PySequence_Fast_ITEMS(seq);
  PyObject* descs = nullptr;
  PyObject* dims = nullptr;
  PyObject* owners = nullptr;
  PyObject* result = nullptr;
  bool refused = false;

  Py_ssize_t total_dims = 0;
  for (Py_ssize_t i = 0; i < n && !refused; ++i) {
    const at::Tensor* t = exportable(items[i], device_id);
    if (!t) {
      refused = true;
    } else {
      total_dims += 2 * t->dim();
    }
  }
  if (!refused) {
    descs = PyByteArray_FromStringAndSize(nullptr, n * static_cast<Py_ssize_t>(sizeof(axr_tensor_t)));
    dims = PyByteArray_FromStringAndSize(nullptr, total_dims * static_cast<Py_ssize_t>(sizeof(int64_t)));
    owners = PyList_New(n);
  }
  if (!refused && descs && dims && owners) {
    auto* out = reinterpret_cast<DLTensor*>(PyByteArray_AS_STRING(descs));
    auto* d = reinterpret_cast<int64_t*>(PyByteArray_AS_STRING(dims));
    try {
      for (Py_ssize_t i = 0; i < n; ++i) {
        const at::Tensor& t = THPVariable_Unpack(items[i]);
        at::toDLPackNonOwning(t, &out[i]);   // shape/strides point at the tensor's own arrays
        const int nd = out[i].ndim;
        if (nd > 0) {
          std::memcpy(d, out[i].shape, sizeof(int64_t) * nd);
          out[i].shape = d;
          d += nd;
          if (out[i].strides) {
            std::memcpy(d, out[i].strides, sizeof(int64_t) * nd);
            out[i].strides = d;
            d += nd;
          }
        } else {
          out[i].shape = nullptr;
          out[i].strides = nullptr;
        }
        Py_INCREF(items[i]);
        PyList_SET_ITEM(owners, i, items[i]);
      }
      result = PyTuple_Pack(3, descs, dims, owners);
    } catch (...) {   // a dtype or device the converter does not export
      refused = true;
    }
  }
  if (!result && !PyErr_Occurred()) {
    result = Py_None;
    Py_INCREF(result);
  }
  Py_XDECREF(descs);
  Py_XDECREF(dims);
  Py_XDECREF(owners);   // a partly filled list releases what it holds
  Py_DECREF(seq);
  return result;
}

PyMethodDef methods[] = {
    {"describe", describe, METH_VARARGS,
     "describe(sequence, device_id) -> (descs bytearray, dims bytearray, owners list) or None"},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef module = {PyModuleDef_HEAD_INIT, "_axr_torch", "Descriptors of torch tensors for tensor bundles.",
                      -1, methods, nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__axr_torch(void) {
  PyObject* m = PyModule_Create(&module);
  if (m) PyModule_AddIntConstant(m, "TENSOR_BYTES", static_cast<long>(sizeof(axr_tensor_t)));
  return m;
}
