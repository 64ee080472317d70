/* Native DLPack extraction for the Python layer: the per-tensor loop of the
 * reference's ExtractDlpackTensor + ExtractTensorMetaFromDlm
 * (axon/python/src/dlpack_helpers.cpp:136-156, 696-724) in C, so that a bundle
 * of thousands of tensors costs one `__dlpack__()` call per tensor and nothing
 * else.  The result is a ready array of axr_tensor_t (layout-identical to
 * DLTensor) for axr_plan_create / axr_plan_bind.
 *
 * describe(sequence) -> (descs: bytearray, dims: bytearray, owners: list)
 *   descs   n * sizeof(axr_tensor_t); shape/strides point into `dims`
 *   dims    the copied shapes and strides (int64)
 *   owners  the capsules; they stay unconsumed, so dropping them runs the
 *           producers' deleters
 * Every element must provide `__dlpack__()` or be a capsule named "dltensor"
 * or "dltensor_versioned".
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>
#include <string.h>

#include "axon_rocm.h"

/* DLManagedTensor starts with its DLTensor; DLManagedTensorVersioned (DLPack
 * 1.0) has {version{u32,u32}, manager_ctx, deleter, flags(u64)} before it. */
#define AXR_VERSIONED_DLTENSOR_OFFSET 32

static const axr_tensor_t* tensor_of_capsule(PyObject* capsule) {
  if (PyCapsule_IsValid(capsule, "dltensor")) {
    return (const axr_tensor_t*)PyCapsule_GetPointer(capsule, "dltensor");
  }
  if (PyCapsule_IsValid(capsule, "dltensor_versioned")) {
    const char* base = (const char*)PyCapsule_GetPointer(capsule, "dltensor_versioned");
    return base ? (const axr_tensor_t*)(base + AXR_VERSIONED_DLTENSOR_OFFSET) : NULL;
  }
  PyErr_SetString(PyExc_TypeError,
                  "object does not provide a DLPack capsule named 'dltensor'");
  return NULL;
}

static PyObject* describe(PyObject* self, PyObject* arg) {
  (void)self;
  PyObject* seq = PySequence_Fast(arg, "describe() needs a sequence of DLPack producers");
  if (!seq) return NULL;
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
  PyObject* owners = PyList_New(n);
  PyObject* descs = NULL;
  PyObject* dims = NULL;
  PyObject* result = NULL;
  if (!owners) goto done;

  Py_ssize_t total_dims = 0;
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* obj = PySequence_Fast_GET_ITEM(seq, i);   /* borrowed */
    PyObject* capsule;
    if (PyCapsule_CheckExact(obj)) {
      capsule = obj;
      Py_INCREF(capsule);
    } else {
      capsule = PyObject_CallMethod(obj, "__dlpack__", NULL);
      if (!capsule) goto done;
    }
    PyList_SET_ITEM(owners, i, capsule);   /* steals */
    const axr_tensor_t* t = tensor_of_capsule(capsule);
    if (!t) goto done;
    if (t->ndim < 0 || t->ndim > 64) {
      PyErr_SetString(PyExc_ValueError, "tensor ndim out of range");
      goto done;
    }
    if (t->ndim > 0 && !t->shape) {
      PyErr_SetString(PyExc_ValueError, "tensor shape is null for ndim > 0");
      goto done;
    }
    total_dims += (Py_ssize_t)t->ndim * (t->strides ? 2 : 1);
  }

  descs = PyByteArray_FromStringAndSize(NULL, n * (Py_ssize_t)sizeof(axr_tensor_t));
  dims = PyByteArray_FromStringAndSize(NULL, total_dims * (Py_ssize_t)sizeof(int64_t));
  if (!descs || !dims) goto done;
  {
    axr_tensor_t* out = (axr_tensor_t*)PyByteArray_AS_STRING(descs);
    int64_t* d = (int64_t*)PyByteArray_AS_STRING(dims);
    for (Py_ssize_t i = 0; i < n; ++i) {
      const axr_tensor_t* t = tensor_of_capsule(PyList_GET_ITEM(owners, i));
      if (!t) goto done;
      out[i] = *t;
      out[i].shape = NULL;
      out[i].strides = NULL;
      if (t->ndim > 0) {
        memcpy(d, t->shape, (size_t)t->ndim * sizeof(int64_t));
        out[i].shape = d;
        d += t->ndim;
        if (t->strides) {
          memcpy(d, t->strides, (size_t)t->ndim * sizeof(int64_t));
          out[i].strides = d;
          d += t->ndim;
        }
      }
    }
  }
  result = PyTuple_Pack(3, descs, dims, owners);

done:
  Py_XDECREF(descs);
  Py_XDECREF(dims);
  Py_XDECREF(owners);
  Py_DECREF(seq);
  return result;
}

static PyMethodDef methods[] = {
    {"describe", describe, METH_O,
     "describe(sequence) -> (descs bytearray, dims bytearray, owners list)"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_axr_dlpack",
                                    "Native DLPack extraction for tensor bundles.", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__axr_dlpack(void) {
  PyObject* m = PyModule_Create(&module);
  if (m) PyModule_AddIntConstant(m, "TENSOR_BYTES", (long)sizeof(axr_tensor_t));
  return m;
}
