"""DLPack in and out.

Mirrors the reference's ``axon/python/src/dlpack_helpers.cpp``:

* ``extract``  <- ExtractDlpackTensor (:136-156) + ExtractTensorMetaFromDlm
  (:696-724): call ``obj.__dlpack__()``, keep the capsule as the owner, read
  device / dtype / ndim / shape / strides / byte_offset.
* ``DLPackExport`` <- DLPackCapsuleWrapper (dlpack_helpers.hpp:63-170): an
  object with ``__dlpack__`` and ``__dlpack_device__`` over memory the bundle
  path owns, consumable once by ``torch.from_dlpack`` / ``numpy.from_dlpack``.

``TensorArray.from_objects`` does the extraction of a whole tensor list in C
(``csrc/py_dlpack.c``, built as ``lib/_axr_dlpack*.so``) when that helper is
present: one ``__dlpack__()`` call per tensor and no other per-tensor Python
work; the pure-Python ``extract`` gives the same descriptors and serves single
tensors, ``TensorView`` inputs and installations without the helper.

kDLROCM (10), kDLROCMHost (11) and kDLCPU (1) tensors are accepted; the
reference maps kDLROCM to ucx_memory_type::ROCM (:92-97, :123-126) but its
runtime refuses a rocm device (bindings_runtime.cpp:131-141).
"""
from __future__ import annotations

import ctypes as C
import itertools
from dataclasses import dataclass
from typing import Any, Callable, List, Optional, Sequence, Tuple

from . import _capi

_py = C.pythonapi
_py.PyCapsule_IsValid.restype = C.c_int
_py.PyCapsule_IsValid.argtypes = [C.py_object, C.c_char_p]
_py.PyCapsule_GetPointer.restype = C.c_void_p
_py.PyCapsule_GetPointer.argtypes = [C.py_object, C.c_char_p]
_py.PyCapsule_SetName.restype = C.c_int
_py.PyCapsule_SetName.argtypes = [C.py_object, C.c_char_p]
_CAPSULE_DTOR = C.CFUNCTYPE(None, C.c_void_p)
_py.PyCapsule_New.restype = C.py_object
_py.PyCapsule_New.argtypes = [C.c_void_p, C.c_char_p, _CAPSULE_DTOR]
# Variants that take the capsule as a raw address: inside a capsule destructor
# the object's reference count is already zero and must not be touched.
_raw_is_valid = C.PYFUNCTYPE(C.c_int, C.c_void_p, C.c_char_p)(("PyCapsule_IsValid", _py))
_raw_get_pointer = C.PYFUNCTYPE(C.c_void_p, C.c_void_p, C.c_char_p)(("PyCapsule_GetPointer", _py))

_NAME = b"dltensor"
_NAME_USED = b"used_dltensor"
_NAME_VERSIONED = b"dltensor_versioned"


class _ManagedTensor(C.Structure):
    pass


_DELETER = C.CFUNCTYPE(None, C.POINTER(_ManagedTensor))
_ManagedTensor._fields_ = [
    ("dl_tensor", _capi.Tensor),
    ("manager_ctx", C.c_void_p),
    ("deleter", _DELETER),
]


class _ManagedTensorVersioned(C.Structure):
    _fields_ = [
        ("major", C.c_uint32),
        ("minor", C.c_uint32),
        ("manager_ctx", C.c_void_p),
        ("deleter", C.c_void_p),
        ("flags", C.c_uint64),
        ("dl_tensor", _capi.Tensor),
    ]


@dataclass
class TensorView:
    """Plain description of one tensor, the Python face of ``axr_tensor_t``.

    ``owner`` keeps the producer's memory alive (the reference holds the
    capsule in the buffer's release function, dlpack_helpers.cpp:739-742).
    """

    data: int
    device_type: int
    device_id: int
    dtype: Tuple[int, int, int]  # (code, bits, lanes)
    shape: Tuple[int, ...]
    strides: Optional[Tuple[int, ...]]  # elements; None = compact row-major
    byte_offset: int = 0
    owner: Any = None
    readonly: bool = False      # the producer's DLPack 1.0 flag: may be read, must not be written

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def itemsize(self) -> int:
        return (self.dtype[1] + 7) // 8

    @property
    def nbytes(self) -> int:
        # CalculateTensorSize, rpc_core/utils/tensor_meta.hpp:91-104
        if self.ndim == 0:
            return 0
        n = 1
        for s in self.shape:
            n *= s
        return n * self.itemsize


def _read(dl: _capi.Tensor, owner: Any, readonly: bool = False) -> TensorView:
    nd = dl.ndim
    shape = tuple(dl.shape[i] for i in range(nd))
    strides = tuple(dl.strides[i] for i in range(nd)) if dl.strides else None
    return TensorView(
        data=dl.data or 0,
        device_type=dl.device_type,
        device_id=dl.device_id,
        dtype=(dl.dtype_code, dl.dtype_bits, dl.dtype_lanes),
        shape=shape,
        strides=strides,
        byte_offset=dl.byte_offset,
        owner=owner,
        readonly=readonly,
    )


class NotDLPackError(TypeError, RuntimeError):
    """An object that is no DLPack producer.  The reference raises RuntimeError here
    (axon/python/src/dlpack_helpers.cpp:153-155); TypeError is what Python code expects:
    this is both."""


def _is_framework_tensor(obj: Any) -> bool:
    import sys
    torch = sys.modules.get("torch")
    return torch is not None and isinstance(obj, torch.Tensor)


def extract(obj: Any, stream: Optional[int] = None) -> TensorView:
    """Describe ``obj`` (anything with ``__dlpack__``, or a capsule).  ``stream`` is the DLPack
    protocol's value for the stream the consumer will read on (``streams.dlpack_stream_argument``):
    a producer other than a torch tensor is asked with ``__dlpack__(stream=stream)`` so that it
    orders its work before that stream (torch tensors are ordered once per bundle by
    ``streams.order_behind_producers``); one that refuses the argument is asked without it."""
    if isinstance(obj, TensorView):
        return obj
    capsule = obj
    if hasattr(obj, "__dlpack__"):
        capsule = None
        if stream is not None and not _is_framework_tensor(obj):
            try:
                capsule = obj.__dlpack__(stream=stream)
            except (MemoryError, KeyboardInterrupt):
                raise
            except Exception:  # noqa: BLE001 - host producers and older protocols refuse the argument
                capsule = None
        if capsule is None:
            try:
                capsule = obj.__dlpack__()
            except BufferError:
                # a producer whose memory is read-only (a numpy array over bytes, a broadcast
                # view) can only say so in DLPack 1.0: ask for that form.  It may be packed
                # from; binding it as a destination is refused.
                capsule = obj.__dlpack__(max_version=(1, 0))
    if _py.PyCapsule_IsValid(capsule, _NAME):
        ptr = _py.PyCapsule_GetPointer(capsule, _NAME)
        managed = C.cast(ptr, C.POINTER(_ManagedTensor)).contents
        # the capsule stays unconsumed: dropping it runs the producer's deleter
        return _read(managed.dl_tensor, (capsule, obj))
    if _py.PyCapsule_IsValid(capsule, _NAME_VERSIONED):
        ptr = _py.PyCapsule_GetPointer(capsule, _NAME_VERSIONED)
        managed = C.cast(ptr, C.POINTER(_ManagedTensorVersioned)).contents
        return _read(managed.dl_tensor, (capsule, obj), readonly=bool(managed.flags & 1))
    raise NotDLPackError(
        f"Invalid dlpack object {obj!r} when extracting: missing __dlpack__ method "
        "or a capsule not named 'dltensor'"
    )


def extract_many(objs: Sequence[Any], stream: Optional[int] = None) -> List[TensorView]:
    return [extract(o, stream) for o in objs]


class TensorArray:
    """A C array of ``axr_tensor_t`` plus the shape/stride storage it points to."""

    def __init__(self, views: Sequence[TensorView]):
        self._views = list(views)
        self._owners = None
        self.readonly = any(v.readonly for v in self._views)   # some tensor must not be written
        n = len(self._views)
        self.array = (_capi.Tensor * max(n, 1))()
        total = sum(v.ndim * (2 if v.strides is not None else 1) for v in self.views)
        self._dims = (C.c_int64 * max(total, 1))()
        base = C.addressof(self._dims)
        at = 0
        for i, v in enumerate(self.views):
            t = self.array[i]
            t.data = v.data
            t.device_type = v.device_type
            t.device_id = v.device_id
            t.ndim = v.ndim
            t.dtype_code, t.dtype_bits, t.dtype_lanes = v.dtype
            t.byte_offset = v.byte_offset
            nd = v.ndim
            if nd:
                self._dims[at:at + nd] = v.shape
                t.shape = C.cast(base + 8 * at, C.POINTER(C.c_int64))
                at += nd
                if v.strides is not None:
                    self._dims[at:at + nd] = v.strides
                    t.strides = C.cast(base + 8 * at, C.POINTER(C.c_int64))
                    at += nd
        self.count = n

    def pointer(self):
        return C.cast(self.array, C.POINTER(_capi.Tensor))

    @classmethod
    def from_objects(cls, objs: Sequence[Any], stream: Optional[int] = None) -> "TensorArray":
        """Descriptors of DLPack producers (or ``TensorView``s).  ``stream``: the DLPack protocol's
        value for the stream the bundle's kernels will run on, handed to producers other than
        torch tensors (see ``extract``)."""
        native = _native()
        exporter = _torch_exporter()
        described = None
        if exporter:   # a bundle of plain torch tensors is read without one capsule per tensor
            direct = _native_torch()
            if direct is not None:
                described = direct.describe(objs, exporter[2])
        if described is None and native is not None:
            try:
                if stream is None:
                    described = native.describe(objs, *exporter)
                else:
                    described = native.describe(objs, *(exporter or (None, None, -1)), stream)
            except BufferError:     # a read-only producer: the slower path asks it in DLPack 1.0
                described = None
        if described is None:   # no helper, or something that is not a DLPack producer
            return cls(extract_many(objs, stream))
        descs, dims, owners = described
        self = cls.__new__(cls)
        n = len(owners)
        self.readonly = False
        self.count = n
        self._descs, self._dims, self._owners = descs, dims, (owners, list(objs))
        self.array = (_capi.Tensor * max(n, 1)).from_buffer(descs) if n else (_capi.Tensor * 1)()
        self._views = None
        return self

    @property
    def views(self) -> List[TensorView]:
        if self._views is None:   # native path: materialised only when somebody asks
            owners = self._owners[0]
            self._views = [_read(self.array[i], owners[i]) for i in range(self.count)]
        return self._views

    @views.setter
    def views(self, value):
        self._views = value


def _torch_exporter() -> tuple:
    """``(torch.Tensor, to_dlpack, device)`` for the C helper, or ``()``.

    ``Tensor.__dlpack__()`` is a page of Python around ``to_dlpack``: it refuses
    tensors that require gradients or carry the conjugate bit, refuses GPU
    tensors of another device than the current one, and makes the default stream
    wait for torch's current stream when the two differ.  The helper repeats the
    first three checks in C; the fourth does nothing while torch runs on its
    default stream, which is checked here once per bundle.  Anywhere else every
    tensor goes through ``__dlpack__()``.
    """
    import sys
    torch = sys.modules.get("torch")
    if torch is None:
        return ()
    device = -1   # no GPU context: only host tensors can exist
    if torch.cuda.is_initialized():
        raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        get_device = getattr(torch._C, "_cuda_getDevice", None)
        if raw_stream is not None and get_device is not None:
            # the same two questions through torch's C entry points (0.3 us instead
            # of 7 us, which matters for bundles of a few tensors); the default
            # stream is the null handle
            device = get_device()
            if raw_stream(device) != 0:
                return ()
        else:
            if torch.cuda.current_stream() != torch.cuda.default_stream():
                return ()
            device = torch.cuda.current_device()
    return (torch.Tensor, torch.utils.dlpack.to_dlpack, device)


_NATIVE: Any = False


def _native():
    """The C helper module, or None when it has not been built."""
    global _NATIVE
    if _NATIVE is False:
        import glob
        import importlib.machinery
        import importlib.util
        import os
        _NATIVE = None
        here = os.path.dirname(os.path.abspath(__file__))
        for path in glob.glob(os.path.join(here, "lib", "_axr_dlpack*.so")):
            loader = importlib.machinery.ExtensionFileLoader("_axr_dlpack", path)
            spec = importlib.util.spec_from_loader("_axr_dlpack", loader)
            mod = importlib.util.module_from_spec(spec)
            loader.exec_module(mod)
            if mod.TENSOR_BYTES == C.sizeof(_capi.Tensor):
                _NATIVE = mod
            break
    return _NATIVE


_NATIVE_TORCH: Any = False


def _native_torch():
    """The helper that reads torch tensors' fields through torch's own non-owning DLPack
    converter, or None when it has not been built or does not load against this torch.
    Only called once torch has been imported (its libraries are the module's dependencies)."""
    global _NATIVE_TORCH
    if _NATIVE_TORCH is False:
        import glob
        import importlib.machinery
        import importlib.util
        import os
        _NATIVE_TORCH = None
        here = os.path.dirname(os.path.abspath(__file__))
        for path in glob.glob(os.path.join(here, "lib", "_axr_torch*.so")):
            try:
                loader = importlib.machinery.ExtensionFileLoader("_axr_torch", path)
                spec = importlib.util.spec_from_loader("_axr_torch", loader)
                mod = importlib.util.module_from_spec(spec)
                loader.exec_module(mod)
            except ImportError:   # built against another torch
                break
            if mod.TENSOR_BYTES == C.sizeof(_capi.Tensor):
                _NATIVE_TORCH = mod
            break
    return _NATIVE_TORCH


# ---------------------------------------------------------------- export

_live_exports = {}  # id -> (managed struct, shape array, release callback)
_next_export = itertools.count(1)   # next() is one step under the interpreter lock: exports may come from several threads


@_DELETER
def _managed_deleter(ptr):  # called by the consumer when it drops the tensor
    exports = _live_exports
    if exports is None:     # interpreter shutdown, this module's globals are already cleared: the
        return              # process is ending, nothing is given back
    entry = exports.pop(ptr.contents.manager_ctx, None)
    if entry is not None and entry[3] is not None:
        entry[3]()


@_CAPSULE_DTOR
def _capsule_destructor(capsule_ptr):
    # runs when a capsule is collected; an unconsumed one still owns the tensor
    if _raw_is_valid(capsule_ptr, _NAME):
        ptr = _raw_get_pointer(capsule_ptr, _NAME)
        managed = C.cast(ptr, C.POINTER(_ManagedTensor))
        managed.contents.deleter(managed)


_DELETER_VERSIONED = C.CFUNCTYPE(None, C.c_void_p)


@_DELETER_VERSIONED
def _managed_deleter_versioned(address):   # the same for a DLManagedTensorVersioned
    exports = _live_exports
    if exports is None:
        return
    managed = C.cast(address, C.POINTER(_ManagedTensorVersioned)).contents
    entry = exports.pop(managed.manager_ctx, None)
    if entry is not None and entry[3] is not None:
        entry[3]()


@_CAPSULE_DTOR
def _capsule_destructor_versioned(capsule_ptr):
    if _raw_is_valid(capsule_ptr, _NAME_VERSIONED):
        ptr = _raw_get_pointer(capsule_ptr, _NAME_VERSIONED)
        managed = C.cast(ptr, C.POINTER(_ManagedTensorVersioned)).contents
        _DELETER_VERSIONED(managed.deleter)(ptr)


# A consumer may keep its tensor until the interpreter shuts down and drop it after this module
# has been cleared: the C entry points of the two callbacks above must stay valid until the
# process ends, so they are never freed.
_py.Py_IncRef.argtypes = [C.py_object]
_py.Py_IncRef.restype = None
for _callback in (_managed_deleter, _capsule_destructor, _managed_deleter_versioned, _capsule_destructor_versioned):
    _py.Py_IncRef(_callback)


class DLPackExport:
    """Single-consume DLPack producer over memory owned by this package.

    ``release`` runs once, when the consumer (or an unconsumed capsule) lets go.
    """

    def __init__(self, data: int, nbytes_or_shape, dtype: Tuple[int, int, int], device_type: int,
                 device_id: int = 0, release: Optional[Callable[[], None]] = None):
        self._data = data
        self._shape = tuple(nbytes_or_shape) if not isinstance(nbytes_or_shape, int) else (nbytes_or_shape,)
        self._dtype = dtype
        self._device = (device_type, device_id)
        self._release = release
        self._consumed = False
        self._exported = False     # a capsule went out: its deleter releases the memory

    def __dlpack_device__(self):
        return self._device

    def __dlpack__(self, stream=None, max_version=None, dl_device=None, copy=None):
        # checks, their order and the exception types follow the reference's wrapper
        # (axon/python/src/dlpack_helpers.hpp:106-155): consumed first (and for good,
        # even when a later check raises), then the stream rule for host memory, then
        # the target device, then copy
        if self._consumed:
            raise RuntimeError("DLPack capsule has already been consumed. "
                               "__dlpack__() can only be called once per capsule.")
        self._consumed = True
        if self._device[0] == _capi.kDLCPU and stream is not None:
            raise ValueError("stream must be None for CPU device (kDLCPU)")
        if dl_device is not None and int(dl_device[0]) != self._device[0]:
            if copy is not None and not copy:
                raise RuntimeError("Cross-device export requires copy=True or copy=None, "
                                   "but copy=False was specified")
            raise RuntimeError("Cross-device DLPack export is not yet supported")
        if copy:
            raise RuntimeError("copy=True is not supported; this implementation is zero-copy only")
        nd = len(self._shape)
        shape = (C.c_int64 * max(nd, 1))(*self._shape)
        # A consumer that speaks DLPack 1.0 (max_version) gets a DLManagedTensorVersioned with no
        # flag set; one that does not gets the unversioned struct, which cannot say whether the
        # memory may be written (numpy then hands out a read-only array).  The reference's wrapper
        # always returns the unversioned form (dlpack_helpers.hpp:149-152).
        versioned = max_version is not None and int(tuple(max_version)[0]) >= 1
        managed = _ManagedTensorVersioned() if versioned else _ManagedTensor()
        if versioned:
            managed.major, managed.minor, managed.flags = 1, 0, 0
        dl = managed.dl_tensor
        dl.data = self._data
        dl.device_type, dl.device_id = self._device
        dl.ndim = nd
        dl.dtype_code, dl.dtype_bits, dl.dtype_lanes = self._dtype
        dl.shape = C.cast(shape, C.POINTER(C.c_int64))
        dl.strides = None
        dl.byte_offset = 0
        key = next(_next_export)
        managed.manager_ctx = key
        if versioned:
            managed.deleter = C.cast(_managed_deleter_versioned, C.c_void_p).value
        else:
            managed.deleter = _managed_deleter
        _live_exports[key] = (managed, shape, self, self._release)
        self._exported = True
        native = _native()
        if native is not None and hasattr(native, "new_capsule"):
            # the C destructor keeps a consumer's pending exception intact when a refused
            # capsule is dropped; the ctypes one below cannot run under a pending exception
            return native.new_capsule(C.addressof(managed), versioned)
        if versioned:
            return _py.PyCapsule_New(C.addressof(managed), _NAME_VERSIONED, _capsule_destructor_versioned)
        return _py.PyCapsule_New(C.addressof(managed), _NAME, _capsule_destructor)

    def __del__(self):
        if not self._exported and self._release is not None:
            release, self._release = self._release, None
            release()


# DLPack dtype codes
kDLInt, kDLUInt, kDLFloat, kDLBfloat, kDLBool = 0, 1, 2, 4, 6
