"""ctypes binding of the C ABI declared in ``include/axon_rocm.h``.

The shared library is loaded from ``lib/libaxon_rocm.so`` next to this file.
There is no fallback: when the library is missing every entry point of the
package raises ``ImportError`` (build it with ``make -C execution-ucx_amd`` or
``__graft_entry__.build()``).
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "lib", "libaxon_rocm.so")

# ---------------------------------------------------------------- status codes

AXR_OK = 0
AXR_ERR_INVALID = -1
AXR_ERR_NOMEM = -2
AXR_ERR_HIP = -3
AXR_ERR_LENGTH = -4
AXR_ERR_UNSUPPORTED = -5
AXR_ERR_NO_MESSAGE = -6
AXR_ERR_NOT_IMPLEMENTED = -7
AXR_ERR_HEADER = -8
AXR_ERR_MISMATCH = -9
AXR_ERR_NO_DEVICE = -10
AXR_ERR_BUSY = -11
AXR_ERR_CANCELED = -12

# ucx_memory_type_t numbering (ucx_context/ucx_context_def.h:27-39)
MEM_HOST = 0
MEM_CUDA = 1
MEM_CUDA_MANAGED = 2
MEM_ROCM = 3
MEM_ROCM_MANAGED = 4
MEM_UNKNOWN = 9

# DLPack device types
kDLCPU = 1
kDLCUDA = 2
kDLROCM = 10
kDLROCMHost = 11


class AxonRocmError(RuntimeError):
    """A C-ABI call failed; ``status`` holds the axr_status value."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status


class LengthError(AxonRocmError, ValueError):
    """Sizes exceed the buffer (the reference throws std::length_error,
    ucx_context/ucx_context_data.hpp:644-646)."""


class UnsupportedMemoryError(AxonRocmError):
    """Memory type or copy combination not served (std::runtime_error in
    ucx_context/cuda/ucx_cuda_memory_manager.hpp:103,150)."""


class HeaderError(AxonRocmError, ValueError):
    """Malformed bundle header."""


class MismatchError(AxonRocmError, ValueError):
    """Bound tensors do not match the plan."""


class NoDeviceError(AxonRocmError):
    """No usable ROCm device."""


class NoMessageError(AxonRocmError, LookupError):
    """Unknown receive key (UCS_ERR_NO_MESSAGE, ucx_am_context.hpp:1570-1574)."""


class NotImplementedForEager(AxonRocmError, NotImplementedError):
    """recv_buffer on an eager message (UCS_ERR_NOT_IMPLEMENTED, :1643-1651)."""


_ERROR_TYPES = {
    AXR_ERR_LENGTH: LengthError,
    AXR_ERR_UNSUPPORTED: UnsupportedMemoryError,
    AXR_ERR_HEADER: HeaderError,
    AXR_ERR_MISMATCH: MismatchError,
    AXR_ERR_NO_DEVICE: NoDeviceError,
    AXR_ERR_NO_MESSAGE: NoMessageError,
    AXR_ERR_NOT_IMPLEMENTED: NotImplementedForEager,
}

# ---------------------------------------------------------------- structures


class Tensor(C.Structure):
    """axr_tensor_t == DLTensor."""

    _fields_ = [
        ("data", C.c_void_p),
        ("device_type", C.c_int32),
        ("device_id", C.c_int32),
        ("ndim", C.c_int32),
        ("dtype_code", C.c_uint8),
        ("dtype_bits", C.c_uint8),
        ("dtype_lanes", C.c_uint16),
        ("shape", C.POINTER(C.c_int64)),
        ("strides", C.POINTER(C.c_int64)),
        ("byte_offset", C.c_uint64),
    ]


class Buffer(C.Structure):
    """axr_buffer_t == ucx_buffer_t."""

    _fields_ = [("data", C.c_void_p), ("size", C.c_size_t)]


class PoolStats(C.Structure):
    _fields_ = [
        ("slabs", C.c_uint64),
        ("slab_bytes", C.c_uint64),
        ("allocated_bytes", C.c_uint64),
        ("live_blocks", C.c_uint64),
        ("peak_bytes", C.c_uint64),
    ]


class LaunchInfo(C.Structure):
    _fields_ = [
        ("workgroups", C.c_uint32),
        ("threads_per_workgroup", C.c_uint32),
        ("tiles", C.c_uint32),
        ("tile_bytes", C.c_uint32),
        ("segments", C.c_uint32),
        ("table_bytes", C.c_uint32),
        ("host_copies", C.c_uint32),
        ("host_chunks", C.c_uint32),
        ("inline_tables", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class SegmentInfo(C.Structure):
    _fields_ = [
        ("tensor", C.c_uint32),
        ("mode", C.c_uint32),
        ("address", C.c_uint64),
        ("offset", C.c_uint64),
        ("run_bytes", C.c_uint64),
        ("nbytes", C.c_uint64),
        ("pad", C.c_uint32),
        ("ndim", C.c_uint32),
        ("granule", C.c_uint32),
        ("tiles", C.c_uint32),
        ("head", C.c_uint32),
        ("lanes_per_run", C.c_uint32),
        ("shape", C.c_uint32 * 6),
        ("stride_bytes", C.c_int64 * 6),
    ]


class Job(C.Structure):
    """axr_job_t: one gather or scatter of axr_submit."""

    _fields_ = [("plan", C.c_void_p), ("unpack", C.c_int), ("payload", C.c_void_p),
                ("payload_bytes", C.c_size_t), ("tensor_delta", C.c_int64), ("flags", C.c_uint32),
                ("reserved", C.c_uint32)]


JOB_PAYLOAD_STREAMING = 1
JOB_PAYLOAD_CACHED = 2


class AmData(C.Structure):
    """axr_am_data_t == ucx_am_data_t."""

    _fields_ = [("header", Buffer), ("buffer", Buffer), ("buffer_type", C.c_int), ("mem_h", C.c_void_p)]


class AmIovec(C.Structure):
    """axr_am_iovec_t == ucx_am_iovec_t."""

    _fields_ = [("header", Buffer), ("buffer_vec", C.POINTER(Buffer)), ("buffer_count", C.c_size_t),
                ("buffer_type", C.c_int), ("mem_h", C.c_void_p)]


class AmMessage(C.Structure):
    _fields_ = [("key", C.c_uint64), ("conn_id", C.c_uint64), ("header", Buffer),
                ("data_length", C.c_uint64), ("is_rndv", C.c_int), ("buffer_type", C.c_int),
                ("eager_data", Buffer)]


class UcxProbe(C.Structure):
    _fields_ = [("available", C.c_int), ("version_major", C.c_uint), ("version_minor", C.c_uint),
                ("version_release", C.c_uint), ("have_symbol", C.c_int * 6), ("library", C.c_char * 256),
                ("message", C.c_char * 512)]


REGISTER_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p))
UNREGISTER_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)

_vp = C.c_void_p
_vpp = C.POINTER(C.c_void_p)
_u64p = C.POINTER(C.c_uint64)
_i64p = C.POINTER(C.c_int64)
_intp = C.POINTER(C.c_int)
_sz = C.c_size_t
_TensorP = C.POINTER(Tensor)

# name -> (restype, argtypes); every AXR_API function of the header is listed
PROTOTYPES = {
    "axr_status_string": (C.c_char_p, [C.c_int]),
    "axr_last_error": (C.c_char_p, []),
    "axr_version": (C.c_char_p, []),
    "axr_dl_device_to_memory_type": (C.c_int, [C.c_int32]),
    "axr_memory_type_to_dl_device": (C.c_int32, [C.c_int]),
    "axr_tensor_nbytes": (C.c_int, [_TensorP, _u64p]),
    "axr_device_count": (C.c_int, [_intp]),
    "axr_device_get": (C.c_int, [_intp]),
    "axr_device_set": (C.c_int, [C.c_int]),
    "axr_device_push": (C.c_int, [C.c_int, _intp]),
    "axr_device_pop": (C.c_int, [C.c_int]),
    "axr_device_synchronize": (C.c_int, []),
    "axr_device_info": (C.c_int, [_intp, _u64p, _u64p]),
    "axr_stream_create": (C.c_int, [_vpp]),
    "axr_stream_destroy": (C.c_int, [_vp]),
    "axr_stream_synchronize": (C.c_int, [_vp]),
    "axr_stream_wait_event": (C.c_int, [_vp, _vp]),
    "axr_event_create": (C.c_int, [_vpp]),
    "axr_event_destroy": (C.c_int, [_vp]),
    "axr_event_record": (C.c_int, [_vp, _vp]),
    "axr_event_synchronize": (C.c_int, [_vp]),
    "axr_event_query": (C.c_int, [_vp, _intp]),
    "axr_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "axr_mem_alloc": (C.c_int, [C.c_int, _sz, _sz, _vpp]),
    "axr_mem_free": (C.c_int, [C.c_int, _vp, _sz]),
    "axr_memcpy": (C.c_int, [C.c_int, _vp, C.c_int, _vp, _sz]),
    "axr_memcpy_async": (C.c_int, [C.c_int, _vp, C.c_int, _vp, _sz, _vp]),
    "axr_memset_async": (C.c_int, [_vp, C.c_int, _sz, _vp]),
    "axr_pool_create": (C.c_int, [C.c_int, _sz, _vpp]),
    "axr_pool_destroy": (C.c_int, [_vp]),
    "axr_pool_default": (C.c_int, [_vpp]),
    "axr_pool_set_registrar": (C.c_int, [_vp, REGISTER_FN, UNREGISTER_FN, _vp]),
    "axr_pool_alloc": (C.c_int, [_vp, _sz, _sz, _vpp, _vpp]),
    "axr_pool_free": (C.c_int, [_vp, _vp]),
    "axr_pool_trim": (C.c_int, [_vp]),
    "axr_pool_get_stats": (C.c_int, [_vp, C.POINTER(PoolStats)]),
    "axr_plan_create": (C.c_int, [_TensorP, _sz, C.c_uint32, C.c_uint32, _vpp]),
    "axr_plan_free": (C.c_int, [_vp]),
    "axr_plan_num_tensors": (C.c_int, [_vp, C.POINTER(_sz)]),
    "axr_plan_payload_bytes": (C.c_int, [_vp, _u64p]),
    "axr_plan_data_bytes": (C.c_int, [_vp, _u64p]),
    "axr_plan_layout": (C.c_int, [_vp, _u64p, _u64p]),
    "axr_plan_tensor_meta": (C.c_int, [_vp, _sz, _TensorP]),
    "axr_plan_header": (C.c_int, [_vp, _vpp, C.POINTER(_sz)]),
    "axr_plan_from_header": (C.c_int, [_vp, _sz, _vpp]),
    "axr_plan_bind": (C.c_int, [_vp, _TensorP, _sz]),
    "axr_plan_from_header_bind": (C.c_int, [_vp, _sz, _TensorP, _sz, _vpp]),
    "axr_plan_split": (C.c_int, [_vp, _vp, _sz, C.POINTER(Buffer)]),
    "axr_pack": (C.c_int, [_vp, _vp, _sz, _vp]),
    "axr_unpack": (C.c_int, [_vp, _vp, _sz, _vp]),
    "axr_plan_prepare": (C.c_int, [_vp, _vp]),
    "axr_pack_noalloc": (C.c_int, [_vp, _vp, _sz, _vp]),
    "axr_submit": (C.c_int, [C.POINTER(Job), _sz, _vp]),
    "axr_plan_launch_info": (C.c_int, [_vp, C.POINTER(LaunchInfo)]),
    "axr_plan_segments": (C.c_int, [_vp, C.POINTER(SegmentInfo), _sz, C.POINTER(_sz)]),
    "axr_tune_set": (C.c_int, [C.c_char_p, C.c_int64]),
    "axr_tune_get": (C.c_int, [C.c_char_p, _i64p]),
    "axr_am_context_create": (C.c_int, [C.c_char_p, _sz, _vpp]),
    "axr_am_context_destroy": (C.c_int, [_vp]),
    "axr_am_connect": (C.c_int, [_vp, _vp, _u64p]),
    "axr_am_send": (C.c_int, [_vp, C.c_uint64, C.POINTER(AmData), _vp, _u64p]),
    "axr_am_send_iov": (C.c_int, [_vp, C.c_uint64, C.POINTER(AmIovec), _vp, _u64p]),
    "axr_am_request_test": (C.c_int, [_vp, C.c_uint64, _intp]),
    "axr_am_request_cancel": (C.c_int, [_vp, C.c_uint64]),
    "axr_am_progress": (C.c_int, [_vp, C.POINTER(_sz), C.POINTER(_sz)]),
    "axr_am_recv_header": (C.c_int, [_vp, C.POINTER(AmMessage)]),
    "axr_am_recv_buffer": (C.c_int, [_vp, C.c_uint64, C.c_int, _vp, _sz, _vp]),
    "axr_am_recv_buffer_async": (C.c_int, [_vp, C.c_uint64, C.c_int, _vp, _sz, _vp]),
    "axr_am_recv_buffer_iov": (C.c_int, [_vp, C.c_uint64, C.c_int, C.POINTER(Buffer), _sz, _vp]),
    "axr_am_recv_buffer_borrow": (C.c_int, [_vp, C.c_uint64, _vpp, C.POINTER(_sz), _intp]),
    "axr_am_borrow_release": (C.c_int, [_vp, C.c_uint64, _vp]),
    "axr_am_message_release": (C.c_int, [_vp, C.c_uint64]),
    "axr_am_message_info": (C.c_int, [_vp, C.c_uint64, _u64p, _u64p, _intp]),
    "axr_am_pending": (C.c_int, [_vp, C.POINTER(_sz)]),
    "axr_ucx_probe": (C.c_int, [C.POINTER(UcxProbe)]),
    "axr_ucx_symbol_name": (C.c_char_p, [C.c_int]),
    "axr_am_context_create_ucx": (C.c_int, [C.c_char_p, _vpp]),
    "axr_transfer_create": (C.c_int, [_vp, _sz, C.c_int, C.c_int, _vpp]),
    "axr_transfer_submit": (C.c_int, [_vp, _vp, C.c_int64, _vp, C.c_int64]),
    "axr_transfer_set_zero_copy": (C.c_int, [_vp, C.c_int]),
    "axr_transfer_finish": (C.c_int, [_vp]),
    "axr_transfer_destroy": (C.c_int, [_vp]),
    "axr_divide_by_two": (C.c_int, [_vp, _sz, _vp]),
    "axr_compare": (C.c_int, [_vp, _vp, _sz, _u64p]),
    "axr_checksum": (C.c_int, [_vp, _sz, C.c_uint64, _u64p]),
    "axr_copy_reference": (C.c_int, [_vp, _vp, _sz, _vp]),
    "axr_copy_reference_shaped": (C.c_int, [_vp, _vp, _sz, C.c_uint32, C.c_uint32, C.c_int, _vp]),
    "axr_rows_reference": (C.c_int, [_vp, _sz, _vp, _sz, _sz, C.c_int, C.c_uint32, _vp]),
}

_lib = None


def _share_hip_runtime() -> None:
    """Make this library and PyTorch use ONE HIP runtime instance.

    PyTorch wheels ship their own libamdhip64.so; streams, events and device
    pointers are only interchangeable inside one runtime instance.  The dynamic
    loader reuses an already loaded library whose SONAME matches, so the wheel's
    copy is loaded first (without importing torch) when it exists; otherwise the
    system ROCm runtime named in the library's RUNPATH is used.
    """
    try:
        with open("/proc/self/maps") as f:
            if "libamdhip64" in f.read():
                return
    except OSError:
        pass
    try:
        import importlib.util
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.submodule_search_locations:
        return
    for base in spec.submodule_search_locations:
        cand = os.path.join(base, "lib", "libamdhip64.so")
        if os.path.exists(cand):
            C.CDLL(cand, mode=C.RTLD_GLOBAL)
            return


def load() -> C.CDLL:
    """Load the shared library once and attach prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise ImportError(
            f"{LIBRARY_PATH} is missing: the HIP extension has not been built "
            "(run `make -C execution-ucx_amd` or `__graft_entry__.build()`); "
            "there is no CPU fallback for the tensor-bundle path"
        )
    _share_hip_runtime()
    lib = C.CDLL(LIBRARY_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    """Raise the Python exception that corresponds to a negative status."""
    if status == AXR_OK:
        return
    lib = load()
    msg = lib.axr_last_error().decode("utf-8", "replace")
    name = lib.axr_status_string(status).decode()
    raise _ERROR_TYPES.get(status, AxonRocmError)(status, f"{name}: {msg}")


def status_name(status: int) -> str:
    return load().axr_status_string(status).decode()
