"""Device objects handed to the runtime, same API shape as the reference's
``axon/python/axon/device.py`` (``Device.get_type / get_type_string /
get_context_handle``, factories ``cpu()`` / ``rocm()`` / ``auto_detect()``).

The reference declares ``RocmDevice`` (device.py:131-167) but its runtime throws
for it (bindings_runtime.cpp:131-141).  Here ``RocmDevice`` is the working one:
its context handle is the HIP device ordinal, and ``activate()`` gives the
thread-level RAII that ``UcxAutoCudaDeviceContext`` gives on CUDA
(ucx_context/cuda/ucx_cuda_context.hpp:55-72).
"""
from __future__ import annotations

import contextlib
import ctypes as C
import enum
from abc import ABC, abstractmethod
from typing import Optional

from . import _capi


class DeviceType(enum.Enum):
    CPU = "cpu"
    CUDA = "cuda"
    ROCM = "rocm"
    SYCL = "sycl"


class Device(ABC):
    @abstractmethod
    def get_type(self) -> DeviceType: ...

    @abstractmethod
    def get_type_string(self) -> str: ...

    @abstractmethod
    def get_context_handle(self) -> Optional[int]: ...


class CpuDevice(Device):
    def __init__(self, numa_node: Optional[int] = None):
        self.numa_node = numa_node

    def get_type(self) -> DeviceType:
        return DeviceType.CPU

    def get_type_string(self) -> str:
        return "cpu"

    def get_context_handle(self) -> Optional[int]:
        return None

    def __repr__(self) -> str:
        if self.numa_node is not None:
            return f"CpuDevice(numa_node={self.numa_node})"
        return "CpuDevice()"


class RocmDevice(Device):
    """One AMD GPU.  ``context`` is accepted for signature compatibility; HIP
    has one primary context per device, so the ordinal identifies it."""

    def __init__(self, device_id: int = 0, context: Optional[int] = None):
        self.device_id = int(device_id)
        self._context = context if context is not None else self.device_id

    def get_type(self) -> DeviceType:
        return DeviceType.ROCM

    def get_type_string(self) -> str:
        return "rocm"

    def get_context_handle(self) -> Optional[int]:
        return self._context

    @contextlib.contextmanager
    def activate(self):
        """Make this device current on the calling thread for the block."""
        lib = _capi.load()
        token = C.c_int(0)
        _capi.check(lib.axr_device_push(self.device_id, C.byref(token)))
        try:
            yield self
        finally:
            _capi.check(lib.axr_device_pop(token.value))

    def clone(self) -> "RocmDevice":
        return RocmDevice(self.device_id, self._context)

    def __repr__(self) -> str:
        return f"RocmDevice(device_id={self.device_id})"


class _DeclaredDevice(Device):
    """A device kind the reference declares (axon/python/axon/device.py:86-128, 170-199) that this
    build has no runtime for: the object carries what the caller gave it, so scripts written for
    the reference construct and inspect it as before, and a runtime created with it moves host
    tensors only (the reference's runtime likewise accepts the object and handles the missing
    platform internally, axon/python/tests/test_device_api.py:106-112)."""

    _kind: DeviceType

    def __init__(self, device_id: int = 0, context: Optional[int] = None):
        self.device_id = device_id
        self._context = context

    def get_type(self) -> DeviceType:
        return self._kind

    def get_type_string(self) -> str:
        return self._kind.value

    def get_context_handle(self) -> Optional[int]:
        return self._context

    def __repr__(self) -> str:
        return f"{type(self).__name__}(device_id={self.device_id})"


class CudaDevice(_DeclaredDevice):
    _kind = DeviceType.CUDA

    def __repr__(self) -> str:
        if self._context is not None:
            return f"CudaDevice(device_id={self.device_id}, context={self._context:#x})"
        return super().__repr__()


class SyclDevice(_DeclaredDevice):
    _kind = DeviceType.SYCL

    def __init__(self, device_id: int = 0, context: Optional[int] = None, queue: Optional[int] = None):
        super().__init__(device_id, context)
        self.queue = queue


def cuda(device_id: int = 0, context: Optional[int] = None) -> CudaDevice:
    return CudaDevice(device_id=device_id, context=context)


def sycl(device_id: int = 0, context: Optional[int] = None, queue: Optional[int] = None) -> SyclDevice:
    return SyclDevice(device_id=device_id, context=context, queue=queue)


def cpu(numa_node: Optional[int] = None) -> CpuDevice:
    return CpuDevice(numa_node=numa_node)


def rocm(device_id: int = 0, context: Optional[int] = None) -> RocmDevice:
    return RocmDevice(device_id=device_id, context=context)


def device_count() -> int:
    n = C.c_int(0)
    _capi.check(_capi.load().axr_device_count(C.byref(n)))
    return n.value


def auto_detect() -> Device:
    """ROCm when a GPU is visible, CPU otherwise."""
    try:
        if device_count() > 0:
            return RocmDevice()
    except (ImportError, _capi.AxonRocmError):
        pass
    return CpuDevice()
