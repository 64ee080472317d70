"""ROCm memory resource: the Python face of the hipMalloc slab pool.

``RocmMemoryResourceManager`` offers the three operations of the reference's
``UcxMemoryResourceManager`` (ucx_context/ucx_memory_resource.hpp:99-123):
``allocate(type, bytes, alignment)``, ``deallocate(type, ptr, bytes)``,
``memcpy(dst_type, dst, src_type, src, count)`` with ucx_memory_type numbering,
in place of ``UcxCudaMemoryResourceManager``
(ucx_context/cuda/ucx_cuda_memory_manager.hpp:43-154).
"""
from __future__ import annotations

import ctypes as C
from typing import Callable, Optional

from . import _capi
from .dlpack import DLPackExport, kDLUInt

HOST = _capi.MEM_HOST
ROCM = _capi.MEM_ROCM
ROCM_MANAGED = _capi.MEM_ROCM_MANAGED


class DevicePool:
    """Slab pool of device memory (``axr_pool_*``)."""

    def __init__(self, device: int = 0, slab_bytes: int = 0, _handle: Optional[int] = None):
        self._lib = _capi.load()
        self._owned = _handle is None
        self._registrar = None
        if _handle is None:
            h = C.c_void_p()
            _capi.check(self._lib.axr_pool_create(device, slab_bytes, C.byref(h)))
            _handle = h.value
        self._h = _handle

    @classmethod
    def default(cls) -> "DevicePool":
        lib = _capi.load()
        h = C.c_void_p()
        _capi.check(lib.axr_pool_default(C.byref(h)))
        return cls(_handle=h.value)

    def set_registrar(self, register: Callable[[int, int], int], unregister: Callable[[int], None]):
        """``register(addr, length) -> mem_h`` runs once per slab; this is where
        ``ucx_am_context::register_ucx_memory`` (ucp_mem_map) plugs in."""

        def _reg(_user, addr, length, out):
            try:
                out[0] = register(addr, length)
                return 0
            except Exception:  # noqa: BLE001 - reported through the status code
                return -1

        def _unreg(_user, mem_h):
            unregister(mem_h)

        self._registrar = (_capi.REGISTER_FN(_reg), _capi.UNREGISTER_FN(_unreg))
        _capi.check(self._lib.axr_pool_set_registrar(self._h, self._registrar[0],
                                                     self._registrar[1], None))

    def alloc(self, nbytes: int, alignment: int = 256) -> "PoolBuffer":
        ptr, memh = C.c_void_p(), C.c_void_p()
        _capi.check(self._lib.axr_pool_alloc(self._h, nbytes, alignment, C.byref(ptr), C.byref(memh)))
        return PoolBuffer(self, ptr.value or 0, nbytes, memh.value)

    def _free(self, ptr: int) -> None:
        _capi.check(self._lib.axr_pool_free(self._h, ptr))

    def trim(self) -> None:
        _capi.check(self._lib.axr_pool_trim(self._h))

    def stats(self) -> dict:
        st = _capi.PoolStats()
        _capi.check(self._lib.axr_pool_get_stats(self._h, C.byref(st)))
        return {f: getattr(st, f) for f, _ in st._fields_}

    def close(self) -> None:
        if self._owned and self._h:
            _capi.check(self._lib.axr_pool_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            if self._owned and self._h:
                self._lib.axr_pool_destroy(self._h)
        except Exception:  # noqa: BLE001
            pass


class PoolBuffer:
    """A block of pool memory: the ``UcxBuffer`` of this package
    (ucx_context/ucx_context_data.hpp:45-219): ``data``, ``size``, ``mem_h``,
    memory type ROCM, freed when released or collected."""

    memory_type = ROCM

    def __init__(self, pool: DevicePool, ptr: int, size: int, mem_h: Optional[int]):
        self._pool = pool
        self.data = ptr
        self.size = size
        self.mem_h = mem_h

    def release(self) -> None:
        if self.data:
            self._pool._free(self.data)
            self.data = 0
            self.size = 0

    def as_dlpack(self, shape=None, dtype=(kDLUInt, 8, 1), device_id: int = 0) -> DLPackExport:
        """Hand the block to a DLPack consumer; the block returns to the pool
        when the consumer drops it."""
        data, self.data = self.data, 0
        pool = self._pool
        return DLPackExport(data, shape if shape is not None else self.size, dtype,
                            _capi.kDLROCM, device_id, release=lambda: pool._free(data))

    def __del__(self):
        try:
            self.release()
        except Exception:  # noqa: BLE001
            pass


class RocmMemoryResourceManager:
    """allocate / deallocate / memcpy over HOST, ROCM and ROCM_MANAGED."""

    def __init__(self):
        self._lib = _capi.load()

    def allocate(self, memory_type: int, nbytes: int, alignment: int = 8) -> int:
        p = C.c_void_p()
        _capi.check(self._lib.axr_mem_alloc(memory_type, nbytes, alignment, C.byref(p)))
        return p.value or 0

    def deallocate(self, memory_type: int, ptr: int, nbytes: int, alignment: int = 8) -> None:
        _capi.check(self._lib.axr_mem_free(memory_type, ptr, nbytes))

    def memcpy(self, dst_type: int, dst: int, src_type: int, src: int, count: int) -> int:
        _capi.check(self._lib.axr_memcpy(dst_type, dst, src_type, src, count))
        return dst
