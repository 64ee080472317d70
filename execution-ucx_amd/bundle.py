"""Tensor-bundle marshalling: N tensors <-> one contiguous HBM payload + header.

Sender side replaces the reference's ``InvokeContext.to_ucx_buffer_vec``
(axon/python/src/bindings_runtime_helpers.hpp:437-467), which builds one iov
entry per tensor and lets UCX gather them: here the tensors are gathered by one
HIP kernel launch into a pool buffer that goes out as a single contiguous
``ucx_am_data``.  Receiver side replaces the iov scatter of
``connection_recv_buffer(key, UcxBufferVec)``: the contiguous payload is
either split into zero-copy views (``UcxBuffer::to_buffer_vec``,
ucx_context/ucx_context_data.hpp:641-665) or scattered by one kernel launch
into destination tensors.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any, Callable, List, NamedTuple, Optional, Sequence, Tuple

from . import _capi, streams
from .dlpack import DLPackExport, TensorArray, TensorView
from .memory import DevicePool, PoolBuffer


class DLDevice(NamedTuple):
    """``meta.device`` of the reference's Python TensorMeta: ``device_type`` (an int, so
    that raw values survive) and ``device_id``
    (axon/python/tests/test_types_enums.py:171-207).  Still a plain 2-tuple."""

    device_type: int = 1
    device_id: int = 0


class DLDataType(NamedTuple):
    """``meta.dtype``: ``code``, ``bits``, ``lanes``.  Still a plain 3-tuple."""

    code: int = 2
    bits: int = 32
    lanes: int = 1


@dataclass(frozen=True)
class TensorMeta:
    """Fields of the reference's TensorMeta (rpc_core/utils/tensor_meta.hpp:77-82) under
    the names its Python binding gives them (``device.device_type``, ``dtype.bits``,
    ``shape``, ``strides`` ...), so that a memory policy written for the reference reads
    them unchanged, plus the packed offset and size.  ``strides`` is always empty: packed
    tensors are compact (the reference leaves it empty for compact tensors as well,
    axon/python/src/dlpack_helpers.cpp:713-719).  Sequences are tuples, not lists."""

    device: DLDevice = DLDevice()
    ndim: int = 0
    dtype: DLDataType = DLDataType()
    byte_offset: int = 0
    shape: Tuple[int, ...] = ()
    strides: Tuple[int, ...] = ()
    offset: int = 0
    nbytes: int = 0


def _dlpack_stream(stream) -> Optional[int]:
    """``stream`` as the DLPack protocol spells it, or None when the caller named none."""
    return None if stream is None else streams.dlpack_stream_argument(_stream_handle(stream))


def _stream_handle(stream) -> Optional[int]:
    if stream is None:
        return None
    if isinstance(stream, int):
        return stream or None
    for attr in ("cuda_stream", "handle", "ptr"):
        if hasattr(stream, attr):
            return int(getattr(stream, attr)) or None
    raise TypeError(f"cannot take a stream handle from {type(stream).__name__}")


def _refuse_readonly_destinations(arr: TensorArray) -> None:
    if getattr(arr, "readonly", False):
        raise BufferError("a read-only tensor cannot be the destination of an unpack")


class BundlePlan:
    """Layout + device tables of one bundle (``axr_plan_t``)."""

    def __init__(self, handle: int, keepalive: Any = None, receiver: bool = False):
        self._lib = _capi.load()
        self._h = handle
        self._keep = keepalive
        self._receiver = receiver      # made from a header: its tensors are written by unpack

    # ---- construction
    @classmethod
    def create(cls, tensors: Sequence[Any], align: int = 1, stream=None) -> "BundlePlan":
        """Sender side: ``tensors`` are DLPack producers (or TensorViews), laid
        out in argument order.  ``align=1`` is the reference's tight layout.
        ``stream``: the stream the plan will be packed on, when it is known already; producers
        other than torch tensors are then told through ``__dlpack__(stream=...)``."""
        lib = _capi.load()
        # descriptors may be prepared once and reused per call
        arr = tensors if isinstance(tensors, TensorArray) else TensorArray.from_objects(
            tensors, stream=_dlpack_stream(stream))
        h = C.c_void_p()
        _capi.check(lib.axr_plan_create(arr.pointer(), arr.count, align, 0, C.byref(h)))
        return cls(h.value, keepalive=arr)     # the array holds the producers' capsules

    @classmethod
    def from_header(cls, header: bytes) -> "BundlePlan":
        lib = _capi.load()
        buf = bytes(header)
        h = C.c_void_p()
        _capi.check(lib.axr_plan_from_header(buf, len(buf), C.byref(h)))
        return cls(h.value, receiver=True)

    @classmethod
    def from_header_bound(cls, header: bytes, tensors: Sequence[Any]) -> "BundlePlan":
        """``from_header(header).bind(tensors)`` in one pass over the header."""
        lib = _capi.load()
        buf = bytes(header)
        arr = tensors if isinstance(tensors, TensorArray) else TensorArray.from_objects(tensors)
        _refuse_readonly_destinations(arr)
        h = C.c_void_p()
        _capi.check(lib.axr_plan_from_header_bind(buf, len(buf), arr.pointer(), arr.count, C.byref(h)))
        return cls(h.value, keepalive=arr, receiver=True)

    def bind(self, tensors: Sequence[Any], stream=None) -> "BundlePlan":
        arr = tensors if isinstance(tensors, TensorArray) else TensorArray.from_objects(
            tensors, stream=_dlpack_stream(stream))
        if self._receiver:
            _refuse_readonly_destinations(arr)
        _capi.check(self._lib.axr_plan_bind(self._h, arr.pointer(), arr.count))
        self._keep = arr
        return self

    # ---- queries
    @property
    def num_tensors(self) -> int:
        n = C.c_size_t()
        _capi.check(self._lib.axr_plan_num_tensors(self._h, C.byref(n)))
        return n.value

    @property
    def payload_bytes(self) -> int:
        n = C.c_uint64()
        _capi.check(self._lib.axr_plan_payload_bytes(self._h, C.byref(n)))
        return n.value

    @property
    def data_bytes(self) -> int:
        n = C.c_uint64()
        _capi.check(self._lib.axr_plan_data_bytes(self._h, C.byref(n)))
        return n.value

    @property
    def header(self) -> bytes:
        p, n = C.c_void_p(), C.c_size_t()
        _capi.check(self._lib.axr_plan_header(self._h, C.byref(p), C.byref(n)))
        return C.string_at(p.value, n.value) if n.value else b""

    def layout(self) -> Tuple[List[int], List[int]]:
        n = self.num_tensors
        offs = (C.c_uint64 * max(n, 1))()
        sizes = (C.c_uint64 * max(n, 1))()
        _capi.check(self._lib.axr_plan_layout(self._h, offs, sizes))
        return list(offs[:n]), list(sizes[:n])

    def metas(self) -> List[TensorMeta]:
        offs, sizes = self.layout()
        out = []
        t = _capi.Tensor()
        for i in range(len(offs)):
            _capi.check(self._lib.axr_plan_tensor_meta(self._h, i, C.byref(t)))
            out.append(TensorMeta(
                device=DLDevice(t.device_type, t.device_id), ndim=t.ndim,
                dtype=DLDataType(t.dtype_code, t.dtype_bits, t.dtype_lanes), byte_offset=0,
                shape=tuple(t.shape[d] for d in range(t.ndim)), offset=offs[i], nbytes=sizes[i]))
        return out

    def launch_info(self) -> dict:
        info = _capi.LaunchInfo()
        _capi.check(self._lib.axr_plan_launch_info(self._h, C.byref(info)))
        return {f: getattr(info, f) for f, _ in info._fields_ if f != "reserved"}

    def segments(self) -> List[dict]:
        n = C.c_size_t()
        _capi.check(self._lib.axr_plan_segments(self._h, None, 0, C.byref(n)))
        arr = (_capi.SegmentInfo * max(n.value, 1))()
        _capi.check(self._lib.axr_plan_segments(self._h, arr, n.value, C.byref(n)))
        out = []
        for s in arr[:n.value]:
            out.append({
                "tensor": s.tensor, "mode": s.mode, "address": s.address, "offset": s.offset,
                "run_bytes": s.run_bytes, "nbytes": s.nbytes, "pad": s.pad, "ndim": s.ndim,
                "granule": s.granule, "tiles": s.tiles, "head": s.head, "lanes_per_run": s.lanes_per_run,
                "shape": tuple(s.shape[:s.ndim]), "stride_bytes": tuple(s.stride_bytes[:s.ndim]),
            })
        return out

    # ---- data movement
    def prepare(self, stream=None) -> "BundlePlan":
        """Upload the device tables now; pack/unpack are then single kernel launches
        that a HIP graph can capture."""
        _capi.check(self._lib.axr_plan_prepare(self._h, _stream_handle(stream)))
        return self

    def pack(self, payload: int, payload_bytes: int, stream=None, order: bool = True) -> None:
        """Gather on ``stream``.  ``order``: when ``stream`` is not the stream the tensor
        framework is enqueueing on, the kernel is ordered behind what that stream holds now
        (the tensors' producers), with an event and no host wait."""
        handle = _stream_handle(stream)
        if order:
            streams.order_behind_producers(handle)
        _capi.check(self._lib.axr_pack(self._h, payload, payload_bytes, handle))

    def unpack(self, payload: int, payload_bytes: int, stream=None, order: bool = True) -> None:
        """Scatter on ``stream``, ordered behind the framework's stream like ``pack`` (the
        destinations may still be written there).  What the framework enqueues afterwards
        sees the data once ``streams.make_visible_to_producers(stream)`` has been called
        (``unpack_bundle`` does) or the stream has been synchronised."""
        handle = _stream_handle(stream)
        if order:
            streams.order_behind_producers(handle)
        _capi.check(self._lib.axr_unpack(self._h, payload, payload_bytes, handle))

    def split(self, payload: int, payload_bytes: int) -> List[Tuple[int, int]]:
        n = self.num_tensors
        views = (_capi.Buffer * max(n, 1))()
        _capi.check(self._lib.axr_plan_split(self._h, payload, payload_bytes, views))
        return [(views[i].data or 0, views[i].size) for i in range(n)]

    def close(self) -> None:
        if self._h:
            _capi.check(self._lib.axr_plan_free(self._h))
            self._h = None
            self._keep = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            if self._h:
                self._lib.axr_plan_free(self._h)
        except Exception:  # noqa: BLE001
            pass


@dataclass
class PackedBundle:
    """What goes on the wire: the AM header bytes and the contiguous payload
    (``ucx_am_data{header, buffer, buffer_type=ROCM, mem_h}``,
    ucx_context/ucx_context_def.h:80-93)."""

    header: bytes
    payload: PoolBuffer
    payload_bytes: int
    plan: BundlePlan

    @property
    def mem_h(self):
        return self.payload.mem_h

    def close(self) -> None:
        """Release the plan first (it waits for the pack kernel on its stream), then
        return the payload block to the pool: a pool block is reusable the moment it
        is freed, so it must not be freed while the kernel may still write it."""
        if self.plan is not None:
            self.plan.close()
        if self.payload is not None:
            self.payload.release()

    def __del__(self):
        # Dropping the object must not free the payload before the plan has drained the
        # pack stream (the fields would otherwise go in declaration order, payload first).
        # The payload itself is left to its own reference count: zero-copy views made
        # from it may still be alive.
        try:
            if self.plan is not None:
                self.plan.close()
        except Exception:  # noqa: BLE001
            pass


def pack_bundle(tensors: Sequence[Any], align: int = 256, pool: Optional[DevicePool] = None,
                stream=None) -> PackedBundle:
    """Gather ``tensors`` into one pool buffer on ``stream`` (asynchronous).  The kernel is
    ordered behind the stream that produced the tensors; no synchronisation is needed between
    producing them and this call."""
    plan = BundlePlan.create(tensors, align=align, stream=stream)
    pool = pool or DevicePool.default()
    nbytes = plan.payload_bytes
    buf = pool.alloc(max(nbytes, 1), 256)
    plan.pack(buf.data, nbytes, stream)
    return PackedBundle(plan.header, buf, nbytes, plan)


def unpack_bundle(header: bytes, payload: Any, payload_bytes: Optional[int] = None,
                  out: Optional[Sequence[Any]] = None, stream=None,
                  from_dlpack_fn: Optional[Callable[[Any], Any]] = None):
    """Receiver side.

    With ``out`` (DLPack producers of matching size): scatter the payload into
    them with one kernel launch and return the plan (keep it until the stream
    has drained).  Without ``out``: zero-copy mode, the payload is split at the
    header's offsets and each piece is returned as a DLPack producer over the
    payload memory (``from_dlpack_fn`` converts them, e.g. ``torch.from_dlpack``),
    typed and shaped from the header.

    The scatter is ordered behind the tensor framework's stream (the destinations may still
    be written there), and that stream is made to wait for the scatter, so the framework's
    next kernels see the data without a host synchronisation.
    """
    if isinstance(payload, PoolBuffer):
        ptr, size = payload.data, payload.size
    else:
        ptr, size = int(payload), payload_bytes
    if payload_bytes is not None:
        size = payload_bytes
    plan = BundlePlan.from_header(header)
    if out is not None:
        plan.bind(out, stream=stream)
        plan.unpack(ptr, size, stream)
        streams.make_visible_to_producers(_stream_handle(stream))
        return plan
    pieces = plan.split(ptr, size)
    metas = plan.metas()
    owner = payload  # every view keeps the payload block alive
    # the views live where the payload does: on the receiver's current device, whatever
    # ordinal the sender's tensors had (the reference writes 0, dlpack_helpers.cpp:82-114)
    device = C.c_int(0)
    _capi.check(_capi.load().axr_device_get(C.byref(device)))
    results = []
    scalars = None
    for (p, n), m in zip(pieces, metas):
        keep = owner
        if len(m.shape) == 0:
            # A 0-d tensor has no bytes in the payload (the reference's size rule,
            # rpc_core/utils/tensor_meta.hpp:91-104), yet its consumer will read one element:
            # it is pointed at a zeroed block of its own instead of at whatever follows its
            # offset in the payload (possibly the end of the allocation).
            if scalars is None:
                lib = _capi.load()
                scalars = DevicePool.default().alloc(256, 256)
                _capi.check(lib.axr_memset_async(scalars.data, 0, 256, None))
                _capi.check(lib.axr_stream_synchronize(None))
            p, keep = scalars.data, scalars
        exp = DLPackExport(p, m.shape, m.dtype, _capi.kDLROCM, device.value,
                           release=(lambda keep=keep: None))
        results.append(from_dlpack_fn(exp) if from_dlpack_fn else exp)
    plan.close()
    return results


def bundle_to_host(header: bytes, payload: Any, payload_bytes: Optional[int] = None,
                   stream=None) -> List[Any]:
    """The tensors of a device payload as host ``numpy`` byte arrays, one per
    tensor: the staging a checkpoint writer needs (the reference copies buffer by
    buffer with ``mr.memcpy(HOST, ...)``, axon/src/storage/avro_serialization.cpp:478-523).
    The payload crosses the bus in 8 MiB pinned blocks, one device copy per block
    whatever the tensor count.  Returns when the arrays are filled."""
    import numpy as np

    from .dlpack import TensorView
    if isinstance(payload, PoolBuffer):
        ptr, size = payload.data, payload.size
    else:
        ptr, size = int(payload), payload_bytes
    if payload_bytes is not None:
        size = payload_bytes
    with BundlePlan.from_header(header) as plan:
        metas = plan.metas()
        arrays = [np.empty(m.nbytes, dtype=np.uint8) for m in metas]
        views = [TensorView(data=a.ctypes.data if a.size else 0, device_type=_capi.kDLCPU, device_id=0,
                            dtype=m.dtype, shape=tuple(m.shape), strides=None)
                 for a, m in zip(arrays, metas)]
        plan.bind(views)
        plan.unpack(ptr, size, stream)
    return arrays
