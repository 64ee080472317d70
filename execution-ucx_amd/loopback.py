"""Loopback active-message context: the AM-bundle API of the reference's
``ucx_am_context`` (``connection_send`` / ``connection_recv_header`` /
``connection_recv_buffer``, ucx_context/ucx_context_concept.hpp:247-470) between
two contexts of one process, for machines without UCX.  The behaviour kept is
listed with the C declarations in ``include/axon_rocm.h``.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

from . import _capi
from .bundle import PackedBundle, _stream_handle
from .memory import DevicePool, PoolBuffer, ROCM


@dataclass
class AmMessage:
    key: int
    conn_id: int
    header: bytes
    data_length: int
    is_rndv: bool
    buffer_type: int
    eager_data: Optional[bytes]     # payload of an eager message (host memory), else None


class LoopbackAmContext:
    def __init__(self, name: str = "", zcopy_thresh: int = 0):
        self._lib = _capi.load()
        h = C.c_void_p()
        _capi.check(self._lib.axr_am_context_create(name.encode(), zcopy_thresh, C.byref(h)))
        self._h = h.value
        self.name = name
        self._keep = {}      # request -> objects the transport may still read

    def connect(self, peer: "LoopbackAmContext") -> int:
        cid = C.c_uint64()
        _capi.check(self._lib.axr_am_connect(self._h, peer._h, C.byref(cid)))
        return cid.value

    # ---- send
    def send(self, conn_id: int, header: bytes, payload: int = 0, nbytes: int = 0,
             memory_type: int = ROCM, mem_h: Optional[int] = None, stream=None, keep=None) -> int:
        """connection_send of one contiguous payload; returns a request id."""
        hdr = bytes(header)
        d = _capi.AmData()
        d.header = _capi.Buffer(C.cast(C.c_char_p(hdr), C.c_void_p).value if hdr else None, len(hdr))
        d.buffer = _capi.Buffer(payload or None, nbytes)
        d.buffer_type = memory_type
        d.mem_h = mem_h
        req = C.c_uint64()
        _capi.check(self._lib.axr_am_send(self._h, conn_id, C.byref(d), _stream_handle(stream), C.byref(req)))
        self._keep[req.value] = keep
        return req.value

    def send_iov(self, conn_id: int, header: bytes, buffers: Sequence[Tuple[int, int]],
                 memory_type: int = ROCM, stream=None, keep=None) -> int:
        """connection_send of an iov payload (always rendezvous): the reference's way
        of sending a tensor list (ucx_connection.cpp:401-426)."""
        hdr = bytes(header)
        n = len(buffers)
        vec = (_capi.Buffer * max(n, 1))()
        for i, (p, s) in enumerate(buffers):
            vec[i] = _capi.Buffer(p or None, s)
        d = _capi.AmIovec()
        d.header = _capi.Buffer(C.cast(C.c_char_p(hdr), C.c_void_p).value if hdr else None, len(hdr))
        d.buffer_vec = C.cast(vec, C.POINTER(_capi.Buffer)) if n else None
        d.buffer_count = n
        d.buffer_type = memory_type
        req = C.c_uint64()
        _capi.check(self._lib.axr_am_send_iov(self._h, conn_id, C.byref(d), _stream_handle(stream), C.byref(req)))
        self._keep[req.value] = keep
        return req.value

    def send_bundle(self, conn_id: int, bundle: PackedBundle, stream=None) -> int:
        """Send a packed bundle as ONE contiguous ROCM payload with the bundle header
        as the AM header.  The pack must have finished before the transport reads
        the buffer, so the stream is drained first."""
        _capi.check(self._lib.axr_stream_synchronize(_stream_handle(stream)))
        return self.send(conn_id, bundle.header, bundle.payload.data, bundle.payload_bytes, ROCM,
                         bundle.mem_h, stream, keep=bundle)

    def test(self, request: int) -> bool:
        """True once the send has completed (raises if it was cancelled)."""
        done = C.c_int()
        _capi.check(self._lib.axr_am_request_test(self._h, request, C.byref(done)))
        if done.value < 0:
            self._keep.pop(request, None)
            raise _capi.AxonRocmError(_capi.AXR_ERR_HIP, "send was cancelled or failed at the receiver")
        if done.value:
            self._keep.pop(request, None)
        return bool(done.value)

    def cancel(self, request: int) -> None:
        """Sender-side cancellation of a send that has not completed (a waiting send is
        dropped, an unfetched rendezvous disappears at the receiver); ``test`` then raises."""
        _capi.check(self._lib.axr_am_request_cancel(self._h, request))

    def progress(self) -> Tuple[int, int]:
        """Start waiting sends where completions made room; returns (sends in flight, sends
        waiting).  A context admits 256 uncompleted sends (ucx_am_context.hpp:94)."""
        a, b = C.c_size_t(), C.c_size_t()
        _capi.check(self._lib.axr_am_progress(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    # ---- receive
    def pending(self) -> int:
        n = C.c_size_t()
        _capi.check(self._lib.axr_am_pending(self._h, C.byref(n)))
        return n.value

    def recv_header(self, release_eager: bool = True) -> Optional[AmMessage]:
        """connection_recv_header: the next message, or None when nothing arrived.
        An eager message carries its payload; its descriptor is dropped at once
        unless ``release_eager`` is False (then call ``release``)."""
        m = _capi.AmMessage()
        rc = self._lib.axr_am_recv_header(self._h, C.byref(m))
        if rc == _capi.AXR_ERR_NO_MESSAGE:
            return None
        _capi.check(rc)
        header = C.string_at(m.header.data, m.header.size) if m.header.size else b""
        eager = None
        if not m.is_rndv:
            eager = C.string_at(m.eager_data.data, m.eager_data.size) if m.eager_data.size else b""
            if release_eager:
                _capi.check(self._lib.axr_am_message_release(self._h, m.key))
        return AmMessage(m.key, m.conn_id, header, m.data_length, bool(m.is_rndv), m.buffer_type, eager)

    def recv_buffer(self, message: AmMessage, dst: Optional[PoolBuffer] = None,
                    pool: Optional[DevicePool] = None, stream=None) -> PoolBuffer:
        """connection_recv_buffer(key, UcxBuffer): fetch into one contiguous ROCM buffer;
        like the reference (ucx_am_context.hpp:1604-1621) a missing or too small
        buffer is (re)allocated, here from the device pool."""
        if dst is None or dst.size < message.data_length:
            if dst is not None:
                dst.release()
            dst = (pool or DevicePool.default()).alloc(max(message.data_length, 1), 256)
        _capi.check(self._lib.axr_am_recv_buffer(self._h, message.key, ROCM, dst.data, dst.size,
                                                 _stream_handle(stream)))
        return dst

    def recv_into(self, message: AmMessage, ptr: int, nbytes: int, memory_type: int = ROCM,
                  stream=None, wait: bool = True) -> None:
        """Fetch into caller memory.  ``wait=False`` only enqueues the copies on
        ``stream`` (work ordered after them on that stream sees the data)."""
        fn = self._lib.axr_am_recv_buffer if wait else self._lib.axr_am_recv_buffer_async
        _capi.check(fn(self._h, message.key, memory_type, ptr, nbytes, _stream_handle(stream)))

    def recv_buffer_iov(self, message: AmMessage, buffers: Sequence[Tuple[int, int]],
                        memory_type: int = ROCM, stream=None) -> None:
        """connection_recv_buffer(key, UcxBufferVec): scatter in order into
        pre-allocated, non-empty entries (ucx_am_context.hpp:1808-1818)."""
        n = len(buffers)
        vec = (_capi.Buffer * max(n, 1))()
        for i, (p, s) in enumerate(buffers):
            vec[i] = _capi.Buffer(p or None, s)
        _capi.check(self._lib.axr_am_recv_buffer_iov(self._h, message.key, memory_type, vec, n,
                                                     _stream_handle(stream)))

    def release(self, message: AmMessage) -> None:
        _capi.check(self._lib.axr_am_message_release(self._h, message.key))

    def close(self) -> None:
        if self._h:
            _capi.check(self._lib.axr_am_context_destroy(self._h))
            self._h = None
        self._keep.clear()      # sends that were never test()ed: nothing reads their bundles any more

    def __del__(self):
        try:
            if self._h:
                self._lib.axr_am_context_destroy(self._h)
        except Exception:  # noqa: BLE001
            pass
