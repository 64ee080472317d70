"""Streamed transfer of a large payload in chunks: double-buffered
pack -> loopback send -> unpack on two HIP streams of one GPU.

Chunk k runs entirely on stream k % 2: the pack kernel writes send slot k % 2,
the loopback transport copies it into receive slot k % 2 (the same-device stand-in
for the wire), the unpack kernel scatters it.  Stream order makes a slot safe to
reuse two chunks later, and the two streams let chunk k + 1's pack overlap chunk
k's copy and unpack.  Nothing blocks the host until ``finish``.
"""
from __future__ import annotations

import ctypes as C
from typing import Any, List, Sequence

from . import _capi
from .bundle import BundlePlan
from .loopback import LoopbackAmContext
from .memory import DevicePool, ROCM


class StreamedTransfer:
    def __init__(self, slot_bytes: int, pool: DevicePool = None, streams: int = 2, align: int = 256):
        self._lib = _capi.load()
        self.pool = pool or DevicePool.default()
        self.align = align
        self.streams = []
        for _ in range(streams):
            s = C.c_void_p()
            _capi.check(self._lib.axr_stream_create(C.byref(s)))
            self.streams.append(s.value)
        self.send_slots = [self.pool.alloc(slot_bytes, 256) for _ in range(streams)]
        self.recv_slots = [self.pool.alloc(slot_bytes, 256) for _ in range(streams)]
        self.slot_bytes = slot_bytes
        self.client = LoopbackAmContext("stream-client")
        self.server = LoopbackAmContext("stream-server")
        self.conn = self.client.connect(self.server)
        self._inflight: List[Any] = [None] * streams     # per slot: (plans, request, event, keep)
        self._events = []
        for _ in range(streams):
            ev = C.c_void_p()
            _capi.check(self._lib.axr_event_create(C.byref(ev)))
            self._events.append(ev.value)
        self._k = 0

    def _retire(self, i: int) -> None:
        """Wait for the chunk that last used slot i and recycle its plans (their
        device tables go back to the table cache)."""
        item = self._inflight[i]
        if item is None:
            return
        plans, req, _keep = item
        _capi.check(self._lib.axr_event_synchronize(self._events[i]))
        if not self.client.test(req):
            raise _capi.AxonRocmError(_capi.AXR_ERR_HIP, "a chunk's send did not complete")
        for p in plans:
            p.close()
        self._inflight[i] = None

    def submit(self, src_views: Sequence[Any], dst_views: Sequence[Any]) -> None:
        """Queue one chunk: gather src_views, move, scatter into dst_views."""
        i = self._k % len(self.streams)
        self._k += 1
        stream = self.streams[i]
        self._retire(i)
        keep = None
        plan = BundlePlan.create(src_views, align=self.align)
        nbytes = plan.payload_bytes
        if nbytes > self.slot_bytes:
            raise _capi.LengthError(_capi.AXR_ERR_LENGTH, "chunk is larger than a pipeline slot")
        plan.pack(self.send_slots[i].data, nbytes, stream)
        req = self.client.send(self.conn, plan.header, self.send_slots[i].data, nbytes, ROCM,
                               self.send_slots[i].mem_h, stream)
        msg = self.server.recv_header()
        if msg.is_rndv:
            self.server.recv_into(msg, self.recv_slots[i].data, nbytes, ROCM, stream, wait=False)
        else:   # small chunk: arrived eagerly in host memory
            host = C.create_string_buffer(msg.eager_data, len(msg.eager_data))
            _capi.check(self._lib.axr_memcpy_async(ROCM, self.recv_slots[i].data, _capi.MEM_HOST,
                                                   C.addressof(host), nbytes, stream))
            keep = host
        rplan = BundlePlan.from_header(msg.header).bind(dst_views)
        rplan.unpack(self.recv_slots[i].data, nbytes, stream)
        _capi.check(self._lib.axr_event_record(self._events[i], stream))
        self._inflight[i] = ((plan, rplan), req, keep)

    def finish(self) -> None:
        """Wait for every queued chunk."""
        for i in range(len(self.streams)):
            self._retire(i)

    def close(self) -> None:
        self.finish()
        for b in self.send_slots + self.recv_slots:
            b.release()
        for s in self.streams:
            _capi.check(self._lib.axr_stream_destroy(s))
        for ev in self._events:
            _capi.check(self._lib.axr_event_destroy(ev))
        self.streams = []
        self._events = []
        self.client.close()
        self.server.close()
