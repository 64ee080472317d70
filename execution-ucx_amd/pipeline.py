"""Streamed transfer of a large payload in chunks: double-buffered
pack -> loopback send -> unpack on two HIP streams of one GPU.

The work is done by the library's ``axr_transfer_*`` object (C ABI): chunk k runs
entirely on lane k % lanes (a stream with a send slot and a receive slot), so stream
order makes a slot safe to reuse two chunks later and chunk k + 1's pack overlaps chunk
k's wire copy and unpack.  Chunks of one geometry share ONE sender plan and ONE
receiver plan; each chunk only names how far its tensors lie from the ones the plans
were bound to.  Nothing blocks the host until ``finish`` (beyond waiting for the chunk
that last used a lane).
"""
from __future__ import annotations

import ctypes as C
from typing import Any, List, Optional, Sequence, Tuple

from . import _capi
from .bundle import BundlePlan
from .dlpack import TensorArray
from .memory import DevicePool


def _geometry(arr: TensorArray) -> Tuple[int, tuple]:
    """(address of the first tensor, everything else relative to it).  A bundle with host
    (kDLCPU) tensors cannot be moved to another base by an address delta (their pieces are
    copied by the host, from the addresses the plan was bound to), so its key also holds the
    base itself: host chunks at another address plan anew instead of being rebased."""
    n = arr.count
    if n == 0:
        return 0, ()
    a = arr.array
    base = (a[0].data or 0) + a[0].byte_offset
    key = []
    if any(a[i].device_type == _capi.kDLCPU for i in range(n)):
        key.append(("host tensors at", base))
    for i in range(n):
        t = a[i]
        nd = t.ndim
        key.append(((t.data or 0) + t.byte_offset - base, t.device_type, t.device_id, t.dtype_code,
                    t.dtype_bits, t.dtype_lanes, tuple(t.shape[:nd]),
                    tuple(t.strides[:nd]) if t.strides else None))
    return base, tuple(key)


class StreamedTransfer:
    def __init__(self, slot_bytes: int, pool: Optional[DevicePool] = None, streams: int = 2,
                 align: int = 256, lanes: Optional[int] = None, zero_copy: bool = True):
        """``lanes`` slot pairs (default: max(2, streams)) over ``streams`` HIP streams.
        ``zero_copy``: the receiver unpacks straight out of the sender's slot (a same-device
        zero-copy rendezvous); False copies every chunk into a receive slot first."""
        self._lib = _capi.load()
        self.pool = pool or DevicePool.default()
        self.align = align
        self.slot_bytes = slot_bytes
        h = C.c_void_p()
        lanes = max(2, streams) if lanes is None else lanes
        _capi.check(self._lib.axr_transfer_create(self.pool._h, slot_bytes, lanes, streams, C.byref(h)))
        self._h = h.value
        if not zero_copy:
            _capi.check(self._lib.axr_transfer_set_zero_copy(self._h, 0))
        self._plans = None            # (src key, dst key, src base, dst base, send plan, recv plan)
        self._keep: List[Any] = []    # descriptor arrays of chunks that may still be in flight

    def submit_plans(self, send_plan: BundlePlan, send_delta: int, recv_plan: BundlePlan,
                     recv_delta: int) -> None:
        """Queue one chunk with plans the caller keeps: the sender's tensors lie
        ``send_delta`` bytes from the ones ``send_plan`` is bound to, the receiver's
        ``recv_delta`` bytes from ``recv_plan``'s."""
        _capi.check(self._lib.axr_transfer_submit(self._h, send_plan._h, send_delta, recv_plan._h,
                                                  recv_delta))

    def submit(self, src_views: Sequence[Any], dst_views: Sequence[Any]) -> None:
        """Queue one chunk: gather src_views, move, scatter into dst_views.  Chunks whose
        tensors have the shapes, strides and mutual distances of the previous chunk reuse
        its plans; another geometry drains the pipeline and plans anew."""
        sa = src_views if isinstance(src_views, TensorArray) else TensorArray.from_objects(src_views)
        da = dst_views if isinstance(dst_views, TensorArray) else TensorArray.from_objects(dst_views)
        sbase, skey = _geometry(sa)
        dbase, dkey = _geometry(da)
        p = self._plans
        if p is None or p[0] != skey or p[1] != dkey:
            self.finish()
            self._drop_plans()
            send = BundlePlan.create(sa, align=self.align)
            try:
                if send.payload_bytes > self.slot_bytes:
                    raise _capi.LengthError(_capi.AXR_ERR_LENGTH, "chunk is larger than a pipeline slot")
                recv = BundlePlan.from_header(send.header).bind(da)
            except BaseException:
                send.close()
                raise
            p = self._plans = (skey, dkey, sbase, dbase, send, recv)
        self._keep.append((sa, da))
        self.submit_plans(p[4], sbase - p[2], p[5], dbase - p[3])

    def _drop_plans(self) -> None:
        if self._plans is not None:
            self._plans[4].close()
            self._plans[5].close()
            self._plans = None

    def finish(self) -> None:
        """Wait for every queued chunk."""
        _capi.check(self._lib.axr_transfer_finish(self._h))
        self._keep.clear()

    def close(self) -> None:
        if self._h:
            try:
                self.finish()
            finally:
                self._drop_plans()
                _capi.check(self._lib.axr_transfer_destroy(self._h))
                self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass
