"""Ordering between the stream that produced the tensors and the stream a bundle runs on.

A DLPack producer's data is ready on the PRODUCER's stream; the DLPack protocol makes the
consumer say which stream it will read on (``__dlpack__(stream=...)``) so that the producer
can order the two.  The reference never launches a kernel on the tensors: it keeps the
owners alive until the transport has finished and relies on the transport's own ordering
(axon/python/src/dlpack_helpers.cpp:136-156, 739-742).  Here the pack and unpack kernels
run on a stream of the caller's choice, which may be a non-blocking stream that does not
synchronise with the producer's, so the order is made explicit:

* before a launch on stream S, ``order_behind_producers(S)`` records an event on the
  producer's current stream P and makes S wait for it (nothing when S is P);
* after a launch, ``make_visible_to_producers(S)`` does the reverse, so that what the
  framework enqueues next on P sees the kernel's writes.

Both are stream-ordered (no host wait).  "The producer's stream" is the current stream of
the framework whose tensors are in play: torch's, when torch is loaded and has a GPU
context.  Producers of other frameworks are handed the consumer stream through
``__dlpack__(stream=...)`` (``dlpack.extract``), which is their half of the same handshake.
"""
from __future__ import annotations

import ctypes as C
import sys
import threading
from typing import Optional

from . import _capi

# (device, direction) -> event handle.  An event may be recorded again while an earlier wait
# on it is still queued: a wait captures the record that was current when it was enqueued.
# Record and wait are enqueued as a pair under a lock: the producer's stream is per thread
# (torch's current stream is thread-local), and another thread's record between the two
# would make this thread wait for the wrong stream.
_events = {}
_pair_lock = threading.Lock()


def _event(device: int, direction: int) -> int:
    key = (device, direction)
    ev = _events.get(key)
    if ev is None:
        h = C.c_void_p()
        _capi.check(_capi.load().axr_event_create(C.byref(h)))
        ev = _events[key] = h.value
    return ev


def producer_stream() -> Optional[tuple]:
    """``(device, raw handle)`` of the stream the tensor framework currently enqueues on (0
    is the device's default stream), or None when no framework with a GPU context is loaded."""
    torch = sys.modules.get("torch")
    if torch is None or not torch.cuda.is_initialized():
        return None
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    get_device = getattr(torch._C, "_cuda_getDevice", None)
    if raw is not None and get_device is not None:
        device = get_device()
        return device, int(raw(device))
    return torch.cuda.current_device(), int(torch.cuda.current_stream().cuda_stream)


def _order(later: Optional[int], earlier: Optional[int], device: int, direction: int) -> None:
    lib = _capi.load()
    with _pair_lock:
        ev = _event(device, direction)
        _capi.check(lib.axr_event_record(ev, earlier or None))
        _capi.check(lib.axr_stream_wait_event(later or None, ev))


def order_behind_producers(stream: Optional[int]) -> bool:
    """Work enqueued on ``stream`` (a raw handle; None or 0: the default stream) from now on
    runs after everything the producer's stream holds now.  Returns True when a wait was
    inserted, False when the two are the same stream or there is no producer stream."""
    prod = producer_stream()
    if prod is None:
        return False
    device, raw = prod
    if (stream or 0) == raw:
        return False
    _order(stream, raw, device, 0)
    return True


def make_visible_to_producers(stream: Optional[int]) -> bool:
    """What the producer's stream is given from now on runs after everything ``stream``
    holds now (the unpack kernel's writes into the framework's tensors)."""
    prod = producer_stream()
    if prod is None:
        return False
    device, raw = prod
    if (stream or 0) == raw:
        return False
    _order(raw, stream, device, 1)
    return True


def dlpack_stream_argument(stream: Optional[int]) -> int:
    """The ``stream`` argument of ``__dlpack__`` for a consumer that reads on ``stream`` on a
    ROCm device: 0 is not allowed there, 1 names the legacy default stream, 2 the per-thread
    default stream, anything else is the stream's handle."""
    return int(stream) if stream else 1
