"""Tensor lists over an active-message context: the sender and receiver halves of
what the reference's Python ``invoke`` does with tensor arguments
(axon/python/src/bindings_runtime.cpp:910-1018), reduced to the payload path.

    request, bundle = send_tensors(client, conn, [a, b, c])
    tensors = recv_tensors(server, memory_policy=lambda metas: [torch.empty(...) ...])

The receive side follows the reference's memory-policy contract
(axon/python/src/memory_policy_helpers.cpp:44-140): the policy is called with the
tensor metas and returns a tensor or a list of tensors to receive into, and those
same objects are handed back.  Without a policy the tensors are zero-copy views
over the received buffer (UcxBuffer::to_buffer_vec,
ucx_context/ucx_context_data.hpp:641-665).
"""
from __future__ import annotations

import ctypes as C
from typing import Any, Callable, List, Optional, Sequence, Tuple

from . import _capi
from .bundle import BundlePlan, PackedBundle, TensorMeta, pack_bundle, unpack_bundle
from .loopback import AmMessage, LoopbackAmContext
from .memory import DevicePool, PoolBuffer, ROCM


def send_tensors(ctx: LoopbackAmContext, conn_id: int, tensors: Sequence[Any], align: int = 256,
                 stream=None, pool: Optional[DevicePool] = None) -> Tuple[int, PackedBundle]:
    """Pack ``tensors`` into one pool buffer and send it as one contiguous payload.
    Keep the returned bundle until ``ctx.test(request)`` is true."""
    bundle = pack_bundle(tensors, align=align, pool=pool, stream=stream)
    request = ctx.send_bundle(conn_id, bundle, stream=stream)
    return request, bundle


def _payload_on_device(ctx: LoopbackAmContext, msg: AmMessage, pool: DevicePool, stream) -> PoolBuffer:
    if msg.is_rndv:
        return ctx.recv_buffer(msg, pool=pool, stream=stream)
    # eager payloads arrive in host memory (ucx_am_context.hpp:1274-1278) and reach
    # the device through the memory resource's copy (:1258-1260)
    buf = pool.alloc(max(msg.data_length, 1), 256)
    if msg.data_length:
        host = C.create_string_buffer(msg.eager_data, msg.data_length)
        _capi.check(_capi.load().axr_memcpy(ROCM, buf.data, _capi.MEM_HOST, C.addressof(host),
                                            msg.data_length))
    return buf


def recv_tensors(ctx: LoopbackAmContext,
                 memory_policy: Optional[Callable[[List[TensorMeta]], Any]] = None,
                 from_dlpack_fn: Optional[Callable[[Any], Any]] = None, stream=None,
                 pool: Optional[DevicePool] = None) -> Optional[List[Any]]:
    """Receive the next tensor bundle, or None when no message is queued."""
    msg = ctx.recv_header()
    if msg is None:
        return None
    pool = pool or DevicePool.default()
    payload = _payload_on_device(ctx, msg, pool, stream)
    if memory_policy is None:
        return unpack_bundle(msg.header, payload, payload_bytes=msg.data_length,
                             from_dlpack_fn=from_dlpack_fn)
    metas = BundlePlan.from_header(msg.header)
    wanted = metas.metas()
    metas.close()
    out = memory_policy(wanted)
    single = not isinstance(out, (list, tuple))
    outs = [out] if single else list(out)
    if len(outs) != len(wanted):
        payload.release()
        raise RuntimeError("Memory policy returned incompatible buffer type")   # axon_worker.cpp:1161-1166
    plan = unpack_bundle(msg.header, payload, payload_bytes=msg.data_length, out=outs, stream=stream)
    plan.close()          # waits for the scatter on its stream
    payload.release()
    return outs
