"""Tensor lists over an active-message context: the sender and receiver halves of
what the reference's Python ``invoke`` does with tensor arguments
(axon/python/src/bindings_runtime.cpp:910-1018), reduced to the payload path.

    request, bundle = send_tensors(client, conn, [a, b, c])
    tensors = recv_tensors(server, memory_policy=lambda metas: [torch.empty(...) ...])

``send_arguments`` / ``recv_arguments`` carry the argument structure as well: each
argument is a tensor, a list of tensors or a list of lists of tensors, classified and
flattened into one tensor stream in argument order the way the reference's
InvokeContext does it (axon/python/src/bindings_runtime_helpers.hpp:262-330,
351-414), with the group sizes of nested lists travelling as uint32 counts in front
of the bundle header so that the receiver rebuilds the same nesting
(axon/python/src/bindings_runtime_wrapper.cpp:183-228).

The receive side follows the reference's memory-policy contract
(axon/python/src/memory_policy_helpers.cpp:44-140): the policy is called with the
tensor metas and returns a tensor or a list of tensors to receive into, and those
same objects are handed back.  Without a policy the tensors are zero-copy views
over the received buffer (UcxBuffer::to_buffer_vec,
ucx_context/ucx_context_data.hpp:641-665).
"""
from __future__ import annotations

import ctypes as C
import struct
from typing import Any, Callable, List, Optional, Sequence, Tuple

from . import _capi
from .bundle import BundlePlan, PackedBundle, TensorMeta, _stream_handle, pack_bundle, unpack_bundle
from .dlpack import TensorView
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
    return _receive(ctx, msg, msg.header, memory_policy, from_dlpack_fn, stream, pool)


def _host_views(plan: BundlePlan, metas: Sequence[TensorMeta], host, from_dlpack_fn) -> List[Any]:
    """kDLCPU producers over ``host`` (a numpy byte array holding the whole payload), split at
    the header's offsets; every view keeps the array alive."""
    from .dlpack import DLPackExport
    import numpy as np
    pieces = plan.split(host.ctypes.data if host.size else 0, host.size)
    out = []
    for (p, _n), m in zip(pieces, metas):
        keep = host
        if len(m.shape) == 0:       # no bytes in the payload, one element read by the consumer
            keep = np.zeros(32, dtype=np.uint8)
            p = keep.ctypes.data
        exp = DLPackExport(p, m.shape, m.dtype, _capi.kDLCPU, 0, release=(lambda keep=keep: None))
        out.append(from_dlpack_fn(exp) if from_dlpack_fn else exp)
    return out


def _receive_without_policy(ctx, msg, bundle_header, from_dlpack_fn, stream, pool) -> List[Any]:
    """Tensors that were in host memory at the sender arrive in host memory (the reference's
    default receive memory is host, axon/src/axon_worker.cpp:1098-1219, and an eager payload
    is in host memory when it is delivered, ucx_context/ucx_am_context/ucx_am_context.cpp:864-953),
    so that ``numpy.from_dlpack`` can take them; device tensors arrive as views of the
    received device payload."""
    import numpy as np
    with BundlePlan.from_header(bundle_header) as plan:
        metas = plan.metas()
        on_host = [m.device.device_type == _capi.kDLCPU and m.nbytes > 0 for m in metas]
        if not any(on_host):
            payload = _payload_on_device(ctx, msg, pool, stream)
            return unpack_bundle(bundle_header, payload, payload_bytes=msg.data_length,
                                 from_dlpack_fn=from_dlpack_fn)
        everything_on_host = all(h or m.nbytes == 0 for h, m in zip(on_host, metas))
        if everything_on_host and not msg.is_rndv:        # the bytes are on the host already
            host = np.frombuffer(msg.eager_data, dtype=np.uint8, count=msg.data_length).copy()
            return _host_views(plan, metas, host, from_dlpack_fn)
        payload = _payload_on_device(ctx, msg, pool, stream)
        try:
            host = np.empty(msg.data_length, dtype=np.uint8)
            if msg.data_length:                            # one copy of the whole payload
                _capi.check(_capi.load().axr_memcpy(_capi.MEM_HOST, host.ctypes.data, ROCM, payload.data,
                                                    msg.data_length))
            views = _host_views(plan, metas, host, None)
            if not everything_on_host:
                device_views = unpack_bundle(bundle_header, payload, payload_bytes=msg.data_length)
                views = [h if is_host else d for h, d, is_host in zip(views, device_views, on_host)]
            return [from_dlpack_fn(v) if from_dlpack_fn else v for v in views]
        finally:
            if everything_on_host:
                payload.release()


def _receive(ctx, msg, bundle_header, memory_policy, from_dlpack_fn, stream, pool) -> List[Any]:
    pool = pool or DevicePool.default()
    if memory_policy is None:
        return _receive_without_policy(ctx, msg, bundle_header, from_dlpack_fn, stream, pool)
    payload = _payload_on_device(ctx, msg, pool, stream)
    metas = BundlePlan.from_header(bundle_header)
    wanted = metas.metas()
    metas.close()
    out = memory_policy(wanted)
    single = not isinstance(out, (list, tuple))
    outs = [out] if single else list(out)
    if len(outs) != len(wanted):
        payload.release()
        raise RuntimeError("Memory policy returned incompatible buffer type")   # axon_worker.cpp:1161-1166
    plan = unpack_bundle(bundle_header, payload, payload_bytes=msg.data_length, out=outs, stream=stream)
    plan.close()          # waits for the scatter on its stream
    payload.release()
    return outs


# ------------------------------------------------------------------ argument structure

SINGLE_TENSOR, FLAT_TENSOR_LIST, NESTED_TENSOR_LIST = 1, 2, 3
_ARGS_MAGIC = b"AXAG"


def _is_tensor(obj: Any) -> bool:
    return (hasattr(obj, "__dlpack__") or isinstance(obj, TensorView)
            or type(obj).__name__ == "PyCapsule")


def classify_argument(arg: Any) -> int:
    """ClassifyArg (bindings_runtime_helpers.hpp:262-330) for the tensor kinds; what the
    reference would send as a non-tensor parameter is a TypeError here, because only
    tensors travel on this path."""
    if _is_tensor(arg):
        return SINGLE_TENSOR
    if not isinstance(arg, (list, tuple)):
        raise TypeError(f"{type(arg).__name__} is not a tensor argument")
    if len(arg) == 0:
        return FLAT_TENSOR_LIST                      # an empty List[Tensor]
    first = arg[0]
    if _is_tensor(first):
        return FLAT_TENSOR_LIST
    if isinstance(first, (list, tuple)):
        for inner in arg:
            if not isinstance(inner, (list, tuple)):
                raise TypeError("Heterogeneous sequences are not supported as RPC arguments: expected "
                                "all elements to be sequences (list/tuple) for List[List[Tensor]]")
            if len(inner) == 0:
                continue                             # empty inner lists are skipped over
            if _is_tensor(inner[0]):
                return NESTED_TENSOR_LIST
            raise TypeError("Unsupported element type inside nested sequence: expected a "
                            "DLPack-compatible tensor for a List[List[Tensor]] argument")
    raise TypeError("argument holds no tensors")


def flatten_arguments(args: Sequence[Any]) -> Tuple[List[Any], List[Tuple[int, List[int]]]]:
    """All tensors of ``args`` in argument order plus, per argument, its kind and counts:
    ``[]`` for a single tensor, ``[n]`` for a list, the group sizes for a nested list."""
    tensors: List[Any] = []
    structure: List[Tuple[int, List[int]]] = []
    for arg in args:
        kind = classify_argument(arg)
        if kind == SINGLE_TENSOR:
            tensors.append(arg)
            structure.append((kind, []))
        elif kind == FLAT_TENSOR_LIST:
            for t in arg:
                if not _is_tensor(t):
                    raise TypeError("Failed to extract DLManagedTensor from dlpack object")
            tensors.extend(arg)
            structure.append((kind, [len(arg)]))
        else:
            sizes = []
            for inner in arg:
                if not isinstance(inner, (list, tuple)):
                    # the reference would iterate a stray tensor's rows here (nb::sequence cast)
                    raise TypeError("Heterogeneous sequences are not supported as RPC arguments")
                for t in inner:
                    if not _is_tensor(t):
                        raise TypeError("Failed to extract DLManagedTensor from dlpack object")
                tensors.extend(inner)
                sizes.append(len(inner))
            structure.append((kind, sizes))
    return tensors, structure


def encode_structure(structure: Sequence[Tuple[int, Sequence[int]]]) -> bytes:
    """``"AXAG" | u32 n_args | per argument: u8 kind, u32 n_counts, u32 counts[]`` (little-endian)."""
    out = [_ARGS_MAGIC, struct.pack("<I", len(structure))]
    for kind, counts in structure:
        out.append(struct.pack(f"<BI{len(counts)}I", kind, len(counts), *counts))
    return b"".join(out)


def decode_structure(header: bytes) -> Tuple[List[Tuple[int, List[int]]], bytes]:
    """The argument structure in front of a bundle header and the bundle header itself.
    A bare bundle header (what ``send_tensors`` sends) reads as one list argument."""
    if header[:4] != _ARGS_MAGIC:
        return [], header
    try:
        (n,), at = struct.unpack_from("<I", header, 4), 8
        structure = []
        for _ in range(n):
            kind, k = struct.unpack_from("<BI", header, at)
            at += 5
            if kind not in (SINGLE_TENSOR, FLAT_TENSOR_LIST, NESTED_TENSOR_LIST) or \
                    (kind == SINGLE_TENSOR) != (k == 0) or (kind == FLAT_TENSOR_LIST and k != 1):
                raise ValueError("malformed argument structure")
            structure.append((kind, list(struct.unpack_from(f"<{k}I", header, at))))
            at += 4 * k
    except struct.error as exc:
        raise ValueError("truncated argument structure") from exc
    return structure, header[at:]


def regroup(structure: Sequence[Tuple[int, Sequence[int]]], tensors: Sequence[Any]) -> List[Any]:
    """Inverse of ``flatten_arguments`` on the receiver's tensors."""
    args: List[Any] = []
    at = 0

    def take(n):
        nonlocal at
        if at + n > len(tensors):
            raise RuntimeError("Not enough tensors for nested tensor list")   # bindings_runtime_wrapper.cpp:199-204
        out = list(tensors[at:at + n])
        at += n
        return out
    for kind, counts in structure:
        if kind == SINGLE_TENSOR:
            args.append(take(1)[0])
        elif kind == FLAT_TENSOR_LIST:
            args.append(take(counts[0]))
        else:
            args.append([take(n) for n in counts])
    if at != len(tensors):
        raise RuntimeError("argument structure does not account for every tensor")
    return args


def send_arguments(ctx: LoopbackAmContext, conn_id: int, args: Sequence[Any], align: int = 256,
                   stream=None, pool: Optional[DevicePool] = None) -> Tuple[int, PackedBundle]:
    """``send_tensors`` for a mixed argument list: every tensor of every argument goes
    into ONE packed payload, the nesting into the AM header."""
    tensors, structure = flatten_arguments(args)
    bundle = pack_bundle(tensors, align=align, pool=pool, stream=stream)
    _capi.check(_capi.load().axr_stream_synchronize(_stream_handle(stream)))
    request = ctx.send(conn_id, encode_structure(structure) + bundle.header, bundle.payload.data,
                       bundle.payload_bytes, ROCM, bundle.mem_h, stream, keep=bundle)
    return request, bundle


def recv_arguments(ctx: LoopbackAmContext,
                   memory_policy: Optional[Callable[[List[TensorMeta]], Any]] = None,
                   from_dlpack_fn: Optional[Callable[[Any], Any]] = None, stream=None,
                   pool: Optional[DevicePool] = None) -> Optional[List[Any]]:
    """Receive the next bundle and rebuild the sender's arguments, or None when no
    message is queued.  ``memory_policy`` sees the flat list of metas, as in the reference."""
    msg = ctx.recv_header()
    if msg is None:
        return None
    structure, bundle_header = decode_structure(msg.header)
    tensors = _receive(ctx, msg, bundle_header, memory_policy, from_dlpack_fn, stream, pool)
    if not structure:
        return [tensors]
    return regroup(structure, tensors)
