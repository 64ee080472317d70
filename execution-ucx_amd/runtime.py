"""``AxonRuntime`` as far as the tensor-bundle path reaches: the reference's Python entry
point (axon/python/src/bindings_runtime.cpp:100-260 the constructor and start/stop,
:700-830 ``register_function``, :910-1016 ``invoke``) with the same names, argument meaning
and error behaviour, over the in-process loopback context.

What it is: the caller either side of pack and unpack.  ``invoke`` classifies the arguments,
packs every tensor of every argument into ONE payload, sends it as one active message, the
serving runtime receives it through the registered function's memory policy (or as views
converted by ``from_dlpack_fn``), runs the handler, and the result travels back the same
way into the caller's memory policy.  The policy's own tensor objects are what the handler
and the caller get (axon/python/src/memory_policy_helpers.cpp:44-140).  Non-tensor
arguments (None, bool, int, float, str, and lists of bool / int / float / str or lists of lists of
bool / int / float, classified and typed as the reference does it) travel in the request record.

What it is not: the RPC runtime.  There is no dispatcher, no hybrid logical clock, no
session or workflow bookkeeping, no thread pool and no network: peers are runtimes of the
same process, found by the address ``get_local_address`` returns, and a request is served
inside the ``invoke`` that sent it (handlers may be coroutines; they are awaited there; a
serving runtime takes one request at a time, concurrent calls to it queue up).
``thread_pool_size``, ``timeout`` and ``lifecycle_policy`` are accepted and kept, nothing
acts on them.  A handler's exception reaches the caller as ``RuntimeError``, an unknown
function or worker likewise, as the reference reports them on the future.
"""
from __future__ import annotations

import asyncio
import contextlib
import inspect
import json
import struct
import threading
import uuid
import weakref
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

from . import _capi
from .bundle import _stream_handle, pack_bundle
from .device import Device, RocmDevice, auto_detect
from .loopback import LoopbackAmContext
from .memory import ROCM, DevicePool
from .transfer import (_is_tensor, _receive, decode_structure, encode_structure, flatten_arguments,
                       regroup)

_ADDRESS_MAGIC = b"axr-loopback\0"
_RECORD_MAGIC = b"AXRQ"
_PLAIN = (type(None), bool, int, float, str)

_workers: "weakref.WeakValueDictionary[bytes, AxonRuntime]" = weakref.WeakValueDictionary()
_workers_mu = threading.Lock()


class _Function:
    __slots__ = ("callable", "function_id", "name", "memory_policy", "lifecycle_policy", "from_dlpack_fn")

    def __init__(self, fn, function_id, name, memory_policy, lifecycle_policy, from_dlpack_fn):
        self.callable, self.function_id, self.name = fn, function_id, name
        self.memory_policy, self.lifecycle_policy, self.from_dlpack_fn = memory_policy, lifecycle_policy, from_dlpack_fn


def _holds_plain_values(arg: Sequence[Any]) -> bool:
    """ClassifyArg for a list or tuple (bindings_runtime_helpers.hpp:262-330): True when the
    reference would send it as a non-tensor parameter, False for a (nested) list of tensors.
    An empty sequence counts as an empty list of tensors."""
    if len(arg) == 0 or _is_tensor(arg[0]):
        return False
    if not isinstance(arg[0], (list, tuple)):
        return True
    for inner in arg:
        if not isinstance(inner, (list, tuple)):
            raise TypeError("Heterogeneous sequences are not supported as RPC arguments: expected all "
                            "elements to be sequences (list/tuple) for List[List[Tensor]]")
        if len(inner) == 0:
            continue
        if _is_tensor(inner[0]):
            return False
        if isinstance(inner[0], (bool, int, float, str)):
            return True
        raise TypeError("Unsupported element type inside nested sequence: expected a DLPack-compatible "
                        "tensor, int, float, bool, or str for List[List[T]] argument")
    return True


def _element_cast(first: Any, nested: bool) -> Callable[[Any], Any]:
    """The element type a list takes from its first element (param_conversion.cpp:381-408; nested
    lists hold bool, int or float only, :435-446) as a function that admits an element."""
    def exactly(kind, name):
        def cast(x):
            if not isinstance(x, kind):
                raise RuntimeError(f"list element {x!r} is not {name}")
            return x
        return cast

    def as_int(x):
        if not isinstance(x, int):
            raise RuntimeError(f"list element {x!r} is not an int")
        return int(x)

    def as_float(x):
        if isinstance(x, bool) or not isinstance(x, (int, float)):
            raise RuntimeError(f"list element {x!r} is not a float")
        return float(x)

    if isinstance(first, bool):
        return exactly(bool, "a bool")
    if isinstance(first, int):
        return as_int
    if isinstance(first, float):
        return as_float
    if isinstance(first, str) and not nested:
        return exactly(str, "a str")
    if nested:
        raise RuntimeError(f"EncodeNestedListToParamMeta: unsupported element type '{type(first)}'. "
                           "List[List[...]] only supports int, float, bool elements.")
    raise RuntimeError("Unsupported list element type for inference")


def _plain_sequence(arg: Sequence[Any]) -> List[Any]:
    """A list or tuple of plain values as the reference's parameter inference admits it
    (InferParamMeta, param_conversion.cpp:369-409: one element type per list, taken from the
    first element; EncodeNestedListToParamMeta, :419-457: from the first element of the first
    inner list that has one).  Arrives as lists."""
    if isinstance(arg[0], (list, tuple)):
        first = next((inner[0] for inner in arg if len(inner)), None)
        if first is None:
            raise RuntimeError("cannot infer element type from List[List[...]] when all inner lists are empty")
        cast = _element_cast(first, nested=True)
        if not all(isinstance(inner, (list, tuple)) for inner in arg):
            raise TypeError("Heterogeneous sequences are not supported as RPC arguments: expected all "
                            "elements to be sequences (list/tuple)")
        return [[cast(x) for x in inner] for inner in arg]
    cast = _element_cast(arg[0], nested=False)
    return [cast(x) for x in arg]


def _split_arguments(args: Sequence[Any]) -> Tuple[List[Any], List[Any]]:
    """Tensor arguments (to be flattened into the bundle) and, per argument, either the
    marker "t" or {"v": plain value}."""
    tensor_args, slots = [], []
    for arg in args:
        if isinstance(arg, _PLAIN):
            slots.append({"v": arg})
        elif _is_tensor(arg):
            tensor_args.append(arg)
            slots.append("t")
        elif isinstance(arg, (list, tuple)):
            if _holds_plain_values(arg):
                slots.append({"v": _plain_sequence(arg)})
            else:
                tensor_args.append(arg)
                slots.append("t")
        else:
            raise RuntimeError(f"Unsupported type for inference: {type(arg)}")     # param_conversion.cpp:410-414
    return tensor_args, slots


def _merge_arguments(slots: Sequence[Any], tensor_args: Sequence[Any]) -> List[Any]:
    it = iter(tensor_args)
    return [next(it) if s == "t" else s["v"] for s in slots]


def _frame(record: dict, rest: bytes) -> bytes:
    blob = json.dumps(record, separators=(",", ":")).encode()
    return _RECORD_MAGIC + struct.pack("<I", len(blob)) + blob + rest


def _unframe(header: bytes) -> Tuple[dict, bytes]:
    if header[:4] != _RECORD_MAGIC or len(header) < 8:
        raise RuntimeError("not a request or reply record")
    (n,) = struct.unpack_from("<I", header, 4)
    return json.loads(header[8:8 + n].decode()), header[8 + n:]


def _timeout_milliseconds(timeout: Any) -> int:
    """ConvertTimeout (axon/python/src/bindings_runtime_helpers.cpp:253-276): None is 300 ms, an
    int is milliseconds, a float is seconds, a timedelta is itself; anything else is refused."""
    import datetime
    if timeout is None:
        return 300
    if isinstance(timeout, bool):
        return int(timeout)
    if isinstance(timeout, int):
        return timeout
    if isinstance(timeout, float):
        return int(timeout * 1000.0)
    if isinstance(timeout, datetime.timedelta):
        return int(timeout.total_seconds() * 1000.0)
    raise RuntimeError("timeout must be int (milliseconds), float (seconds), or timedelta")


class AxonRuntime:
    def __init__(self, worker_name: str, thread_pool_size: int = 4, timeout: Any = None,
                 device: Optional[Device] = None, resource_manager: Any = None):
        if not worker_name:
            raise ValueError("worker_name must not be empty")
        self.worker_name = worker_name
        self.thread_pool_size = thread_pool_size
        self.timeout = timeout
        self.timeout_ms = _timeout_milliseconds(timeout)    # kept; in-process calls wait for nothing
        self.device = device if device is not None else auto_detect()
        self.resource_manager = resource_manager
        self._pool: Optional[DevicePool] = getattr(resource_manager, "pool", None)
        self._ctx: Optional[LoopbackAmContext] = None
        self._address = _ADDRESS_MAGIC + worker_name.encode() + b"\0" + uuid.uuid4().bytes
        self._functions_by_name: Dict[str, _Function] = {}
        self._functions_by_id: Dict[int, _Function] = {}
        self._peers: Dict[str, Tuple["AxonRuntime", int, int]] = {}   # name -> (peer, conn to it, conn back)
        self._next_function_id = 1
        self._next_request_id = 1
        self._serving = False
        self._serve_locks: "weakref.WeakKeyDictionary" = weakref.WeakKeyDictionary()   # one per event loop
        self._stash: Dict[int, tuple] = {}      # replies taken off the queue by another call, by request id

    # ------------------------------------------------------------------ lifecycle
    def _activate(self):
        return self.device.activate() if isinstance(self.device, RocmDevice) else contextlib.nullcontext()

    def _start(self, serving: bool) -> None:
        if self._ctx is None:
            with self._activate():
                self._ctx = LoopbackAmContext(self.worker_name)
            with _workers_mu:
                _workers[self._address] = self
        self._serving = self._serving or serving

    def start(self) -> None:
        """Server and client halves."""
        self._start(True)

    def start_server(self) -> None:
        self._start(True)

    def start_client(self) -> None:
        self._start(False)

    def stop(self) -> None:
        with _workers_mu:
            _workers.pop(self._address, None)
        self._peers.clear()
        self._stash.clear()
        self._serving = False
        if self._ctx is not None:
            self._ctx.close()
            self._ctx = None

    stop_server = stop
    stop_client = stop

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.stop()

    def get_local_address(self) -> bytes:
        if self._ctx is None:
            raise RuntimeError("the runtime has not been started")
        return self._address

    def get_local_signatures(self) -> bytes:
        """Names and ids of the registered functions (the reference serialises full
        signatures; only what ``invoke`` needs to find a function is kept here)."""
        return json.dumps({f.name: f.function_id for f in self._functions_by_id.values()}).encode()

    async def connect_endpoint_async(self, ucp_address: bytes, worker_name: str) -> int:
        if self._ctx is None:
            raise RuntimeError("the runtime has not been started")
        address = bytes(ucp_address)
        with _workers_mu:
            peer = _workers.get(address)
        if peer is None or peer._ctx is None or not address.startswith(_ADDRESS_MAGIC):
            raise RuntimeError(f"no worker at this address in this process (worker_name={worker_name!r}): "
                               "only in-process loopback peers can be reached, there is no UCX here")
        conn = self._ctx.connect(peer._ctx)
        back = peer._ctx.connect(self._ctx)
        self._peers[worker_name] = (peer, conn, back)
        return conn

    # ------------------------------------------------------------------ functions
    def register_function(self, callable: Callable, function_id: Optional[int] = None,   # noqa: A002
                          function_name: Optional[str] = None, memory_policy: Optional[Callable] = None,
                          lifecycle_policy: Any = None, from_dlpack_fn: Optional[Callable] = None) -> int:
        """Register ``callable`` under ``function_name`` (default: its ``__name__``) and
        ``function_id`` (default: the next free id).  ``memory_policy`` receives the request's
        tensors (rendezvous path), ``from_dlpack_fn`` converts them otherwise."""
        if not hasattr(callable, "__call__"):
            raise TypeError("callable must be callable")
        name = function_name or getattr(callable, "__name__", None)
        if not name:
            raise ValueError("function_name is required for a callable without a __name__")
        if function_id is None:
            while self._next_function_id in self._functions_by_id:
                self._next_function_id += 1
            function_id = self._next_function_id
        function_id = int(function_id)
        if function_id in self._functions_by_id:
            raise RuntimeError(f"function id {function_id} is already registered")
        if name in self._functions_by_name:
            raise RuntimeError(f"function name {name!r} is already registered")
        f = _Function(callable, function_id, name, memory_policy, lifecycle_policy, from_dlpack_fn)
        self._functions_by_id[function_id] = f
        self._functions_by_name[name] = f
        return function_id

    # ------------------------------------------------------------------ the path
    def _send(self, conn: int, record: dict, values: Sequence[Any], stream=None):
        """One active message: the record, the argument structure and the bundle header in the
        AM header, every tensor of ``values`` in one packed payload."""
        tensor_args, slots = _split_arguments(values)
        record = dict(record, slots=slots)
        tensors, structure = flatten_arguments(tensor_args) if tensor_args else ([], [])
        if not tensors:
            request = self._ctx.send(conn, _frame(record, encode_structure(structure)))
            return request, None
        bundle = pack_bundle(tensors, align=256, pool=self._pool, stream=stream)
        _capi.check(_capi.load().axr_stream_synchronize(_stream_handle(stream)))
        header = _frame(record, encode_structure(structure) + bundle.header)
        request = self._ctx.send(conn, header, bundle.payload.data, bundle.payload_bytes, ROCM,
                                 bundle.mem_h, stream, keep=bundle)
        return request, bundle

    def _take(self):
        """The next message and its record (the record is in the AM header, which arrives
        before the payload is placed: the serving side reads the function's name from it to
        choose the memory policy)."""
        msg = self._ctx.recv_header()
        if msg is None:
            raise RuntimeError("no message queued")
        try:
            record, rest = _unframe(msg.header)
        except Exception:
            self._ctx.release(msg)
            raise
        return msg, record, rest

    def _open(self, msg, record, rest, memory_policy, from_dlpack_fn, stream=None) -> List[Any]:
        structure, bundle_header = decode_structure(rest)
        if not bundle_header:                   # no tensor anywhere: empty lists keep their shape
            return _merge_arguments(record["slots"], regroup(structure, []))
        # the memory policy serves rendezvous payloads only; an eager payload is already in
        # host memory when the header arrives and bypasses it (axon_worker.cpp:1150-1172)
        policy = memory_policy if msg.is_rndv else None
        try:
            tensors = _receive(self._ctx, msg, bundle_header, policy, from_dlpack_fn, stream, self._pool)
        except Exception:
            self._ctx.release(msg)          # an unfetched rendezvous fails at its sender
            raise
        return _merge_arguments(record["slots"], regroup(structure, tensors))

    def _serve_lock(self) -> asyncio.Lock:
        loop = asyncio.get_running_loop()
        lock = self._serve_locks.get(loop)
        if lock is None:
            lock = self._serve_locks[loop] = asyncio.Lock()
        return lock

    async def _serve_one(self, back: int):
        """Receive one request, run its function, send the reply on ``back``; returns the
        reply's send (request handle, bundle) for the caller to finish."""
        msg, record, rest = self._take()
        reply = {"kind": "reply", "id": record.get("id")}
        fn = self._lookup(record.get("function"))
        try:
            if fn is None:
                self._ctx.release(msg)
                raise LookupError(f"function {record.get('function')!r} is not registered with "
                                  f"worker {self.worker_name!r}")
            with self._activate():
                args = self._open(msg, record, rest, fn.memory_policy, fn.from_dlpack_fn)
                result = fn.callable(*args)
            if inspect.isawaitable(result):     # awaited outside the activation: the device that is
                result = await result           # current on this thread is not held across a suspension
            values = list(result) if isinstance(result, tuple) else [result]
            with self._activate():
                return self._send(back, dict(reply, tuple=isinstance(result, tuple)), values)
        except Exception as e:  # noqa: BLE001  (a handler's failure is the caller's RuntimeError)
            return self._send(back, dict(reply, kind="error", error=f"{type(e).__name__}: {e}"), [])

    def _lookup(self, function: Any) -> Optional[_Function]:
        if isinstance(function, int) and not isinstance(function, bool):
            return self._functions_by_id.get(function)
        return self._functions_by_name.get(function)

    def _finish(self, sent, tolerate_failure: bool = False) -> None:
        request, bundle = sent
        try:
            if self._ctx is not None and not self._ctx.test(request):
                # nobody fetched the payload: withdraw the message before its memory goes back
                self._ctx.cancel(request)
                raise _capi.AxonRocmError(_capi.AXR_ERR_CANCELED, "the peer did not fetch the payload")
        except _capi.AxonRocmError:
            if not tolerate_failure:
                raise
        finally:
            if bundle is not None:
                bundle.close()

    async def invoke(self, *args, worker_name: str, session_id: int, function: Any, workflow_id: int = 0,
                     memory_policy: Optional[Callable] = None, from_dlpack_fn: Optional[Callable] = None):
        """Call ``function`` (a name or an id) of worker ``worker_name`` with ``args``.  Returns
        what the function returned: tensors arrive in the objects ``memory_policy`` creates
        (rendezvous replies) or converted by ``from_dlpack_fn``."""
        if self._ctx is None:
            raise RuntimeError("the runtime has not been started")
        if worker_name not in self._peers:
            raise RuntimeError(f"not connected to worker {worker_name!r}")
        peer, conn, back = self._peers[worker_name]
        if peer._ctx is None or not peer._serving:
            raise RuntimeError(f"worker {worker_name!r} is not serving")
        request_id, self._next_request_id = self._next_request_id, self._next_request_id + 1
        record = {"kind": "request", "id": request_id, "function": function, "session": int(session_id),
                  "workflow": int(workflow_id)}
        # one request at a time per serving runtime: the request is sent, served and answered
        # under the server's lock, so the message the server takes is this one
        async with peer._serve_lock():
            with self._activate():
                sent = self._send(conn, record, list(args))
            try:
                pending = await peer._serve_one(back)
            except BaseException:                   # the server could not even answer (or the call
                self._finish(sent, tolerate_failure=True)   # was cancelled): the request's bundle
                raise                                       # goes back to its pool all the same
        try:
            with self._activate():
                msg, reply, rest = self._take_reply(request_id)
                failed = reply.get("kind") == "error"
                self._finish(sent, tolerate_failure=failed)     # a refused request was never fetched
                values = self._open(msg, reply, rest, memory_policy, from_dlpack_fn)
        finally:
            peer._finish(pending, tolerate_failure=True)
        if failed:
            raise RuntimeError(reply.get("error", "remote error"))
        return tuple(values) if reply.get("tuple") else values[0]

    def _take_reply(self, request_id: int):
        """The reply to ``request_id``: replies to other calls of this runtime that are still
        suspended (calls to several servers run concurrently) are set aside for them."""
        while True:
            if request_id in self._stash:
                return self._stash.pop(request_id)
            msg, record, rest = self._take()
            if record.get("id") == request_id:
                return msg, record, rest
            self._stash[record.get("id")] = (msg, record, rest)
