"""CPU oracle of the tensor-bundle path: Python face of ``bundle_oracle.c``.

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the product package never imports
it.  ``liborc.so`` is the plain-C restatement; ``_ref/libref_oracle.so`` (when
built) is the reference's own C++ behind ``ref_driver.cpp``.

The bundle header codec below is a second, independent implementation of the
build's own wire format (the reference's header is cista-serialised by a
third-party library that is not vendored: cista v0.15, fetched by
third_party/cista/repositories.bzl:5-7; its byte layout has no fixture in the
reference, so header parity with the reference is UNPINNED and the build
defines its own format carrying the TensorMeta fields of
rpc_core/utils/tensor_meta.hpp:77-82).
"""
from __future__ import annotations

import ctypes as C
import os
import struct
import subprocess
from typing import List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBORC = os.path.join(_HERE, "liborc.so")
LIBREF = os.path.join(_HERE, "_ref", "libref_oracle.so")

_orc = None
_ref = None


def build(force: bool = False) -> None:
    """Compile liborc.so (and _ref/ when the reference tree is mounted)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def lib() -> C.CDLL:
    global _orc
    if _orc is None:
        if not os.path.exists(LIBORC):
            build()
        L = C.CDLL(LIBORC)
        L.orc_tensor_nbytes.restype = C.c_uint64
        L.orc_tensor_nbytes.argtypes = [C.c_int32, C.POINTER(C.c_int64), C.c_uint8]
        L.orc_layout.restype = C.c_uint64
        L.orc_layout.argtypes = [C.POINTER(C.c_uint64), C.c_size_t, C.c_uint64, C.POINTER(C.c_uint64)]
        L.orc_pack.restype = C.c_int
        L.orc_pack.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                               C.c_size_t, C.c_void_p, C.c_uint64]
        L.orc_unpack.restype = C.c_int
        L.orc_unpack.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                 C.c_size_t, C.POINTER(C.c_void_p)]
        L.orc_split.restype = C.c_int
        L.orc_split.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64), C.c_size_t,
                                C.POINTER(C.c_void_p)]
        for fn in (L.orc_gather_strided, L.orc_scatter_strided):
            fn.restype = None
            fn.argtypes = [C.c_void_p, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                           C.c_uint64, C.c_void_p]
        L.orc_divide_by_two.restype = None
        L.orc_divide_by_two.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_checksum.restype = C.c_uint64
        L.orc_checksum.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        L.orc_time_pack_unpack.restype = C.c_double
        L.orc_time_pack_unpack.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                           C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.c_size_t,
                                           C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_int]
        _orc = L
    return _orc


def ref_lib() -> Optional[C.CDLL]:
    """The compiled reference, or None where it was never built."""
    global _ref
    if _ref is None and os.path.exists(LIBREF):
        L = C.CDLL(LIBREF)
        L.ref_pack.restype = None
        L.ref_pack.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.c_size_t, C.c_void_p]
        L.ref_unpack.restype = None
        L.ref_unpack.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.c_size_t, C.POINTER(C.c_void_p)]
        L.ref_split.restype = C.c_int
        L.ref_split.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64), C.c_size_t,
                                C.POINTER(C.c_void_p), C.POINTER(C.c_uint64)]
        L.ref_time_pack_unpack.restype = C.c_double
        L.ref_time_pack_unpack.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                           C.POINTER(C.c_uint64), C.c_size_t, C.c_void_p,
                                           C.c_int, C.c_int]
        if hasattr(L, "ref_release_count"):
            L.ref_release_count.restype = C.c_int
            L.ref_release_count.argtypes = [C.c_int]
        _ref = L
    return _ref


# ---------------------------------------------------------------- helpers

def _u64(values: Sequence[int]):
    return (C.c_uint64 * max(len(values), 1))(*values)


def _ptrs(arrays: Sequence[np.ndarray]):
    return (C.c_void_p * max(len(arrays), 1))(*[a.ctypes.data for a in arrays])


def _as_bytes(a: np.ndarray) -> np.ndarray:
    """Flat uint8 view of a C-contiguous array."""
    a = np.ascontiguousarray(a)
    return a.reshape(-1).view(np.uint8) if a.size else np.zeros(0, np.uint8)


def tensor_nbytes(shape: Sequence[int], bits: int) -> int:
    sh = (C.c_int64 * max(len(shape), 1))(*shape)
    return lib().orc_tensor_nbytes(len(shape), sh, bits)


def layout(sizes: Sequence[int], align: int = 1) -> Tuple[List[int], int]:
    n = len(sizes)
    offs = (C.c_uint64 * max(n, 1))()
    total = lib().orc_layout(_u64(sizes), n, align, offs)
    return list(offs[:n]), total


def pack(chunks: Sequence[np.ndarray], align: int = 1) -> np.ndarray:
    """Packed payload of C-contiguous byte chunks (uint8 arrays)."""
    chunks = [np.ascontiguousarray(c, dtype=np.uint8) for c in chunks]
    sizes = [c.size for c in chunks]
    offs, total = layout(sizes, align)
    out = np.full(total, 0xA5, np.uint8)   # poison: the oracle must write every byte
    rc = lib().orc_pack(_ptrs(chunks), _u64(sizes), _u64(offs), len(chunks),
                        out.ctypes.data if total else None, total)
    if rc != 0:
        raise ValueError("orc_pack rejected the layout")
    return out


def unpack(payload: np.ndarray, sizes: Sequence[int], align: int = 1) -> List[np.ndarray]:
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    offs, total = layout(sizes, align)
    outs = [np.empty(s, np.uint8) for s in sizes]
    rc = lib().orc_unpack(payload.ctypes.data if payload.size else None, payload.size, _u64(sizes),
                          _u64(offs), len(sizes), _ptrs(outs))
    if rc != 0:
        raise ValueError("payload is smaller than the layout")
    return outs


def split(payload: np.ndarray, sizes: Sequence[int]) -> List[int]:
    """Offsets of the to_buffer_vec views relative to the payload start."""
    views = (C.c_void_p * max(len(sizes), 1))()
    base = payload.ctypes.data
    rc = lib().orc_split(base, payload.size, _u64(sizes), len(sizes), views)
    if rc != 0:
        raise OverflowError("Total size of chunks exceeds buffer size")
    return [(views[i] or base) - base for i in range(len(sizes))]


def gather_strided(storage: np.ndarray, byte_start: int, shape: Sequence[int],
                   strides: Sequence[int], itemsize: int) -> np.ndarray:
    """C-order bytes of the view (strides in elements) over ``storage`` bytes."""
    storage = np.ascontiguousarray(storage, dtype=np.uint8)
    n = 0 if len(shape) == 0 else int(np.prod(shape, dtype=np.int64)) * itemsize
    out = np.empty(n, np.uint8)
    nd = len(shape)
    sh = (C.c_int64 * max(nd, 1))(*shape)
    st = (C.c_int64 * max(nd, 1))(*strides)
    lib().orc_gather_strided(storage.ctypes.data + byte_start, nd, sh, st, itemsize, out.ctypes.data)
    return out


def scatter_strided(flat: np.ndarray, storage: np.ndarray, byte_start: int, shape: Sequence[int],
                    strides: Sequence[int], itemsize: int) -> None:
    """Inverse of gather_strided; writes into ``storage`` in place."""
    flat = np.ascontiguousarray(flat, dtype=np.uint8)
    assert storage.dtype == np.uint8 and storage.flags.c_contiguous
    nd = len(shape)
    sh = (C.c_int64 * max(nd, 1))(*shape)
    st = (C.c_int64 * max(nd, 1))(*strides)
    lib().orc_scatter_strided(flat.ctypes.data, nd, sh, st, itemsize, storage.ctypes.data + byte_start)


def divide_by_two(values: np.ndarray) -> np.ndarray:
    out = np.array(values, dtype=np.float32, copy=True)
    lib().orc_divide_by_two(out.ctypes.data, out.size)
    return out


def checksum(data: np.ndarray, start: int = 0) -> int:
    b = _as_bytes(data)
    return lib().orc_checksum(b.ctypes.data if b.size else None, b.size, start)


# ---------------------------------------------------------------- header codec

MAGIC = 0x42545841   # "AXTB"
VERSION = 1


def encode_header(tensors: Sequence[dict], align: int) -> bytes:
    """tensors: dicts with device=(type,id), dtype=(code,bits,lanes), shape."""
    sizes = [tensor_nbytes(t["shape"], t["dtype"][1]) for t in tensors]
    offs, total = layout(sizes, align)
    out = [struct.pack("<IHHIIQ", MAGIC, VERSION, 0, len(tensors), align, total)]
    for t, off, nb in zip(tensors, offs, sizes):
        out.append(struct.pack("<QQiiiBBHQ", off, nb, t["device"][0], t["device"][1],
                               len(t["shape"]), t["dtype"][0], t["dtype"][1], t["dtype"][2], 0))
        out.append(struct.pack(f"<{len(t['shape'])}q", *t["shape"]))
    return b"".join(out)


def decode_header(blob: bytes) -> Tuple[int, int, List[dict]]:
    magic, version, flags, n, align, total = struct.unpack_from("<IHHIIQ", blob, 0)
    if magic != MAGIC or version != VERSION or flags != 0:
        raise ValueError("bad bundle header")
    at = 24
    tensors = []
    for _ in range(n):
        off, nb, dt, di, nd, code, bits, lanes, bo = struct.unpack_from("<QQiiiBBHQ", blob, at)
        at += 40
        shape = struct.unpack_from(f"<{nd}q", blob, at)
        at += 8 * nd
        tensors.append({"offset": off, "nbytes": nb, "device": (dt, di), "dtype": (code, bits, lanes),
                        "shape": tuple(shape), "byte_offset": bo})
    if at != len(blob):
        raise ValueError("trailing bytes in bundle header")
    return align, total, tensors


# ---------------------------------------------------------------- argument structure

def flatten_arguments(args: Sequence, is_tensor) -> Tuple[list, List[Tuple[str, List[int]]]]:
    """Restatement of how the reference turns invoke() arguments into ONE tensor
    stream (axon/python/src/bindings_runtime_helpers.hpp): ClassifyArg (:262-330)
    decides per argument -- a tensor; a list/tuple whose first element is a tensor, or
    an empty one (flat list); a list/tuple of lists/tuples where the first non-empty
    inner one starts with a tensor (nested list) -- then add_tensor (:351-362) appends
    single tensors and the elements of flat lists in order, and add_nested_tensor_list
    (:387-414) appends every inner list's tensors in order and records one uint32
    group size per inner list, empty ones included.  Pinned by the cases of the
    reference's own test (axon/python/tests/test_numpy_rpc.py:271-298: a tuple of
    tensors is a flat list, `[[], [t]]` is a nested list although its first inner list
    is empty, `[]` is an empty flat list), by the description at :366-386 (all tensors
    of every inner list in order, one count per inner list) and by the receiver's
    regrouping loop (bindings_runtime_wrapper.cpp:183-228), which regroup_arguments
    restates: flatten followed by regroup must give the arguments back.

    Returns (tensors, [(kind, counts)]) with kind in "single" / "flat" / "nested".
    """
    tensors, structure = [], []
    for arg in args:
        if is_tensor(arg):
            tensors.append(arg)
            structure.append(("single", []))
            continue
        if not isinstance(arg, (list, tuple)):
            raise TypeError("non-tensor argument")
        if len(arg) == 0 or is_tensor(arg[0]):
            tensors.extend(arg)
            structure.append(("flat", [len(arg)]))
            continue
        found = False
        for inner in arg:                       # the scan of ClassifyArg
            if not isinstance(inner, (list, tuple)):
                raise TypeError("heterogeneous sequence")
            if len(inner) == 0:
                continue
            if not is_tensor(inner[0]):
                raise TypeError("unsupported element inside nested sequence")
            found = True
            break
        if not found:
            raise TypeError("non-tensor argument")
        sizes = []
        for inner in arg:                       # add_nested_tensor_list
            tensors.extend(inner)
            sizes.append(len(inner))
        structure.append(("nested", sizes))
    return tensors, structure


def regroup_arguments(structure: Sequence[Tuple[str, Sequence[int]]], tensors: Sequence) -> list:
    """The receiver's loop (bindings_runtime_wrapper.cpp:183-228): consume the flat
    tensor stream in order, `gsz` tensors per inner list."""
    out, at = [], 0
    for kind, counts in structure:
        if kind == "single":
            out.append(tensors[at])
            at += 1
        elif kind == "flat":
            out.append(list(tensors[at:at + counts[0]]))
            at += counts[0]
        else:
            outer = []
            for gsz in counts:
                outer.append(list(tensors[at:at + gsz]))
                at += gsz
            out.append(outer)
    return out


def encode_argument_structure(structure: Sequence[Tuple[str, Sequence[int]]]) -> bytes:
    """Independent writer of the build's own framing of that structure (the reference
    carries the group sizes as a cista VECTOR_UINT32 header parameter, unpinned like the
    rest of its header): "AXAG", u32 argument count, then per argument u8 kind (1 single,
    2 flat, 3 nested), u32 number of counts, the counts as u32 -- little-endian."""
    code = {"single": 1, "flat": 2, "nested": 3}
    blob = bytearray(b"AXAG")
    blob += len(structure).to_bytes(4, "little")
    for kind, counts in structure:
        blob.append(code[kind])
        blob += len(counts).to_bytes(4, "little")
        for c in counts:
            blob += int(c).to_bytes(4, "little")
    return bytes(blob)


# ---------------------------------------------------------------- CPU timing

def time_pack_unpack(chunks: Sequence[np.ndarray], align: int = 1, threads: int = 1,
                     warmup: int = 3, reps: int = 20, use_reference: bool = True) -> dict:
    """Median seconds of pack + unpack on the host.

    ``use_reference`` and threads == 1 and align == 1: timed through the
    compiled reference (DefaultUcxMemoryResourceManager::memcpy) when
    ``_ref/libref_oracle.so`` exists -> kind "reference"; otherwise the C port.
    """
    chunks = [np.ascontiguousarray(c, dtype=np.uint8) for c in chunks]
    sizes = [c.size for c in chunks]
    offs, total = layout(sizes, align)
    packed = np.empty(max(total, 1), np.uint8)
    dsts = [np.empty(max(s, 1), np.uint8) for s in sizes]
    r = ref_lib() if (use_reference and threads == 1 and align == 1) else None
    if r is not None:
        sec = r.ref_time_pack_unpack(_ptrs(chunks), _ptrs(dsts), _u64(sizes), len(chunks),
                                     packed.ctypes.data, warmup, reps)
        kind = "reference"
    else:
        sec = lib().orc_time_pack_unpack(_ptrs(chunks), _ptrs(dsts), _u64(sizes), _u64(offs),
                                         len(chunks), packed.ctypes.data, total, threads, warmup, reps)
        kind = "port"
    for c, d in zip(chunks, dsts):
        if c.size and not np.array_equal(c, d[:c.size]):
            raise AssertionError("CPU baseline round trip corrupted data")
    return {"seconds": sec, "kind": kind, "threads": threads, "data_bytes": int(sum(sizes))}
