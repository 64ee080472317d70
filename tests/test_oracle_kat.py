"""Pins the CPU oracle: the reference's own known-answer tests, the compiled
reference (oracle/_ref, when built) and what the mathematics fixes."""
import ctypes as C
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def pattern(n, start=0):
    """byte = running index % 256, the fill used throughout the reference tests
    (ucx_am_connection_test.cpp:949-952, ucx_am_context_test.cpp:286-291)."""
    return ((np.arange(n, dtype=np.uint64) + start) % 256).astype(np.uint8)


# ---- size rule: rpc_core/utils/tensor_meta.hpp:91-104 -----------------------

@pytest.mark.parametrize("shape,bits,expect", [
    ((1024,), 32, 4096),              # fp32[1024]   axon_worker_test.cpp:1241-1250
    ((512,), 32, 2048),               # int32[512]   :1329-1347
    ((256,), 32, 1024),               # int32[256]
    ((5 * 1024 * 1024 // 4,), 32, 5 * 1024 * 1024),   # 5 MiB fp32  :1448-1472
    ((3 * 1024 * 1024 // 4,), 32, 3 * 1024 * 1024),
    ((), 32, 0),                      # ndim == 0 -> 0 bytes
    ((3, 5, 7), 16, 210),
    ((10,), 4, 10),                   # sub-byte types round up to one byte
    ((10,), 12, 20),
    ((2, 0, 4), 64, 0),
    ((7,), 64, 56),
    ((9,), 8, 9),
])
def test_nbytes_rule(orc, shape, bits, expect):
    assert orc.tensor_nbytes(shape, bits) == expect


# ---- split: ucx_context/ucx_context_data_test.cpp:41-83 ---------------------

def test_split_kat(orc):
    buf = np.arange(100, dtype=np.uint8)            # std::iota
    offs = orc.split(buf, [10, 20, 30, 40])
    assert offs == [0, 10, 30, 60]
    for off, n in zip(offs, [10, 20, 30, 40]):
        assert np.array_equal(buf[off:off + n], np.arange(off, off + n, dtype=np.uint8))


def test_split_overflow_kat(orc):
    with pytest.raises(OverflowError):
        orc.split(np.zeros(100, np.uint8), [50, 51])


def test_split_matches_compiled_reference(orc):
    ref = orc.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(3)
    for trial in range(50):
        n = int(rng.integers(0, 12))
        sizes = [int(x) for x in rng.integers(0, 500, size=n)]
        slack = int(rng.integers(-3, 20))
        total = max(0, sum(sizes) + slack)
        buf = np.zeros(max(total, 1), np.uint8)
        views = (C.c_void_p * max(n, 1))()
        vs = (C.c_uint64 * max(n, 1))()
        rc = ref.ref_split(buf.ctypes.data, total, (C.c_uint64 * max(n, 1))(*sizes), n, views, vs)
        if sum(sizes) > total:
            assert rc == -1
            with pytest.raises(OverflowError):
                orc.split(buf[:total], sizes)
        else:
            assert rc == 0
            got = orc.split(buf[:total] if total else buf[:0], sizes) if n else []
            want = [(views[i] or buf.ctypes.data) - buf.ctypes.data for i in range(n)]
            assert got == want
            assert list(vs[:n]) == sizes


def test_release_function_ownership_kat(orc):
    """ucx_context_data_test.cpp:85-128 on the compiled UcxBuffer: a release callback
    moved with own_buffer=true runs exactly once, moved with own_buffer=false never."""
    ref = orc.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    assert ref.ref_release_count(1) == 1
    assert ref.ref_release_count(0) == 0


# ---- pack = ordered tight concat --------------------------------------------

@pytest.mark.parametrize("lens", [(256, 512, 300),                       # ucx_am_connection_test.cpp:933-994
                                  (512 * 1024, 256 * 1024, 800 * 1024)])   # :1051-1108
def test_iov_to_contig_kat(orc, lens):
    segs, cursor = [], 0
    for n in lens:
        segs.append(pattern(n, cursor))
        cursor += n
    expected = pattern(sum(lens))          # "expected flat": the running pattern itself
    assert np.array_equal(orc.pack(segs, align=1), expected)
    back = orc.unpack(expected, lens, align=1)     # iov -> iov, :996-1049
    for a, b in zip(segs, back):
        assert np.array_equal(a, b)


def test_four_segment_float_kat(orc):
    # ucx_am_context_test.cpp:1260-1271,1310-1314: 4 x 8192 B of float(i % 256) over the
    # global index; the contiguous receive equals the flat vector.
    per = 8192 // 4
    flat = (np.arange(4 * per) % 256).astype(np.float32)
    segs = [flat[i * per:(i + 1) * per].view(np.uint8) for i in range(4)]
    assert np.array_equal(orc.pack(segs, 1), flat.view(np.uint8))


def test_vec_to_buffer_and_back_kat(orc):
    # axon_worker_test.cpp:1547-1654: int32[1024] = i, int32[512] = i + 2000 -> one buffer
    a = np.arange(1024, dtype=np.int32)
    b = np.arange(512, dtype=np.int32) + 2000
    packed = orc.pack([a.view(np.uint8), b.view(np.uint8)], 1)
    assert packed.size == (1024 + 512) * 4
    assert np.array_equal(packed.view(np.int32), np.concatenate([a, b]))
    # :1656-1774: fp32[2048] = i split four ways, global index preserved
    f = np.arange(2048, dtype=np.float32)
    parts = orc.unpack(f.view(np.uint8), [2048] * 4, 1)
    for k, part in enumerate(parts):
        assert np.array_equal(part.view(np.float32), np.arange(512 * k, 512 * (k + 1), dtype=np.float32))


def test_pack_matches_compiled_reference(orc):
    ref = orc.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(11)
    for trial in range(20):
        n = int(rng.integers(1, 40))
        chunks = [rng.integers(0, 256, size=int(rng.integers(0, 5000)), dtype=np.uint8) for _ in range(n)]
        sizes = [c.size for c in chunks]
        total = sum(sizes)
        out = np.full(max(total, 1), 0x5A, np.uint8)
        ptrs = (C.c_void_p * n)(*[c.ctypes.data for c in chunks])
        ref.ref_pack(ptrs, (C.c_uint64 * n)(*sizes), n, out.ctypes.data)
        assert np.array_equal(orc.pack(chunks, 1), out[:total])
        dsts = [np.zeros(max(s, 1), np.uint8) for s in sizes]
        dp = (C.c_void_p * n)(*[d.ctypes.data for d in dsts])
        ref.ref_unpack(out.ctypes.data, (C.c_uint64 * n)(*sizes), n, dp)
        mine = orc.unpack(out[:total], sizes, 1)
        for d, m, s in zip(dsts, mine, sizes):
            assert np.array_equal(d[:s], m)


# ---- aligned layout: invariants (not in the reference) ----------------------

@pytest.mark.parametrize("align", [1, 2, 16, 256, 4096])
def test_aligned_layout_invariants(orc, align):
    rng = np.random.default_rng(align)
    sizes = [int(x) for x in rng.integers(0, 3000, size=60)]
    sizes[5] = 0
    sizes[-1] = 0 if align == 16 else sizes[-1]
    offs, total = orc.layout(sizes, align)
    assert offs[0] == 0
    for i in range(len(sizes)):
        assert offs[i] % align == 0
        if i + 1 < len(sizes):
            assert offs[i + 1] == -(-(offs[i] + sizes[i]) // align) * align
    assert total == offs[-1] + sizes[-1]
    chunks = [rng.integers(1, 256, size=s, dtype=np.uint8) for s in sizes]   # no zero bytes in data
    packed = orc.pack(chunks, align)
    mask = np.zeros(total, bool)
    for o, s in zip(offs, sizes):
        mask[o:o + s] = True
    assert np.array_equal(packed[mask], np.concatenate(chunks))   # gaps removed -> tight concat
    assert not packed[~mask].any()                                # gaps are zero
    if align == 1:
        assert np.array_equal(packed, np.concatenate(chunks))


# ---- strided gather / scatter: numpy is the textbook routine ----------------

def random_view(rng, ndim):
    """A random strided view (positive, negative and permuted strides) of a parent array."""
    parent_shape = tuple(int(x) for x in rng.integers(1, 7, size=ndim))
    parent = rng.integers(0, 2 ** 31, size=parent_shape, dtype=np.int64)
    view = parent
    index = []
    for d in range(ndim):
        n = parent_shape[d]
        lo = int(rng.integers(0, n))
        hi = int(rng.integers(lo + 1, n + 1))
        step = int(rng.choice([1, 1, 2, -1]))
        index.append(slice(lo, hi, step) if step > 0 else slice(hi - 1, lo - 1 if lo > 0 else None, -1))
    view = parent[tuple(index)]
    view = view.transpose(rng.permutation(ndim))
    return parent, view


@pytest.mark.parametrize("itemsize_dtype", [np.uint8, np.int16, np.float32, np.int64, np.complex128])
def test_gather_matches_numpy(orc, itemsize_dtype):
    rng = np.random.default_rng(5)
    for trial in range(40):
        ndim = int(rng.integers(1, 6))
        parent64, view64 = random_view(rng, ndim)
        parent = parent64.astype(itemsize_dtype)
        # rebuild the same view on the typed parent
        item = parent.dtype.itemsize
        start = (view64.__array_interface__["data"][0] - parent64.__array_interface__["data"][0]) // 8
        strides = [s // 8 for s in view64.strides]
        view = np.lib.stride_tricks.as_strided(parent.reshape(-1)[start:], view64.shape,
                                               [s * item for s in strides])
        storage = parent.reshape(-1).view(np.uint8)
        got = orc.gather_strided(storage, start * item, view.shape, strides, item)
        want = np.ascontiguousarray(view).reshape(-1).view(np.uint8)
        assert np.array_equal(got, want)
        # scatter(gather(x)) puts every touched element back and touches nothing else
        target = np.full(storage.size, 0xEE, np.uint8)
        orc.scatter_strided(got, target, start * item, view.shape, strides, item)
        tview = np.lib.stride_tricks.as_strided(
            target.view(itemsize_dtype)[start:], view.shape, [s * item for s in strides])
        assert np.array_equal(tview, view)
        untouched = np.ones(parent.size, bool)
        flat_index = np.lib.stride_tricks.as_strided(
            np.arange(parent.size)[start:], view.shape, [s * 8 for s in strides])
        untouched[flat_index.reshape(-1)] = False
        assert (target.view(itemsize_dtype)[untouched].view(np.uint8) == 0xEE).all()


def test_gather_kv_block_closed_form(orc):
    # run r = (layer, kv) of block b starts at ((layer*2+kv)*blocks + b) * block_bytes
    layers, blocks, be = 3, 5, 8          # tiny cache [3, 2, 5, 2, 2, 2] of 2-byte elements
    cache = np.arange(layers * 2 * blocks * be, dtype=np.uint16)
    b = 3
    got = orc.gather_strided(cache.view(np.uint8), b * be * 2, (layers, 2, 2, 2, 2),
                             (2 * blocks * be, blocks * be, 4, 2, 1), 2).view(np.uint16)
    want = np.concatenate([cache[((l * 2 + kv) * blocks + b) * be:][:be]
                           for l in range(layers) for kv in range(2)])
    assert np.array_equal(got, want)


# ---- device-side "process" step ----------------------------------------------

def test_divide_by_two_kat(orc):
    # ucx_am_context_test.cpp:321-333: received float(i % 256) comes back as (i % 256) / 2
    n = 4096
    x = (np.arange(n) % 256).astype(np.float32)
    assert np.array_equal(orc.divide_by_two(x), (np.arange(n) % 256).astype(np.float32) / 2)


# ---- checksum -----------------------------------------------------------------

def test_checksum_definition_and_additivity(orc):
    rng = np.random.default_rng(9)
    data = rng.integers(0, 256, size=200_000, dtype=np.uint8)
    start = 65500
    w = 1 + ((np.arange(data.size, dtype=np.uint64) + np.uint64(start)) % np.uint64(65521))
    brute = int((data.astype(np.uint64) * w).sum(dtype=np.uint64))   # wraps mod 2^64
    assert orc.checksum(data, start) == brute
    cut = 77_777
    assert (orc.checksum(data[:cut], start) + orc.checksum(data[cut:], start + cut)) % (1 << 64) == brute


# ---- header codec (build's own format) -----------------------------------------

def test_header_roundtrip(orc):
    tensors = [
        {"device": (10, 0), "dtype": (2, 32, 1), "shape": (16384,)},
        {"device": (10, 0), "dtype": (4, 16, 1), "shape": (3, 5)},
        {"device": (1, 0), "dtype": (0, 8, 1), "shape": ()},
        {"device": (10, 1), "dtype": (0, 8, 1), "shape": (0, 9)},
    ]
    blob = orc.encode_header(tensors, 256)
    align, total, back = orc.decode_header(blob)
    assert align == 256 and total == 65792   # trailing empty tensors sit at the next boundary
    assert [t["offset"] for t in back] == [0, 65536, 65792, 65792]
    assert [t["nbytes"] for t in back] == [65536, 30, 0, 0]
    for a, b in zip(tensors, back):
        assert a["device"] == b["device"] and a["dtype"] == b["dtype"] and tuple(a["shape"]) == b["shape"]


# ------------------------------------------------------------------ argument structure

def test_argument_classification_cases_of_the_reference(orc):
    """axon/python/tests/test_numpy_rpc.py:271-298: a tuple of tensors, a nested list
    that starts with an empty inner list, and an empty outer list."""
    t = np.ones((10,), dtype=np.float32)
    is_tensor = lambda x: isinstance(x, np.ndarray)
    assert orc.flatten_arguments([(t, t)], is_tensor)[1] == [("flat", [2])]
    flat, structure = orc.flatten_arguments([[[], [t]]], is_tensor)
    assert structure == [("nested", [0, 1])] and len(flat) == 1 and flat[0] is t
    assert orc.flatten_arguments([[]], is_tensor) == ([], [("flat", [0])])
    # flatten then regroup is the identity (lists and tuples both come back as lists)
    args = [t, [t, t], [[t], [], [t, t]], []]
    flat, structure = orc.flatten_arguments(args, is_tensor)
    assert len(flat) == 6
    back = orc.regroup_arguments(structure, flat)
    assert back[0] is t and [len(x) for x in back[2]] == [1, 0, 2] and back[3] == []


def test_argument_structure_fixture(orc):
    cases = json.load(open(os.path.join(GOLDEN, "argument_structure_v1.json")))
    assert cases[0]["flat"] == ["a", "b", "c"] and cases[0]["structure"] == [["nested", [2, 1]]]
    for c in cases:
        flat, structure = orc.flatten_arguments(c["args"], lambda x: isinstance(x, str))
        assert flat == c["flat"] and [[k, n] for k, n in structure] == c["structure"]
        assert orc.encode_argument_structure(structure).hex() == c["blob_hex"]
        assert orc.regroup_arguments(structure, flat) == c["args"]
