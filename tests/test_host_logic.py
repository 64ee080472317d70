"""Host-side logic that needs no GPU: the C-ABI library loads and exports what
the header declares, the planner agrees with the oracle, the header codec
matches the golden fixtures, the segment table is what the design says, and
every path that would need a device fails loudly instead of falling back."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def tv(pkg, ptr, shape, strides=None, dtype=(1, 8, 1), device_type=10):
    return pkg.TensorView(data=ptr, device_type=device_type, device_id=0, dtype=dtype,
                          shape=tuple(shape), strides=None if strides is None else tuple(strides))


# ------------------------------------------------------------------ the C ABI itself

def declared_functions():
    text = open(os.path.join(ROOT, "include", "axon_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"AXR_API\s+[\w\s\*]+?\b(axr_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg._capi.load()
    names = declared_functions()
    assert len(names) >= 55
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/axon_rocm.h but not exported"
    assert sorted(pkg._capi.PROTOTYPES) == names      # the ctypes binding covers the same set


def test_structs_match_dlpack_and_ucx_layouts(pkg):
    t = pkg._capi.Tensor
    assert C.sizeof(t) == 48                           # sizeof(DLTensor) on LP64
    assert (t.data.offset, t.device_type.offset, t.device_id.offset, t.ndim.offset) == (0, 8, 12, 16)
    assert (t.dtype_code.offset, t.dtype_bits.offset, t.dtype_lanes.offset) == (20, 21, 22)
    assert (t.shape.offset, t.strides.offset, t.byte_offset.offset) == (24, 32, 40)
    assert C.sizeof(pkg._capi.Buffer) == 16            # ucx_buffer_t {void*, size_t}


def test_status_and_version(pkg):
    lib = pkg._capi.load()
    assert lib.axr_version().decode().count(".") == 2
    assert lib.axr_status_string(0) == b"AXR_OK"
    assert lib.axr_status_string(-4) == b"AXR_ERR_LENGTH"
    assert lib.axr_status_string(-12345).startswith(b"AXR_ERR_")


def test_device_type_maps(pkg):
    # axon/python/src/dlpack_helpers.cpp:82-134 and ucx_context_def.h:27-39
    lib = pkg._capi.load()
    to_mem = {1: 0, 2: 1, 13: 2, 10: 3, 11: 4, 14: 9, 4: 9, 7: 9, 8: 9}
    for dl, mem in to_mem.items():
        assert lib.axr_dl_device_to_memory_type(dl) == mem
    to_dl = {0: 1, 1: 2, 2: 13, 3: 10, 4: 11, 5: 1, 6: 14, 7: 14, 8: 14, 9: 1}
    for mem, dl in to_dl.items():
        assert lib.axr_memory_type_to_dl_device(mem) == dl


def test_tunables(pkg):
    lib = pkg._capi.load()
    v = C.c_int64()
    for key, good, bad in ((b"tile_rows", 4, 3), (b"threads", 512, 100), (b"max_waves", 99, 0),
                           (b"gather_run_bytes", 64, 0), (b"max_tiles", 1000, 0),
                           (b"spin_wait_us", 150, -1)):
        before = C.c_int64()
        assert lib.axr_tune_get(key, C.byref(before)) == 0
        assert lib.axr_tune_set(key, good) == 0
        assert lib.axr_tune_get(key, C.byref(v)) == 0 and v.value == good
        assert lib.axr_tune_set(key, bad) == pkg._capi.AXR_ERR_INVALID
        assert lib.axr_tune_set(key, before.value) == 0
    assert lib.axr_tune_set(b"no_such_knob", 1) == pkg._capi.AXR_ERR_INVALID
    with pytest.raises(pkg.AxonRocmError):
        pkg.tune(no_such_knob=1)


def test_tensor_meta_reads_like_the_reference_binding(pkg):
    """axon/python/tests/test_types_enums.py:171-207: default-constructible, fields device
    (device_type, device_id as ints), ndim, dtype (code, bits, lanes), byte_offset, shape,
    strides -- what a memory policy written for the reference touches."""
    meta = pkg.TensorMeta()
    for field in ("device", "ndim", "dtype", "byte_offset", "shape", "strides"):
        assert hasattr(meta, field)
    assert meta.ndim == 0 and meta.byte_offset == 0
    assert isinstance(meta.device, pkg.DLDevice) and isinstance(meta.dtype, pkg.DLDataType)
    assert isinstance(meta.device.device_type, int) and isinstance(meta.device.device_id, int)
    assert all(hasattr(meta.dtype, f) for f in ("code", "bits", "lanes"))
    plan = pkg.BundlePlan.create([tv(pkg, 0x1000, [3, 5], dtype=(4, 16, 1))], align=64)
    m = plan.metas()[0]
    assert (m.device.device_type, m.device.device_id, m.ndim) == (10, 0, 2)
    assert (m.dtype.code, m.dtype.bits, m.dtype.lanes) == (4, 16, 1) and m.dtype == (4, 16, 1)
    assert tuple(m.shape) == (3, 5) and list(m.strides) == [] and m.byte_offset == 0
    assert np.zeros(tuple(m.shape)).shape == (3, 5)          # the way policies use it


def test_plan_create_refuses_what_it_does_not_know(pkg):
    lib = pkg._capi.load()
    arr = pkg.dlpack.TensorArray([tv(pkg, 0x1000, [16])])
    h = C.c_void_p()
    assert lib.axr_plan_create(arr.pointer(), 1, 256, 1, C.byref(h)) == pkg._capi.AXR_ERR_INVALID   # reserved flags
    assert not h.value
    assert lib.axr_plan_create(arr.pointer(), 1, 3, 0, C.byref(h)) == pkg._capi.AXR_ERR_INVALID     # alignment
    assert lib.axr_plan_create(None, 1, 256, 0, C.byref(h)) == pkg._capi.AXR_ERR_INVALID
    assert lib.axr_plan_create(arr.pointer(), 1, 256, 0, None) == pkg._capi.AXR_ERR_INVALID
    assert lib.axr_plan_create(None, 0, 256, 0, C.byref(h)) == 0 and h.value                     # an empty bundle
    assert lib.axr_plan_free(h) == 0


# ------------------------------------------------------------------ size rule and layout

def test_nbytes_rule_matches_oracle(pkg, orc):
    lib = pkg._capi.load()
    rng = np.random.default_rng(0)
    for _ in range(300):
        nd = int(rng.integers(0, 6))
        shape = [int(x) for x in rng.integers(0, 9, size=nd)]
        bits = int(rng.choice([1, 4, 8, 12, 16, 32, 64, 128]))
        arr = pkg.dlpack.TensorArray([tv(pkg, 0x1000, shape, dtype=(0, bits, 1))])
        out = C.c_uint64()
        pkg._capi.check(lib.axr_tensor_nbytes(arr.pointer(), C.byref(out)))
        assert out.value == orc.tensor_nbytes(shape, bits)
    bad = pkg.dlpack.TensorArray([tv(pkg, 0x1000, [3, -1])])
    assert lib.axr_tensor_nbytes(bad.pointer(), C.byref(out)) == pkg._capi.AXR_ERR_INVALID


@pytest.mark.parametrize("align", [1, 2, 16, 256, 4096])
def test_layout_matches_oracle(pkg, orc, align):
    rng = np.random.default_rng(align)
    for _ in range(20):
        n = int(rng.integers(0, 50))
        sizes = [int(x) for x in rng.integers(0, 5000, size=n)]
        views = [tv(pkg, 0x10000, [s]) for s in sizes]
        plan = pkg.BundlePlan.create(views, align=align)
        offs, got_sizes = plan.layout()
        want_offs, want_total = orc.layout(sizes, align)
        assert got_sizes == sizes and offs == want_offs and plan.payload_bytes == want_total
        assert plan.data_bytes == sum(sizes)
        plan.close()


@pytest.mark.parametrize("align", [0, 3, 8192])
def test_bad_alignment_rejected(pkg, align):
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0x1000, [4])], align=align)


def test_split_matches_reference_semantics(pkg, orc):
    kat = json.load(open(os.path.join(GOLDEN, "kat_patterns.json")))["split"]
    buf = np.arange(kat["buffer_bytes"], dtype=np.uint8)
    plan = pkg.BundlePlan.create([tv(pkg, 0x1000, [s]) for s in kat["sizes"]], align=1)
    views = plan.split(buf.ctypes.data, buf.size)
    assert [p - buf.ctypes.data for p, _ in views] == kat["offsets"] == orc.split(buf, kat["sizes"])
    assert [n for _, n in views] == kat["sizes"]
    over = json.load(open(os.path.join(GOLDEN, "kat_patterns.json")))["split_overflow"]
    plan2 = pkg.BundlePlan.create([tv(pkg, 0x1000, [s]) for s in over["sizes"]], align=1)
    with pytest.raises(pkg.LengthError):
        plan2.split(buf.ctypes.data, over["buffer_bytes"])


# ------------------------------------------------------------------ header

def fixture_views(pkg, tensors):
    return [tv(pkg, 0x7000_0000_0000, t["shape"], dtype=tuple(t["dtype"]), device_type=t["device"][0])
            for t in tensors]


def test_header_matches_golden_fixture_and_oracle(pkg, orc):
    fx = json.load(open(os.path.join(GOLDEN, "bundle_header_v1.json")))
    for case in fx["cases"]:
        views = fixture_views(pkg, fx["tensors"])
        for v, t in zip(views, fx["tensors"]):
            v.device_id = t["device"][1]
        plan = pkg.BundlePlan.create(views, align=case["align"])
        assert plan.header.hex() == case["header_hex"]
        align, total, tensors = orc.decode_header(plan.header)
        assert align == case["align"] and total == plan.payload_bytes
        back = pkg.BundlePlan.from_header(bytes.fromhex(case["header_hex"]))
        assert back.layout() == plan.layout() and back.payload_bytes == plan.payload_bytes
        for m, t in zip(back.metas(), fx["tensors"]):
            assert m.device == tuple(t["device"]) and m.dtype == tuple(t["dtype"])
            assert m.shape == tuple(t["shape"]) and m.byte_offset == 0
        assert back.header == plan.header


def test_malformed_headers_are_refused(pkg, orc):
    good = orc.encode_header([{"device": (10, 0), "dtype": (2, 32, 1), "shape": (100,)},
                              {"device": (10, 0), "dtype": (0, 8, 1), "shape": (7, 3)}], 256)
    pkg.BundlePlan.from_header(good)

    def broken(edit):
        b = bytearray(good)
        edit(b)
        return bytes(b)

    cases = {
        "magic": broken(lambda b: b.__setitem__(0, b[0] ^ 1)),
        "version": broken(lambda b: b.__setitem__(4, 2)),
        "flags": broken(lambda b: b.__setitem__(6, 1)),
        "align": broken(lambda b: b.__setitem__(12, 3)),
        "payload size": broken(lambda b: b.__setitem__(16, b[16] ^ 1)),
        "offset": broken(lambda b: b.__setitem__(24 + 48, 1)),      # second tensor's offset
        "nbytes": broken(lambda b: b.__setitem__(24 + 8, b[24 + 8] ^ 1)),
        "byte_offset": broken(lambda b: b.__setitem__(24 + 32, 1)),
        "ndim": broken(lambda b: b.__setitem__(24 + 24, 5)),
        "truncated": good[:-3],
        "trailing": good + b"\0",
        "short": good[:10],
    }
    for what, blob in cases.items():
        with pytest.raises(pkg.HeaderError):
            pkg.BundlePlan.from_header(blob)
            pytest.fail(f"header with bad {what} accepted")


# ------------------------------------------------------------------ segment table

def seg_of(pkg, view, align=256, **tune):
    if tune:
        pkg.tune(**tune)
    try:
        plan = pkg.BundlePlan.create([view], align=align)
        return plan.segments(), plan.launch_info()
    finally:
        if tune:
            pkg.tune(tile_rows=0, gather_run_bytes=1280, transpose=1, ragged_runs=1)


def test_compact_tensor_is_one_run(pkg):
    segs, info = seg_of(pkg, tv(pkg, 0x10000, [3, 1, 500], strides=[500, 77, 1], dtype=(2, 32, 1)))
    assert len(segs) == 1
    s = segs[0]
    assert (s["mode"], s["run_bytes"], s["nbytes"], s["ndim"]) == (0, 6000, 6000, 0)
    assert s["tiles"] == 3 and info["tile_bytes"] == 2048 and info["tiles"] == 3


def test_kv_block_view_collapses_to_64_runs(pkg):
    from execution_ucx_amd import workloads
    spec = workloads.kv_gather()
    v = workloads.kv_block_view(0x7f00_0000_0000, spec, 17)
    segs, info = seg_of(pkg, v)
    assert len(segs) == 1
    s = segs[0]
    assert s["mode"] == 1 and s["run_bytes"] == 32768 and s["nbytes"] == 64 * 32768
    assert s["shape"] == (64,) and s["stride_bytes"] == (4096 * 32768,)      # layer and K/V merge
    assert s["address"] == 0x7f00_0000_0000 + 17 * 32768


def test_pitched_view_rows(pkg):
    from execution_ucx_amd import workloads
    spec = workloads.pitched_chunk()
    v = workloads.pitched_views(0x7f00_0000_0000, spec)[1]
    segs, info = seg_of(pkg, v)
    s = segs[0]
    assert (s["mode"], s["run_bytes"], s["shape"], s["stride_bytes"]) == (1, 4096, (1024,), (6144,))
    assert s["tiles"] == 1024 and info["tile_bytes"] == 4096       # one tile per 4 KiB row
    segs, info = seg_of(pkg, v, tile_rows=2)
    assert segs[0]["tiles"] == 2048 and info["tile_bytes"] == 2048


def test_short_runs_use_element_mode(pkg):
    # transposed matrix: no contiguous inner run
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [30, 20], strides=[1, 30], dtype=(4, 16, 1)), transpose=0)
    s = segs[0]
    assert (s["mode"], s["run_bytes"], s["granule"]) == (2, 2, 2)
    assert s["shape"] == (30, 20) and s["stride_bytes"] == (2, 60)
    # 24-byte runs of fp64 -> ragged 16-byte granules (two per run, the second one
    # overlapping); 12-byte elements are shorter than a vector -> 4-byte granules
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 3], strides=[10, 1], dtype=(2, 64, 1)))
    assert (segs[0]["mode"], segs[0]["run_bytes"], segs[0]["granule"]) == (2, 24, 16)
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 3], strides=[10, 1], dtype=(2, 64, 1)), ragged_runs=0)
    assert (segs[0]["mode"], segs[0]["run_bytes"], segs[0]["granule"]) == (2, 24, 8)
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 3], strides=[7, 2], dtype=(2, 96, 1)))
    assert (segs[0]["mode"], segs[0]["run_bytes"], segs[0]["granule"]) == (2, 12, 4)
    # the threshold is a tunable
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 304], strides=[1000, 1]), gather_run_bytes=304)
    assert segs[0]["mode"] == 1
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 304], strides=[1000, 1]), gather_run_bytes=305)
    assert segs[0]["mode"] == 2 and segs[0]["granule"] == 16
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 300], strides=[1000, 1]), gather_run_bytes=300)
    assert segs[0]["mode"] == 1
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 300], strides=[1000, 1]), gather_run_bytes=301)
    assert segs[0]["mode"] == 2 and segs[0]["granule"] == 16          # ragged granules: the same limit
    assert segs[0]["lanes_per_run"] == 20                             # 19 granules in five groups of four lanes
    # without ragged granules, runs that are no multiple of 16 switch at a fifth of it
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 300], strides=[1000, 1]), gather_run_bytes=1496,
                     ragged_runs=0)
    assert segs[0]["mode"] == 1
    segs, _ = seg_of(pkg, tv(pkg, 0x10000, [5, 300], strides=[1000, 1]), gather_run_bytes=1501,
                     ragged_runs=0)
    assert segs[0]["mode"] == 2 and segs[0]["granule"] == 4
    # defaults: 1280 bytes
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 1264], strides=[4000, 1]))[0][0]["mode"] == 2
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 1280], strides=[4000, 1]))[0][0]["mode"] == 1
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 1279], strides=[4000, 1]))[0][0]["mode"] == 2
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 1281], strides=[4000, 1]))[0][0]["mode"] == 1
    # runs of a whole number of 64-byte groups keep counting packed bytes; others pad to four lanes
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 128], strides=[4000, 1]))[0][0]["lanes_per_run"] == 0
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 112], strides=[4000, 1]))[0][0]["lanes_per_run"] == 8
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 100], strides=[4000, 1]))[0][0]["lanes_per_run"] == 8
    assert seg_of(pkg, tv(pkg, 0x10000, [5, 260], strides=[4000, 1]), ragged_runs=0)[0][0]["mode"] == 1


def test_transposed_views_use_square_blocks(pkg):
    # fp16 [300, 200] transposed: B (contiguous in the tensor) = 300, A (packed inner) = 200
    segs, info = seg_of(pkg, tv(pkg, 0x10000, [300, 200], strides=[1, 300], dtype=(4, 16, 1)))
    s = segs[0]
    assert (s["mode"], s["granule"], s["nbytes"]) == (5, 2, 120000)
    assert s["shape"] == (300, 200) and s["stride_bytes"] == (2, 600)
    assert s["tiles"] == 5 * 4                      # 64 x 64 element blocks
    assert info["threads_per_workgroup"] <= 256
    # fp32 [B, H, S, D] -> permute(2, 0, 3, 1): H becomes the innermost packed dim
    b, h, sq, d = 2, 40, 3, 50
    v = tv(pkg, 0x10000, [sq, b, d, h], strides=[d, h * sq * d, 1, sq * d], dtype=(2, 32, 1))
    s = seg_of(pkg, v)[0][0]
    assert (s["mode"], s["granule"]) == (5, 4)
    # batch dims (sq, b), then the tensor-contiguous dim d, then the packed-inner dim h
    assert s["shape"] == (sq, b, d, h)
    assert s["stride_bytes"] == (4 * d, 4 * h * sq * d, 4, 4 * sq * d)
    assert s["tiles"] == b * sq * 2 * 2             # 32 x 32 element blocks
    # a short dimension: rectangular blocks of about 8 KiB (channels-first -> channels-last, fp32)
    n, c, hw = 16, 3, 512 * 512
    s = seg_of(pkg, tv(pkg, 0x10000, [n, hw, c], strides=[c * hw, 1, hw], dtype=(2, 32, 1)))[0][0]
    assert (s["mode"], s["granule"]) == (5, 4) and s["shape"] == (n, hw, c)
    assert s["tiles"] == n * -(-hw // 680)          # 3 x 680 elements per block (whole vectors)
    # and the other way round: the short dimension is the one contiguous in the tensor
    s = seg_of(pkg, tv(pkg, 0x10000, [n, c, hw], strides=[c * hw, 1, c], dtype=(2, 32, 1)))[0][0]
    assert (s["mode"], s["tiles"]) == (5, n * -(-hw // 680))
    # tiny extents and odd element sizes stay in element mode
    assert seg_of(pkg, tv(pkg, 0x10000, [30, 4], strides=[1, 30]))[0][0]["mode"] == 2
    assert seg_of(pkg, tv(pkg, 0x10000, [30, 20], strides=[1, 30], dtype=(2, 96, 1)))[0][0]["mode"] == 2
    # 16-byte elements transpose as 16 x 16 blocks, 8-byte ones as 32 x 32
    s = seg_of(pkg, tv(pkg, 0x10000, [30, 20], strides=[1, 30], dtype=(2, 128, 1)))[0][0]
    assert (s["mode"], s["granule"], s["tiles"]) == (5, 16, 2 * 2)
    s = seg_of(pkg, tv(pkg, 0x10000, [70, 40], strides=[1, 70], dtype=(2, 64, 1)))[0][0]
    assert (s["mode"], s["granule"], s["tiles"]) == (5, 8, 3 * 2)


def test_negative_and_many_strides(pkg):
    segs, _ = seg_of(pkg, tv(pkg, 0x20000, [4, 2400], strides=[-4000, 1]))
    assert segs[0]["stride_bytes"] == (-4000,) and segs[0]["mode"] == 1
    # 8 strided outer dims: the two outermost are peeled on the host
    shape = [2, 3, 2, 2, 2, 2, 2, 2, 2400]
    strides, acc = [], 2800
    for n in reversed(shape[:-1]):
        strides.insert(0, acc)
        acc *= n + 1                       # leave gaps so nothing merges
    strides.append(1)
    segs, _ = seg_of(pkg, tv(pkg, 0x100000, shape, strides=strides))
    assert len(segs) == 6 and all(s["ndim"] == 6 and s["mode"] == 1 for s in segs)
    assert [s["offset"] for s in segs] == [i * 64 * 2400 for i in range(6)]
    assert segs[1]["address"] - segs[0]["address"] == strides[1]
    assert segs[3]["address"] - segs[0]["address"] == strides[0]


def test_small_bundles_carry_their_tables_in_the_kernel_arguments(pkg):
    """Tables of up to 3.5 KiB (minus a 16-byte head) and bundles of up to `inline_tables`
    tiles with the default geometry need no device table block."""
    def info(views, **tune):
        if tune:
            pkg.tune(**tune)
        try:
            return pkg.BundlePlan.create(views, align=256).launch_info()
        finally:
            pkg.tune(tile_rows=0, inline_tables=16384, nontemporal=-1, group_bytes=512)
    few = [tv(pkg, 0x10000 * (i + 1), [5000]) for i in range(4)]
    i = info(few)
    assert i["inline_tables"] == 1 and i["table_bytes"] + 16 <= 3584
    assert info(few, inline_tables=0)["inline_tables"] == 0
    assert info(few, tile_rows=4)["inline_tables"] == 0            # another geometry: uploaded tables
    assert info(few, nontemporal=3)["inline_tables"] == 0
    assert info([tv(pkg, 0x10000, [3 * 2048])], inline_tables=2)["inline_tables"] == 0   # 3 tiles > 2
    assert info([tv(pkg, 0x10000, [3 * 2048])], inline_tables=3)["inline_tables"] == 1
    many = [tv(pkg, 0x1000 * (i + 1), [100]) for i in range(120)]  # 121 x 32 B of segments alone
    assert info(many, group_bytes=0)["inline_tables"] == 0
    assert info(many[:90], group_bytes=0)["inline_tables"] == 1
    grouped = info(many)                                           # short tensors share tiles
    assert grouped["tiles"] <= 20 and grouped["inline_tables"] == 0     # 18 blocks of 288 B
    assert info(many[:60])["inline_tables"] == 1
    big = [tv(pkg, 0x10000000, [64 << 20])]                        # 32768 tiles
    assert info(big)["inline_tables"] == 0
    strided = [tv(pkg, 0x10000, [64, 64], strides=[1, 64], dtype=(2, 32, 1)),
               tv(pkg, 0x90000, [100, 40], strides=[100, 1])]
    assert info(strided)["inline_tables"] == 1                     # Dims records fit as well
    assert info([tv(pkg, 0x10000, [0])])["inline_tables"] == 0     # nothing to launch


def test_pads_fill_segments_and_host_copies(pkg):
    views = [tv(pkg, 0x10000, [100]),                       # device, pad 156
             tv(pkg, 0x20000, [0]),                         # empty: no segment
             tv(pkg, 0x30000, [256]),                       # device, pad 0
             tv(pkg, 0x40000, [3, 10], strides=[20, 1], device_type=1),   # host, 3 copies + fill
             tv(pkg, 0x50000, [7], device_type=11)]         # pinned host: device segment, last
    plan = pkg.BundlePlan.create(views, align=256)
    segs = plan.segments()
    dev = [s for s in segs if s["mode"] != 4]
    host = [s for s in segs if s["mode"] == 4]
    # the two short device tensors share one group tile; the last one has no neighbour
    assert [(s["tensor"], s["mode"], s["pad"]) for s in dev] == [(0, 6, 156), (2, 6, 0), (3, 3, 226), (4, 0, 0)]
    assert [s["tiles"] for s in dev] == [1, 0, 1, 1]
    assert dev[2]["offset"] == 512 + 30
    assert [(s["address"], s["offset"], s["nbytes"]) for s in host] == [
        (0x40000, 512, 10), (0x40000 + 20, 522, 10), (0x40000 + 40, 532, 10)]
    assert plan.launch_info()["host_copies"] == 3 and plan.launch_info()["host_chunks"] == 1
    assert plan.payload_bytes == 768 + 7


def test_unsupported_device_type_fails(pkg):
    plan = pkg.BundlePlan.create([tv(pkg, 0x1000, [16], device_type=2)], align=1)   # kDLCUDA
    with pytest.raises(pkg.UnsupportedMemoryError):
        plan.segments()


def test_bind_validation(pkg, orc):
    hdr = orc.encode_header([{"device": (10, 0), "dtype": (2, 32, 1), "shape": (100,)},
                             {"device": (10, 0), "dtype": (4, 16, 1), "shape": (8, 8)}], 256)
    plan = pkg.BundlePlan.from_header(hdr)
    with pytest.raises(pkg.AxonRocmError):
        plan.segments()                                          # nothing bound
    with pytest.raises(pkg.MismatchError):
        plan.bind([tv(pkg, 0x1000, [100], dtype=(2, 32, 1))])    # count
    with pytest.raises(pkg.MismatchError):
        plan.bind([tv(pkg, 0x1000, [100], dtype=(2, 32, 1)), tv(pkg, 0x2000, [8, 9], dtype=(4, 16, 1))])
    with pytest.raises(pkg.MismatchError):                       # same bytes, other element width
        plan.bind([tv(pkg, 0x1000, [100], dtype=(2, 32, 1)), tv(pkg, 0x2000, [32], dtype=(2, 32, 1))])
    # a destination view with other strides but the same shape is fine
    plan.bind([tv(pkg, 0x1000, [100], dtype=(0, 32, 1)),
               tv(pkg, 0x2000, [8, 8], strides=[16, 1], dtype=(2, 16, 1))])
    assert [s["mode"] for s in plan.segments()] == [0, 2]


def test_header_and_tensors_in_one_pass(pkg, orc):
    """axr_plan_from_header_bind gives the plan that axr_plan_from_header + axr_plan_bind give,
    with the same refusals."""
    metas = [{"device": (10, 0), "dtype": (2, 32, 1), "shape": (100,)},
             {"device": (10, 0), "dtype": (4, 16, 1), "shape": (8, 8)},
             {"device": (10, 0), "dtype": (1, 8, 1), "shape": (0,)},
             {"device": (10, 0), "dtype": (1, 8, 1), "shape": (5000,)}]
    for align in (1, 256):
        hdr = orc.encode_header(metas, align)
        views = [tv(pkg, 0x1000, [100], dtype=(0, 32, 1)),
                 tv(pkg, 0x2000, [8, 8], strides=[16, 1], dtype=(2, 16, 1)),
                 tv(pkg, 0, [0]), tv(pkg, 0x5003, [5000])]
        two = pkg.BundlePlan.from_header(hdr).bind(views)
        one = pkg.BundlePlan.from_header_bound(hdr, views)
        assert one.segments() == two.segments()
        assert one.layout() == two.layout() and one.header == two.header == hdr
        assert one.launch_info() == two.launch_info()
        assert one.payload_bytes == two.payload_bytes and one.data_bytes == two.data_bytes
        assert [m.shape for m in one.metas()] == [m.shape for m in two.metas()]
        with pytest.raises(pkg.MismatchError):
            pkg.BundlePlan.from_header_bound(hdr, views[:3])
        with pytest.raises(pkg.MismatchError):
            pkg.BundlePlan.from_header_bound(hdr, views[:3] + [tv(pkg, 0x5003, [5001])])
        with pytest.raises(pkg.MismatchError):      # same bytes, other element width
            pkg.BundlePlan.from_header_bound(hdr, [tv(pkg, 0x1000, [200], dtype=(0, 16, 1))] + views[1:])
        with pytest.raises(pkg.AxonRocmError):      # null data for a tensor with bytes
            pkg.BundlePlan.from_header_bound(hdr, views[:3] + [tv(pkg, 0, [5000])])
        with pytest.raises(pkg.HeaderError):
            pkg.BundlePlan.from_header_bound(hdr[:-1], views)
        with pytest.raises(pkg.HeaderError):
            pkg.BundlePlan.from_header_bound(hdr[:20] + b"\x01" + hdr[21:], views)


# ------------------------------------------------------------------ DLPack and devices

def test_dlpack_extract_numpy(pkg):
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    v = pkg.extract(a[:, 1:4])
    assert v.device_type == 1 and v.dtype == (2, 32, 1) and v.shape == (4, 3)
    assert v.strides == (6, 1) and v.data + v.byte_offset == a[:, 1:4].ctypes.data
    assert v.nbytes == 48
    with pytest.raises(TypeError):
        pkg.extract(object())
    # read-only producers (an array over bytes, a broadcast view) refuse the unversioned export;
    # they are asked in DLPack 1.0, may be packed from, and are refused as unpack destinations
    frozen = np.frombuffer(bytes(range(64)), dtype=np.uint8)
    spread = np.broadcast_to(np.float32(3), (4, 2))
    assert not frozen.flags.writeable
    v = pkg.extract(frozen)
    assert v.readonly and v.shape == (64,) and v.data == frozen.ctypes.data
    assert pkg.extract(spread).strides == (0, 0) and not pkg.extract(a).readonly
    plan = pkg.BundlePlan.create([a, frozen, spread], align=1)
    assert plan.payload_bytes == 96 + 64 + 32
    receiver = pkg.BundlePlan.from_header(plan.header)
    with pytest.raises(BufferError, match="read-only"):
        receiver.bind([np.zeros_like(a), frozen, np.zeros((4, 2), np.float32)])
    with pytest.raises(BufferError, match="read-only"):
        pkg.BundlePlan.from_header_bound(plan.header, [np.zeros_like(a), frozen, np.zeros((4, 2), np.float32)])
    receiver.bind([np.zeros_like(a), np.zeros(64, np.uint8), np.zeros((4, 2), np.float32)])
    plan.bind([a, frozen, spread])                      # a sender's plan takes them again
    plan.close()
    receiver.close()


def fresh_of(pkg, array, released, tag):
    dtype = {np.dtype(np.int32): (0, 32, 1), np.dtype(np.float32): (2, 32, 1)}[array.dtype]
    return pkg.DLPackExport(array.ctypes.data, array.shape, dtype, 1, 0, release=lambda: released.append(tag))


def test_dlpack_export_single_consume(pkg):
    released = []
    src = np.arange(40, dtype=np.int32)
    exp = pkg.DLPackExport(src.ctypes.data, (5, 8), (0, 32, 1), 1, 0, release=lambda: released.append(1))
    assert exp.__dlpack_device__() == (1, 0)
    out = np.from_dlpack(exp)
    assert out.shape == (5, 8) and out.dtype == np.int32 and np.array_equal(out.reshape(-1), src)
    with pytest.raises(RuntimeError):
        exp.__dlpack__()
    del out
    import gc
    gc.collect()
    assert released == [1]
    # never consumed: released when dropped
    exp2 = pkg.DLPackExport(src.ctypes.data, 160, (1, 8, 1), 1, 0, release=lambda: released.append(2))
    del exp2
    gc.collect()
    assert released == [1, 2]
    # argument checks of the reference's wrapper (axon/python/src/dlpack_helpers.hpp:106-155):
    # each refusal still consumes the capsule, and the memory is released with the wrapper
    def fresh(tag, device_type=1):
        return pkg.DLPackExport(src.ctypes.data, 160, (1, 8, 1), device_type, 0,
                                release=lambda: released.append(tag))
    for tag, kwargs, device_type, error, text in (
            (3, {"stream": 0}, 1, ValueError, "stream must be None for CPU"),
            (4, {"dl_device": (10, 0)}, 1, RuntimeError, "not yet supported"),
            (5, {"dl_device": (10, 0), "copy": False}, 1, RuntimeError, "copy=False was specified"),
            (6, {"copy": True}, 1, RuntimeError, "zero-copy only"),
            (7, {"copy": True, "stream": 0}, 10, RuntimeError, "zero-copy only")):
        exp = fresh(tag, device_type)
        with pytest.raises(error, match=text):
            exp.__dlpack__(**kwargs)
        with pytest.raises(RuntimeError, match="already been consumed"):
            exp.__dlpack__()
        del exp
        gc.collect()
        assert released[-1] == tag
    ok = fresh(8)
    capsule = ok.__dlpack__(stream=None, max_version=(1, 0), dl_device=(1, 0), copy=False)   # all accepted
    del capsule, ok
    gc.collect()
    assert released[-1] == 8
    # a consumer that speaks DLPack 1.0 is given the versioned struct with no flag set: numpy's
    # array over it is writable and can be exported again (a handler may modify or return it)
    mine = np.arange(6, dtype=np.int32)
    taken = np.from_dlpack(fresh_of(pkg, mine, released, 20))
    assert taken.flags.writeable
    taken[0] = 77
    assert mine[0] == 77 and pkg.extract(taken).shape == (6,)
    del taken
    gc.collect()
    assert released[-1] == 20
    versioned = fresh_of(pkg, mine, released, 21).__dlpack__(max_version=(1, 0))
    legacy = fresh_of(pkg, mine, released, 22).__dlpack__(max_version=(0, 8))
    assert '"dltensor_versioned"' in repr(versioned) and '"dltensor"' in repr(legacy)
    assert pkg.extract(versioned).shape == (6,) and pkg.extract(legacy).shape == (6,)
    del versioned
    gc.collect()
    assert released[-1] == 21
    del legacy
    gc.collect()
    assert released[-1] == 22
    # a consumer that refuses the capsule (numpy takes host memory only) drops it with its own
    # exception pending: that exception is what the caller sees, and the memory is released
    refused = pkg.DLPackExport(0x1000, (4,), (2, 32, 1), 10, 0, release=lambda: released.append(9))
    with pytest.raises(RuntimeError, match="Unsupported device"):
        np.from_dlpack(refused)
    del refused
    gc.collect()
    assert released[-1] == 9


def test_exported_tensors_may_outlive_the_interpreter(pkg):
    """A consumer that still holds tensors made from this package's capsules when the interpreter
    shuts down (script globals) must not bring the process down: the tensors are dropped after the
    modules have been cleared, and the deleters they call have to be valid and quiet then."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = (
        "import sys; sys.path.insert(0, %r)\n"
        "import numpy as np, torch\n"
        "import __graft_entry__ as e\n"
        "pkg = e.load_package()\n"
        "buf = np.arange(8, dtype=np.float32)\n"
        "x = np.from_dlpack(pkg.DLPackExport(buf.ctypes.data, (8,), (2, 32, 1), 1, 0, release=lambda: None))\n"
        "y = torch.from_dlpack(pkg.DLPackExport(buf.ctypes.data, (2, 4), (2, 32, 1), 1, 0, release=lambda: None))\n"
        "z = pkg.DLPackExport(buf.ctypes.data, (8,), (2, 32, 1), 1, 0).__dlpack__()   # a capsule nobody consumed\n"
        "print('end', float(x.sum()), float(y.sum()))\n" % root)
    out = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, (out.returncode, out.stderr[-800:])
    assert "end 28.0 28.0" in out.stdout
    assert "Exception ignored" not in out.stderr and "Traceback" not in out.stderr, out.stderr[-800:]


def test_device_objects(pkg):
    d = pkg.rocm(3)
    assert d.get_type() == pkg.DeviceType.ROCM and d.get_type_string() == "rocm"
    assert d.get_context_handle() == 3 and repr(d) == "RocmDevice(device_id=3)"
    assert d.clone().device_id == 3
    c = pkg.cpu(numa_node=1)
    assert c.get_type_string() == "cpu" and c.get_context_handle() is None
    assert isinstance(pkg.auto_detect(), pkg.Device)
    # the rest of the reference's device module (axon/python/tests/test_device_api.py:7-131)
    for name in ("CPU", "CUDA", "ROCM", "SYCL"):
        assert hasattr(pkg.DeviceType, name)
    assert pkg.CpuDevice().get_type() == pkg.DeviceType.CPU and "CpuDevice" in repr(pkg.CpuDevice())
    assert c.numa_node == 1 and "numa_node=1" in repr(c) and pkg.cpu(numa_node=0).numa_node == 0
    cuda_dev = pkg.CudaDevice(device_id=0)
    assert cuda_dev.get_type() == pkg.DeviceType.CUDA and cuda_dev.get_type_string() == "cuda"
    assert cuda_dev.device_id == 0 and "CudaDevice" in repr(cuda_dev)
    with_context = pkg.CudaDevice(device_id=1, context=0x12345678)
    assert with_context.device_id == 1 and with_context.get_context_handle() == 0x12345678
    sycl_dev = pkg.SyclDevice(device_id=0)
    assert sycl_dev.get_type() == pkg.DeviceType.SYCL and sycl_dev.get_type_string() == "sycl"
    assert sycl_dev.device_id == 0 and "SyclDevice" in repr(sycl_dev)
    assert isinstance(pkg.cuda(), pkg.CudaDevice) and pkg.cuda(device_id=1).device_id == 1
    assert isinstance(pkg.rocm(), pkg.RocmDevice) and isinstance(pkg.sycl(), pkg.SyclDevice)
    # a runtime takes any of them (and none); with a host device its whole lifecycle runs here
    for device in (pkg.cpu(), pkg.cuda(context=None), None):
        assert pkg.AxonRuntime("test_worker", device=device) is not None
    runtime = pkg.AxonRuntime("test_worker", device=pkg.cpu())
    runtime.start()
    assert len(runtime.get_local_address()) > 0
    runtime.stop()
    runtime.stop()                                                   # stopping twice is harmless
    pkg.AxonRuntime("never_started", device=pkg.cpu()).stop()        # so is stopping without a start


# ------------------------------------------------------------------ no device: fail loudly

def test_no_silent_cpu_fallback_without_gpu(pkg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert pkg.device_count() == 0
    assert isinstance(pkg.auto_detect(), pkg.CpuDevice)
    src = np.arange(64, dtype=np.uint8)
    plan = pkg.BundlePlan.create([src], align=1)
    host_payload = np.zeros(64, np.uint8)
    with pytest.raises(pkg.AxonRocmError):          # host tensors still move through HIP copies
        plan.pack(host_payload.ctypes.data, 64)
    assert not host_payload.any()
    with pytest.raises(pkg.AxonRocmError):
        pkg.DevicePool(device=0)
    with pytest.raises(pkg.AxonRocmError):
        pkg.RocmMemoryResourceManager().allocate(3, 1024)
    with pytest.raises(pkg.AxonRocmError):
        with pkg.rocm(0).activate():
            pass


def test_missing_library_is_an_import_error(pkg, monkeypatch):
    monkeypatch.setattr(pkg._capi, "_lib", None)
    monkeypatch.setattr(pkg._capi, "LIBRARY_PATH", "/nonexistent/libaxon_rocm.so")
    with pytest.raises(ImportError):
        pkg._capi.load()


# ------------------------------------------------------------------ native DLPack extraction

def test_native_extraction_matches_the_python_path(pkg):
    """csrc/py_dlpack.c builds the same axr_tensor_t array as the ctypes reader,
    for contiguous, strided, 0-d and empty producers (numpy and torch, CPU)."""
    import torch
    from execution_ucx_amd import dlpack
    assert dlpack._native() is not None, "build lib/_axr_dlpack*.so with `make -C execution-ucx_amd`"
    base = np.arange(5 * 7 * 3, dtype=np.float32).reshape(5, 7, 3)
    objs = [base, base[1:4, ::2], np.zeros((0, 4), np.int16), np.array(3.0),
            torch.arange(24, dtype=torch.int64).reshape(2, 3, 4).permute(2, 0, 1),
            torch.zeros(17, dtype=torch.bfloat16)]
    native = dlpack.TensorArray.from_objects(objs)
    python = dlpack.TensorArray(dlpack.extract_many(objs))
    assert native.count == python.count == len(objs)
    fields = ("data", "device_type", "device_id", "ndim", "dtype_code", "dtype_bits", "dtype_lanes",
              "byte_offset")
    for i in range(native.count):
        a, b = native.array[i], python.array[i]
        assert [getattr(a, f) for f in fields] == [getattr(b, f) for f in fields], i
        assert [a.shape[d] for d in range(a.ndim)] == [b.shape[d] for d in range(b.ndim)]
        assert bool(a.strides) == bool(b.strides)
        if a.strides:
            assert [a.strides[d] for d in range(a.ndim)] == [b.strides[d] for d in range(b.ndim)]
    assert [v.shape for v in native.views] == [v.shape for v in python.views]
    # both give the same plan
    assert pkg.BundlePlan.create(objs, align=64).header == \
        pkg.BundlePlan.create(dlpack.extract_many(objs), align=64).header
    # TensorViews and foreign objects take the Python path / fail as before
    mixed = dlpack.TensorArray.from_objects([objs[0], dlpack.extract(objs[1])])
    assert mixed.count == 2
    with pytest.raises(TypeError):
        dlpack.TensorArray.from_objects([object()])


def test_torch_tensors_skip_the_python_wrapper_but_keep_its_refusals(pkg):
    """Plain torch.Tensor objects are exported with torch.utils.dlpack.to_dlpack from
    C; what Tensor.__dlpack__ refuses is still refused with its own error, subclasses
    keep going through __dlpack__, and both routes describe the same memory."""
    import torch
    from execution_ucx_amd import dlpack
    native = dlpack._native()
    assert native is not None
    fast = dlpack._torch_exporter()
    assert fast[0] is torch.Tensor and fast[2] == -1      # no GPU context in this process

    tensors = [torch.arange(60, dtype=torch.float32).reshape(3, 4, 5)[:, 1:3],
               torch.zeros(0, 7, dtype=torch.int8), torch.tensor(2.5, dtype=torch.float64),
               torch.arange(8, dtype=torch.int16).view(torch.bfloat16)]
    calls = []
    counting = (fast[0], lambda t: (calls.append(1), fast[1](t))[1], fast[2])
    a = native.describe(tensors, *counting)
    b = native.describe(tensors)
    assert len(calls) == len(tensors)
    assert bytes(a[0])[:8] == bytes(b[0])[:8] and bytes(a[1]) == bytes(b[1])
    va = dlpack.TensorArray.from_objects(tensors).views
    vb = dlpack.extract_many(tensors)
    assert [(x.data, x.shape, x.strides or None, x.dtype) for x in va] == \
        [(x.data, x.shape, x.strides or None, x.dtype) for x in vb]   # 0-d: () or None

    class Wrapped(torch.Tensor):
        pass
    calls.clear()
    native.describe([tensors[0].as_subclass(Wrapped)], *counting)
    assert calls == []                                    # a subclass may override __dlpack__

    for bad, text in ((torch.zeros(3, requires_grad=True), "gradient"),
                      (torch.zeros(3, dtype=torch.complex64).conj(), "conjugate"),
                      (torch.zeros(3, 3).to_sparse(), "layout")):
        with pytest.raises(BufferError, match=text):
            dlpack.TensorArray.from_objects([tensors[0], bad])
    # a GPU tensor of another device than the one passed goes to __dlpack__ as well:
    # with device -1 every GPU tensor does, so a process without a context never
    # hands out GPU memory through the short route (checked on the capsule in C)


def test_torch_tensors_read_without_capsules_match_the_capsule_route(pkg):
    """lib/_axr_torch reads plain torch tensors through torch's non-owning DLPack converter:
    every descriptor field equals what a capsule from torch.utils.dlpack.to_dlpack carries, for
    each dtype torch exports and for views with size-1, size-0, stepped and permuted dimensions;
    anything Tensor.__dlpack__ would refuse, a subclass or a foreign producer makes it decline
    (None), and the bundle then takes the capsule route with that route's answer."""
    import torch
    from execution_ucx_amd import dlpack
    direct = dlpack._native_torch()
    native = dlpack._native()
    assert direct is not None, "build lib/_axr_torch*.so with `make -C execution-ucx_amd`"
    to_dlpack = torch.utils.dlpack.to_dlpack
    tensors = []
    for dt in (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64, torch.float16,
               torch.bfloat16, torch.float32, torch.float64, torch.bool, torch.complex64,
               torch.complex128, torch.uint16, torch.uint32, torch.uint64):
        base = torch.zeros(4 * 6 * 8, dtype=dt)
        cube = base.view(4, 6, 8)
        tensors += [base, cube, cube[:, ::2, 1:], cube.permute(2, 0, 1), cube[1], base.view(4, 1, 48),
                    base.view(4, 1, 48)[:, :, ::3], base[:0], cube[:, :0], base[3:4].reshape(()),
                    base.view(1, 192), base.view(192, 1).t()]
    for dt in (torch.float8_e4m3fn, torch.float8_e5m2):   # exported or not, both routes agree
        try:
            to_dlpack(torch.zeros(4, dtype=dt))
            tensors.append(torch.zeros(4, 6, dtype=dt)[:, ::2])
        except (BufferError, RuntimeError, TypeError):
            assert direct.describe([torch.zeros(4, dtype=dt)], -1) is None
    a = direct.describe(tensors, -1)
    b = native.describe(tensors, torch.Tensor, to_dlpack, -1)
    assert a is not None and a[2] == tensors                       # the owners are the tensors
    assert len(a[0]) == len(b[0]) and bytes(a[1]) == bytes(b[1])   # shapes and strides
    ta = (dlpack._capi.Tensor * len(tensors)).from_buffer(a[0])
    tb = (dlpack._capi.Tensor * len(tensors)).from_buffer(b[0])
    fields = ("data", "device_type", "device_id", "ndim", "dtype_code", "dtype_bits", "dtype_lanes",
              "byte_offset")
    dims_a = C.addressof((C.c_char * len(a[1])).from_buffer(a[1])) if len(a[1]) else 0
    dims_b = C.addressof((C.c_char * len(b[1])).from_buffer(b[1])) if len(b[1]) else 0
    for i in range(len(tensors)):
        assert [getattr(ta[i], f) for f in fields] == [getattr(tb[i], f) for f in fields], i
        for name in ("shape", "strides"):   # the pointers name the same places of the two dims blocks
            pa = C.cast(getattr(ta[i], name), C.c_void_p).value
            pb = C.cast(getattr(tb[i], name), C.c_void_p).value
            assert (pa is None) == (pb is None), (i, name)
            if pa is not None:
                assert pa - dims_a == pb - dims_b, (i, name)
    del ta, tb
    assert pkg.BundlePlan.create(tensors[:40], align=64).header == \
        pkg.BundlePlan.create(dlpack.extract_many(tensors[:40]), align=64).header

    class Wrapped(torch.Tensor):
        pass
    good = tensors[1]
    for other in (good.as_subclass(Wrapped), torch.zeros(3, requires_grad=True),
                  torch.zeros(3, dtype=torch.complex64).conj(), torch.zeros(3, 3).to_sparse(),
                  torch.nn.Parameter(torch.zeros(3)), np.zeros(3), object(),
                  torch.zeros(3, device="meta")):
        assert direct.describe([good, other], -1) is None, type(other)
    # a Parameter that requires no gradient is a Tensor as far as the export goes
    frozen = torch.nn.Parameter(torch.arange(6.0).view(2, 3), requires_grad=False)
    assert bytes(direct.describe([frozen], -1)[0])[:24] == \
        bytes(native.describe([frozen], torch.Tensor, to_dlpack, -1)[0])[:24]   # up to the shape pointer
    assert direct.describe([], -1) is not None and direct.describe((good,), -1) is not None
    # the capsule route still has the last word on what was declined
    with pytest.raises(BufferError, match="gradient"):
        dlpack.TensorArray.from_objects([good, torch.zeros(3, requires_grad=True)])
    mixed = dlpack.TensorArray.from_objects([good, np.zeros(3, np.float32)])
    assert mixed.count == 2 and mixed.views[1].shape == (3,)


# ------------------------------------------------------------------ bench.py contract (no GPU needed)

def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "one GPU" in (out.stderr + out.stdout)


def test_product_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under the package may import it."""
    pkg_dir = os.path.join(ROOT, "execution-ucx_amd")
    for name in os.listdir(pkg_dir):
        if name.endswith(".py"):
            text = open(os.path.join(pkg_dir, name)).read()
            assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), name


# ------------------------------------------------------------------ edge cases of the planner

def test_empty_and_extreme_bundles(pkg, orc):
    # no tensors at all: an empty payload and a header that round-trips
    plan = pkg.BundlePlan.create([], align=256)
    assert plan.payload_bytes == 0 and plan.num_tensors == 0
    back = pkg.BundlePlan.from_header(plan.header)
    assert back.num_tensors == 0 and back.payload_bytes == 0
    assert orc.decode_header(plan.header) == (256, 0, [])
    # only empty and 0-d tensors: offsets exist, no bytes, no segments
    views = [tv(pkg, 0, [0]), tv(pkg, 0, []), tv(pkg, 0, [4, 0, 3])]
    plan = pkg.BundlePlan.create(views, align=64)
    assert plan.payload_bytes == 0 and plan.segments() == []
    assert plan.launch_info()["tiles"] == 0
    # 64 dimensions (the most a tensor may have); 65 are refused
    shape = [1] * 62 + [3, 5]
    plan = pkg.BundlePlan.create([tv(pkg, 0x1000, shape)], align=1)
    assert plan.payload_bytes == 15 and plan.segments()[0]["mode"] == 0
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0x1000, [1] * 65)], align=1)
    # element counts that overflow 64 bits are refused, unless an extent is zero
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0x1000, [2 ** 40, 2 ** 40])], align=1)
    assert pkg.BundlePlan.create([tv(pkg, 0, [2 ** 40, 2 ** 40, 0])], align=1).payload_bytes == 0
    # a null data pointer is only acceptable for an empty tensor
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0, [8])], align=1)
    # sizes that each fit 64 bits but add up past 2^64 are refused as well
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0x1000, [2 ** 62], dtype=(1, 16, 1))] * 2, align=1)
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.create([tv(pkg, 0x1000, [2 ** 63 - 4], dtype=(1, 16, 1)), tv(pkg, 0x1000, [1])],
                              align=16)


def test_header_whose_sizes_wrap_64_bits_is_refused(pkg):
    """Two tensors of 2^63 bytes each: offset 0 and 2^63, payload 2^64 = 0 after
    wrapping.  Such a header must not decode into views that lie outside the payload."""
    import struct
    n, align, payload = 2, 1, 0
    h = struct.pack("<IHHIIQ", 0x42545841, 1, 0, n, align, payload)
    for off in (0, 2 ** 63):
        h += struct.pack("<QQiiiBBHQq", off, 2 ** 63, 10, 0, 1, 1, 16, 1, 0, 2 ** 62)
    with pytest.raises(pkg.AxonRocmError) as e:
        pkg.BundlePlan.from_header(h)
    assert e.value.status == pkg._capi.AXR_ERR_HEADER
    # the align-up step can wrap too: offset 2^64 - 8 rounded up to 16
    h = struct.pack("<IHHIIQ", 0x42545841, 1, 0, 2, 16, 1)
    h += struct.pack("<QQiiiBBHQq", 0, 2 ** 64 - 8, 10, 0, 1, 1, 16, 1, 0, 2 ** 63 - 4)
    h += struct.pack("<QQiiiBBHQq", 0, 1, 10, 0, 1, 1, 8, 1, 0, 1)
    with pytest.raises(pkg.AxonRocmError):
        pkg.BundlePlan.from_header(h)


def _probe_in_subprocess(env_library=None):
    """axr_ucx_probe and axr_am_context_create_ucx in a fresh process (the probe runs once per
    process), optionally with AXR_UCX_LIBRARY naming the library to load."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import ctypes as C, json, sys\n"
        f"sys.path.insert(0, {root!r})\n"
        "import __graft_entry__ as e\n"
        "pkg = e.load_package(); capi = pkg._capi; lib = capi.load()\n"
        "p = capi.UcxProbe(); assert lib.axr_ucx_probe(C.byref(p)) == 0\n"
        "ctx = C.c_void_p(1)\n"
        "rc = lib.axr_am_context_create_ucx(b'x', C.byref(ctx))\n"
        "print(json.dumps({'available': p.available, 'version': [p.version_major, p.version_minor, p.version_release],\n"
        "  'have': list(p.have_symbol), 'library': p.library.decode(), 'message': p.message.decode(),\n"
        "  'names': [lib.axr_ucx_symbol_name(i).decode() for i in range(6)],\n"
        "  'rc': rc, 'ctx': ctx.value, 'error': lib.axr_last_error().decode()}))\n")
    env = dict(os.environ)
    env.pop("AXR_UCX_LIBRARY", None)
    if env_library is not None:
        env["AXR_UCX_LIBRARY"] = env_library
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, env=env)
    assert out.returncode == 0, out.stderr[-2000:]
    return json.loads(out.stdout.strip().splitlines()[-1])


def test_ucx_backend_is_probed_and_refused_clearly(pkg, tmp_path):
    """No UCX on this image: the probe says so, and the UCX-backed context is refused with
    AXR_ERR_UNSUPPORTED and a message that names the library and the loopback alternative.
    With a library that exports the entry points (a stand-in built here: the probe only looks
    symbols up and asks for the version) the refusal names the other missing piece, the UCX
    headers at build time.  Nothing beyond this probe exists of a UCX backend."""
    import shutil
    import subprocess
    capi = pkg._capi
    r = _probe_in_subprocess()
    assert r["names"] == ["ucp_init_version", "ucp_worker_create", "ucp_mem_map", "ucp_am_send_nbx",
                          "ucp_am_recv_data_nbx", "ucp_worker_progress"]
    if not r["available"]:                       # the image as it is
        assert r["library"] == "" and r["have"] == [0] * 6
        assert "libucp.so.0" in r["message"]
        assert r["rc"] == capi.AXR_ERR_UNSUPPORTED and r["ctx"] is None
        assert "libucp.so.0" in r["error"] and "axr_am_context_create" in r["error"]
    # a named library that does not exist is the only one tried
    r = _probe_in_subprocess(str(tmp_path / "nowhere" / "libucp.so.0"))
    assert not r["available"] and "nowhere" in r["message"] and r["rc"] == capi.AXR_ERR_UNSUPPORTED
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no C compiler for the stand-in library")
    src = tmp_path / "standin.c"
    src.write_text(
        "void ucp_get_version(unsigned* a, unsigned* b, unsigned* c) { *a = 1; *b = 20; *c = 0; }\n"
        + "".join(f"int {n}(void) {{ return -1; }}\n" for n in
                  ("ucp_init_version", "ucp_worker_create", "ucp_mem_map", "ucp_am_send_nbx", "ucp_worker_progress")))
    partial = tmp_path / "libucp_partial.so"
    subprocess.run([gcc, "-shared", "-fPIC", str(src), "-o", str(partial)], check=True)
    r = _probe_in_subprocess(str(partial))
    assert not r["available"] and r["version"] == [1, 20, 0]
    assert r["have"] == [1, 1, 1, 1, 0, 1] and "ucp_am_recv_data_nbx" in r["message"]
    src.write_text(src.read_text() + "int ucp_am_recv_data_nbx(void) { return -1; }\n")
    whole = tmp_path / "libucp_whole.so"
    subprocess.run([gcc, "-shared", "-fPIC", str(src), "-o", str(whole)], check=True)
    r = _probe_in_subprocess(str(whole))
    assert r["available"] == 1 and r["have"] == [1] * 6 and r["library"] == str(whole)
    assert r["rc"] == capi.AXR_ERR_UNSUPPORTED and r["ctx"] is None
    assert "ucp.h" in r["error"] and "UCX 1.20.0" in r["error"]


def test_runtime_registration_addresses_and_plain_calls_without_a_gpu(pkg):
    """The AxonRuntime-shaped entry (axon/python/src/bindings_runtime.cpp:700-830, 910-1016):
    registration rules, in-process addresses, and a call whose arguments and result are plain
    values only (no tensor, so no payload and no GPU work: the record travels as an eager
    header-only message)."""
    import asyncio
    rt = pkg.runtime
    with pytest.raises(ValueError):
        pkg.AxonRuntime("")
    # the timeout argument in the reference's forms (bindings_runtime_helpers.cpp:253-276)
    import datetime
    for given, ms in ((None, 300), (3000, 3000), (1.5, 1500), (datetime.timedelta(seconds=2), 2000)):
        assert pkg.AxonRuntime("t", timeout=given, device=pkg.cpu()).timeout_ms == ms
    with pytest.raises(RuntimeError, match="timeout must be int"):
        pkg.AxonRuntime("t", timeout="soon", device=pkg.cpu())
    server = pkg.AxonRuntime("cpu_server", device=pkg.cpu())
    with pytest.raises(RuntimeError, match="not been started"):
        server.get_local_address()
    server.start()
    assert server.register_function(lambda a, b="x": f"{a}:{b}", function_name="join") == 1
    assert server.register_function(len, 7) == 7 and server.register_function(abs) == 2
    server.register_function(lambda *a: a if len(a) > 1 else a[0], 30, function_name="echo_all")
    with pytest.raises(RuntimeError, match="already registered"):
        server.register_function(len, 9)               # name "len" taken
    with pytest.raises(RuntimeError, match="already registered"):
        server.register_function(max, 7)
    with pytest.raises(TypeError):
        server.register_function(3)
    import json
    assert json.loads(server.get_local_signatures()) == {"join": 1, "len": 7, "abs": 2, "echo_all": 30}
    client = pkg.AxonRuntime("cpu_client", device=pkg.cpu())
    client.start_client()
    assert server.get_local_address() != client.get_local_address()
    assert server.get_local_address().startswith(b"axr-loopback\0cpu_server\0")

    async def body():
        with pytest.raises(RuntimeError, match="no worker at this address"):
            await client.connect_endpoint_async(b"axr-loopback\0cpu_server\0" + bytes(16), "cpu_server")
        await client.connect_endpoint_async(server.get_local_address(), "cpu_server")
        kw = dict(worker_name="cpu_server", session_id=3, workflow_id=1)
        assert await client.invoke(5, "y", function="join", **kw) == "5:y"
        assert await client.invoke(-2.5, function=2, **kw) == 2.5
        assert await client.invoke(None, function="join", **kw) == "None:x"
        with pytest.raises(RuntimeError, match="not registered"):
            await client.invoke(1, function="nobody", **kw)
        with pytest.raises(RuntimeError, match="TypeError"):
            await client.invoke(1, function=7, **kw)      # len(1) fails in the handler
        with pytest.raises(RuntimeError, match="not serving"):
            await server.connect_endpoint_async(client.get_local_address(), "cpu_client")
            await server.invoke(1, worker_name="cpu_client", session_id=0, function=1)
        with pytest.raises(RuntimeError, match="Unsupported type for inference"):
            await client.invoke(object(), function="join", **kw)
        # lists of plain values travel as parameters, typed by their first element
        # (axon/python/tests/test_numpy_rpc.py:216-247 receive_shards, :399-436 nested bool)
        names, counts, flags = ["tensor_1", "tensor_2"], [[2, 2], [1]], [False, True]
        assert await client.invoke(names, counts, flags, function="echo_all", **kw) == (names, counts, flags)
        nested = await client.invoke([[True, False], [], [False]], function="echo_all", **kw)
        assert nested == [[True, False], [], [False]] and all(isinstance(x, bool) for row in nested for x in row)
        assert await client.invoke([1.5, 2], function="echo_all", **kw) == [1.5, 2.0]
    asyncio.run(body())
    for bad, error in (([[], []], RuntimeError), ([1, "a"], RuntimeError), ([["a"]], RuntimeError),
                       ([[1], 2], TypeError), ({"a": 1}, RuntimeError), ([object()], RuntimeError),
                       ([[object()]], TypeError), ([1, 2.5], RuntimeError)):
        with pytest.raises(error):
            rt._split_arguments([bad])
    # the record framing
    rec, rest = rt._unframe(rt._frame({"a": 1}, b"tail"))
    assert rec == {"a": 1} and rest == b"tail"
    with pytest.raises(RuntimeError):
        rt._unframe(b"nope")
    targs, slots = rt._split_arguments([1, [], "s", None, [1, 2]])
    assert slots == [{"v": 1}, "t", {"v": "s"}, {"v": None}, {"v": [1, 2]}] and targs == [[]]
    assert rt._merge_arguments(slots, ["A"]) == [1, "A", "s", None, [1, 2]]
    client.stop()
    server.stop()
    with pytest.raises(RuntimeError, match="not been started"):
        asyncio.run(client.invoke(1, worker_name="cpu_server", session_id=0, function=1))


def test_runtime_calls_itself_by_name(pkg):
    """axon/python/tests/test_invoke_by_name.py:11-84: one runtime started as server and client,
    connected to its own address, a function registered without an id (and then without a name
    either: the callable's __name__), invoked by name."""
    import asyncio

    def simple_echo(x):
        return x

    async def body():
        runtime = pkg.AxonRuntime("test_worker_name_func", device=pkg.cpu())
        runtime.start_server()
        runtime.start_client()
        try:
            runtime.register_function(callable=simple_echo, function_id=None, function_name="named_echo")
            await runtime.connect_endpoint_async(runtime.get_local_address(), "test_worker_name_func")
            assert await runtime.invoke(42, worker_name="test_worker_name_func", session_id=1,
                                        function="named_echo", workflow_id=1) == 42
        finally:
            runtime.stop()
        implicit = pkg.AxonRuntime("test_worker_implicit", device=pkg.cpu())
        implicit.start()
        try:
            implicit.register_function(callable=simple_echo, function_id=None)
            await implicit.connect_endpoint_async(implicit.get_local_address(), "test_worker_implicit")
            assert await implicit.invoke(100, worker_name="test_worker_implicit", session_id=1,
                                         function="simple_echo", workflow_id=1) == 100
            # addresses that name no worker of this process are refused, empty ones included
            for bad in (bytes([]), bytes([0] * 100)):
                with pytest.raises(RuntimeError, match="no worker at this address"):
                    await implicit.connect_endpoint_async(bad, "non_existent_worker")
        finally:
            implicit.stop()
    asyncio.run(body())


def test_runtime_concurrent_calls_keep_their_replies(pkg):
    """Calls that overlap in one event loop: two clients on one server (served one at a time)
    and one client on two servers whose handlers finish in the opposite order."""
    import asyncio
    order = []

    async def slow(tag, delay):
        order.append(("in", tag))
        await asyncio.sleep(delay)
        order.append(("out", tag))
        return f"done {tag}"

    async def body():
        s1, s2 = pkg.AxonRuntime("srv1", device=pkg.cpu()), pkg.AxonRuntime("srv2", device=pkg.cpu())
        c1, c2 = pkg.AxonRuntime("cli1", device=pkg.cpu()), pkg.AxonRuntime("cli2", device=pkg.cpu())
        for s in (s1, s2):
            s.start()
            s.register_function(slow, 1)
        for c in (c1, c2):
            c.start_client()
            await c.connect_endpoint_async(s1.get_local_address(), "srv1")
            await c.connect_endpoint_async(s2.get_local_address(), "srv2")
        kw = dict(session_id=0, function=1)
        # two clients, one server: the second request waits for the first reply
        r = await asyncio.gather(c1.invoke("a", 0.05, worker_name="srv1", **kw),
                                 c2.invoke("b", 0.0, worker_name="srv1", **kw))
        assert r == ["done a", "done b"]
        assert order == [("in", "a"), ("out", "a"), ("in", "b"), ("out", "b")]
        order.clear()
        # one client, two servers: the slower server's reply arrives second, each call gets its own
        r = await asyncio.gather(c1.invoke("x", 0.05, worker_name="srv1", **kw),
                                 c1.invoke("y", 0.0, worker_name="srv2", **kw))
        assert r == ["done x", "done y"]
        assert order == [("in", "x"), ("in", "y"), ("out", "y"), ("out", "x")]
        for rt in (c1, c2, s1, s2):
            rt.stop()
    asyncio.run(body())
