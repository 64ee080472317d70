"""The planner's device tables, interpreted on the CPU.

Every segment the planner emits (one run, strided run tiles, strided elements,
transposed blocks, zero fill, host copy) says where bytes come from and where
they go.  This test walks those records over a numpy "memory" and compares the
resulting payload with the oracle's pack of the same views, so the address
arithmetic of the planner is checked without a GPU.  (The kernels' own walk of
the same records is checked against the oracle by the GPU tests.)
"""
import itertools

import numpy as np
import pytest

BASE = 0x7F00_0000_0000


def interpret(segments, memory, payload_bytes):
    """Payload produced by moving every segment as its record describes."""
    out = np.full(payload_bytes, 0xEE, np.uint8)
    for s in segments:
        off, run = s["offset"], s["run_bytes"]
        if s["mode"] in (0, 4, 6):
            a = s["address"] - BASE
            out[off:off + run] = memory[a:a + run]
            end = off + run
        elif s["mode"] == 3:
            end = off
        else:
            unit = s["granule"] if s["mode"] == 5 else run
            r = 0
            for idx in itertools.product(*[range(n) for n in s["shape"]]):
                a = s["address"] - BASE + sum(i * st for i, st in zip(idx, s["stride_bytes"]))
                out[off + r * unit:off + (r + 1) * unit] = memory[a:a + unit]
                r += 1
            assert r * unit == s["nbytes"]
            end = off + s["nbytes"]
        out[end:end + s["pad"]] = 0
    return out


def random_view(rng, parent):
    index = []
    for n in parent.shape:
        lo = int(rng.integers(0, n))
        hi = int(rng.integers(lo + 1, n + 1))
        step = int(rng.choice([1, 1, 1, 2, 3, -1, -2]))
        # a negative step walks the same range backwards (numpy exports negative strides)
        index.append(slice(lo, hi, step) if step > 0 else slice(hi - 1, lo - 1 if lo else None, step))
    v = parent[tuple(index)]
    if rng.random() < 0.7:
        v = v.transpose(*[int(i) for i in rng.permutation(parent.ndim)])
    return v


DTYPES = [(np.uint8, (1, 8, 1)), (np.int16, (0, 16, 1)), (np.float32, (2, 32, 1)),
          (np.float64, (2, 64, 1)), (np.complex128, (5, 128, 1))]


MODES_SEEN = set()


@pytest.mark.parametrize("seed", range(8))
def test_tables_reproduce_the_oracle_pack(pkg, orc, seed):
    rng = np.random.default_rng(seed)
    memory = rng.integers(0, 256, size=1 << 25, dtype=np.uint8)
    modes_seen = MODES_SEEN
    for trial in range(25):
        views, chunks, at = [], [], 0
        for _ in range(int(rng.integers(1, 6))):
            np_dt, dl_dt = DTYPES[int(rng.integers(0, len(DTYPES)))]
            item = np.dtype(np_dt).itemsize
            ndim = int(rng.integers(1, 5))
            cap = 70 if ndim <= 2 else (30 if ndim == 3 else 12)
            shape = [int(x) for x in rng.integers(1, cap + 1, size=ndim)]
            if rng.random() < 0.3:                                 # long runs: run tiles
                shape = [min(n, 6) for n in shape[:-1]] + [int(rng.integers(100, 3000))]
            nbytes = int(np.prod(shape)) * item
            at = (at + 15) // 16 * 16 + int(rng.choice([0, 0, item]))
            assert at + nbytes <= memory.size
            parent = memory[at:at + nbytes].view(np_dt).reshape(shape)
            v = random_view(rng, parent)
            byte_start = v.__array_interface__["data"][0] - memory.__array_interface__["data"][0]
            views.append(pkg.TensorView(data=BASE + byte_start, device_type=10, device_id=0, dtype=dl_dt,
                                        shape=tuple(v.shape), strides=tuple(st // item for st in v.strides)))
            chunks.append(np.ascontiguousarray(v).view(np.uint8).reshape(-1))
            assert np.array_equal(chunks[-1], orc.gather_strided(memory, byte_start, v.shape,
                                                                 [st // item for st in v.strides], item))
            at += nbytes
        align = int(rng.choice([1, 64, 256, 4096]))
        plan = pkg.BundlePlan.create(views, align=align)
        segs = plan.segments()
        modes_seen |= {s["mode"] for s in segs}
        got = interpret(segs, memory, plan.payload_bytes)
        assert np.array_equal(got, orc.pack(chunks, align)), (seed, trial)
        # tile ids are consecutive and cover the launch exactly
        assert sum(s["tiles"] for s in segs if s["mode"] != 4) == plan.launch_info()["tiles"]


def test_every_device_mode_was_exercised():
    if not MODES_SEEN:
        pytest.skip("runs after test_tables_reproduce_the_oracle_pack")
    assert {0, 1, 2, 5} <= MODES_SEEN, MODES_SEEN


def test_host_pieces_and_fill_segments(pkg, orc):
    rng = np.random.default_rng(9)
    memory = rng.integers(0, 256, size=1 << 16, dtype=np.uint8)
    host = memory[0x100:0x100 + 30 * 40].reshape(30, 40)[::3, 4:36]        # 10 pieces of 32 B
    views = [pkg.TensorView(data=BASE + 0x100 + 4, device_type=1, device_id=0, dtype=(1, 8, 1),
                            shape=host.shape, strides=(120, 1)),
             pkg.TensorView(data=BASE + 0x4000, device_type=10, device_id=0, dtype=(1, 8, 1),
                            shape=(1000,), strides=None)]
    plan = pkg.BundlePlan.create(views, align=256)
    segs = plan.segments()
    assert sorted(s["mode"] for s in segs) == [0, 3] + [4] * 10
    got = interpret(segs, memory, plan.payload_bytes)
    want = orc.pack([np.ascontiguousarray(host).reshape(-1), memory[0x4000:0x4000 + 1000]], 256)
    assert np.array_equal(got, want)


def move_group_slots(members, memory, out):
    """One group tile moved slot by slot, the way a wavefront does it: slot s belongs to the
    last member whose first slot is <= s; a member of n >= 16 bytes moves 16 bytes per data
    slot, the last one covering its final 16 bytes; shorter members and gaps under 16 bytes move
    in pieces of 8, 4, 2 and 1 bytes; gaps of 16 bytes or more are zero slots."""
    begins = [m["granule"] for m in members]
    total = members[-1]["granule"] + members[-1]["lanes_per_run"]
    assert begins[0] == 0 and total <= 128 and len(members) <= 64
    for a, b in zip(members, members[1:]):
        assert b["granule"] == a["granule"] + a["lanes_per_run"]
    for s in range(total):
        m = max(i for i, b in enumerate(begins) if b <= s)
        mem = members[m]
        n, pad, k = mem["nbytes"], mem["pad"], s - mem["granule"]
        dslots = (n + 15) // 16 if n >= 16 else 1
        pslots = (pad + 15) // 16 if pad >= 16 else 0
        assert mem["lanes_per_run"] == dslots + pslots
        src, dst = mem["address"] - BASE, mem["offset"]
        if k < dslots:
            if n >= 16:
                o = n - 16 if k + 1 == dslots else 16 * k
                out[dst + o:dst + o + 16] = memory[src + o:src + o + 16]
            else:
                for piece, at in ((8, 0), (4, n & 8), (2, n & 12), (1, n & 14)):
                    if n & piece:
                        out[dst + at:dst + at + piece] = memory[src + at:src + at + piece]
            if k + 1 == dslots and 0 < pad < 16:
                for piece, at in ((8, 0), (4, pad & 8), (2, pad & 12), (1, pad & 14)):
                    if pad & piece:
                        out[dst + n + at:dst + n + at + piece] = 0
        else:
            j = k - dslots
            o = n + (pad - 16 if j + 1 == pslots else 16 * j)
            out[dst + o:dst + o + 16] = 0


@pytest.mark.parametrize("align", [1, 2, 16, 256, 4096])
def test_short_tensors_share_group_tiles(pkg, orc, align):
    """Bundles of many short tensors: the planner packs consecutive ones into group tiles
    (mode 6).  The records moved slot by slot must give the oracle's payload, the tile count
    must follow the payload rather than the tensor count, and long tensors in between keep
    their own segments."""
    rng = np.random.default_rng(100 + align)
    memory = rng.integers(0, 256, size=1 << 22, dtype=np.uint8)
    views, chunks, at = [], [], 64
    for i in range(1500):
        np_dt, dl_dt = DTYPES[i % 3]
        item = np.dtype(np_dt).itemsize
        if i % 97 == 50:
            nbytes = int(rng.integers(600, 5000)) // item * item       # a long tensor between the short ones
        elif i % 41 == 7:
            nbytes = 0
        else:
            nbytes = max(item, int(np.exp(rng.uniform(np.log(1), np.log(512)))) // item * item)
        at += int(rng.integers(0, 5)) * item
        views.append(pkg.TensorView(data=BASE + at, device_type=10, device_id=0, dtype=dl_dt,
                                    shape=(nbytes // item,), strides=None))
        chunks.append(memory[at:at + nbytes])
        at += nbytes
    plan = pkg.BundlePlan.create(views, align=align)
    segs = plan.segments()
    if align == 4096:
        # gaps of up to 4095 zero bytes per tensor would be most of a tile: no groups
        assert {s["mode"] for s in segs} == {0}
        assert np.array_equal(interpret(segs, memory, plan.payload_bytes), orc.pack(chunks, align))
        return
    assert {s["mode"] for s in segs} == {0, 6}
    # the records as plain copies
    assert np.array_equal(interpret(segs, memory, plan.payload_bytes), orc.pack(chunks, align))
    # and the group tiles slot by slot
    out = np.full(plan.payload_bytes, 0xEE, np.uint8)
    group, tiles = [], 0
    for s in segs + [None]:
        if s is not None and s["mode"] == 6 and not (s["tiles"] == 1 and group):
            group.append(s)
            tiles += s["tiles"]
            continue
        if group:
            assert len(group) >= 2
            move_group_slots(group, memory, out)
            group = []
        if s is None:
            break
        if s["mode"] == 6:
            group.append(s)
            tiles += 1
        else:
            a = s["address"] - BASE
            out[s["offset"]:s["offset"] + s["run_bytes"]] = memory[a:a + s["run_bytes"]]
            out[s["offset"] + s["run_bytes"]:s["offset"] + s["run_bytes"] + s["pad"]] = 0
            tiles += s["tiles"]
    assert np.array_equal(out, orc.pack(chunks, align))
    info = plan.launch_info()
    assert tiles == info["tiles"]
    short = sum(1 for s in segs if s["mode"] == 6)
    assert short > 1300
    if align <= 16:
        assert info["tiles"] < 1500 // 4       # far fewer wavefronts than tensors
    # switched off, every tensor gets a segment of its own
    pkg.tune(group_bytes=0)
    try:
        plain = pkg.BundlePlan.create(views, align=align)
        assert {s["mode"] for s in plain.segments()} == {0}
        assert plain.launch_info()["tiles"] >= 1400
    finally:
        pkg.tune(group_bytes=512)
