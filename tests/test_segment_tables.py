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
        if s["mode"] in (0, 4):
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
