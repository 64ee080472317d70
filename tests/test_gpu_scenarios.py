"""Random scenarios: bundles of random views (contiguous, pitched, transposed, sliced and
permuted N-D, empty; six element sizes) under random kernel tunables, moved by axr_pack /
axr_unpack or by axr_submit batches that mix directions.  The expected payload is the oracle's
layout of torch's own compact copies; the expected destinations are torch's own strided
copies, compared over the whole parent allocation (nothing outside a view may change).
Bit-exact: this is byte movement."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xCD
UNTOUCHED = 0x77
DTYPE_NAMES = ["uint8", "int16", "bfloat16", "float32", "float64", "complex128"]
TUNABLES = {
    "threads": [0, 0, 64, 128, 256, 512, 1024], "tile_rows": [0, 0, 0, 1, 2, 4, 8, 16],
    "nontemporal": [-1, -1, 0, 1, 2, 3], "max_waves": [1 << 20, 1 << 20, 96, 1024],
    "xcd_remap": [-1, 0, 1], "group_bytes": [512, 512, 0, 128], "group_slots": [64, 128],
    "payload_cache_bytes": [256 << 20, 256 << 20, 0], "head_align": [16, 0, 64],
    "inline_tables": [16384, 0], "device_tables": [512, 0, 8], "transpose": [1, 1, 0],
    "ragged_runs": [1, 1, 0], "gather_run_bytes": [1280, 256, 4096], "submit_interleave": [1, 2, 0],
}


def compact_bytes(t):
    import torch
    if t.numel() == 0:
        return np.zeros(0, np.uint8)
    c = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    c.copy_(t)
    return c.reshape(-1).view(torch.uint8).cpu().numpy()


def random_view(rng, gpu):
    """A view and the uint8 allocation it lives in."""
    import torch
    dt = getattr(torch, DTYPE_NAMES[int(rng.integers(0, len(DTYPE_NAMES)))])
    item = torch.empty((), dtype=dt).element_size()

    def allocation(nbytes):
        return torch.from_numpy(rng.integers(0, 256, size=nbytes, dtype=np.uint8)).to(gpu)

    kind = int(rng.integers(0, 12))
    if kind == 0:                                       # no bytes
        base = torch.zeros(16, dtype=torch.uint8, device=gpu)
        return base.view(dt)[:0], base
    if kind <= 4:                                       # contiguous, 1 B .. 300 KB, at an odd start
        nb = max(int(np.exp(rng.uniform(0.0, np.log(300000)))) // item * item, item)
        off = int(rng.integers(0, 8)) * item
        base = allocation(nb + off + 64)
        return base[off:off + nb].view(dt), base
    if kind <= 6:                                       # rows at a pitch
        rows = int(rng.integers(1, 40))
        cols = max(int(np.exp(rng.uniform(0.0, np.log(6000)))) // item, 1)
        pitch = cols + int(rng.integers(0, 50))
        base = allocation(rows * pitch * item + 64)
        return base[:rows * pitch * item].view(dt).reshape(rows, pitch)[:, :cols], base
    if kind == 7:                                       # a transposed matrix
        r, c = int(rng.integers(1, 300)), int(rng.integers(1, 300))
        base = allocation(r * c * item)
        return base.view(dt).reshape(r, c).t(), base
    ndim = int(rng.integers(2, 6))                      # sub-ranges with steps, permuted
    shape = [int(x) for x in rng.integers(1, 7, size=ndim)]
    shape[int(rng.integers(0, ndim))] = int(rng.integers(1, 200))
    base = allocation(int(np.prod(shape)) * item)
    v = base.view(dt).reshape(shape)
    index = []
    for n in shape:
        a = int(rng.integers(0, n))
        index.append(slice(a, int(rng.integers(a + 1, n + 1)), int(rng.integers(1, 4))))
    v = v[tuple(index)]
    if rng.integers(0, 2):
        v = v.permute(*[int(x) for x in rng.permutation(ndim)])
    return v, base


def destination_like(v, base):
    """(destination view with v's strides in a fresh allocation, that allocation, the
    allocation as it must look after the scatter)"""
    import torch
    fresh = torch.full_like(base, UNTOUCHED)
    expect = torch.full_like(base, UNTOUCHED)
    if v.numel() == 0:
        return fresh.view(v.dtype)[:0], fresh, expect
    off, item = v.data_ptr() - base.data_ptr(), v.element_size()
    nb = (base.numel() - off) // item * item
    torch.as_strided(expect[off:off + nb].view(v.dtype), v.shape, v.stride(), 0).copy_(v)
    return torch.as_strided(fresh[off:off + nb].view(v.dtype), v.shape, v.stride(), 0), fresh, expect


def one_scenario(pkg, orc, gpu, stream, seed, defaults):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(777_000 + seed)
    tun = {k: int(rng.choice(v)) for k, v in TUNABLES.items()}
    if rng.integers(0, 3) == 0:
        tun = dict(defaults)
    pkg.tune(**tun)
    bundles = []
    for _ in range(int(rng.integers(1, 5))):
        n = int(rng.integers(1, int(rng.choice([1, 3, 17, 120, 700])) + 1))
        bundles.append([random_view(rng, gpu) for _ in range(n)])
    align = int(rng.choice([1, 1, 256, 256, 16, 64, 4096]))
    plans, bufs, wants = [], [], []
    for views in bundles:
        tensors = [v for v, _ in views]
        plan = pkg.BundlePlan.create(tensors, align=align)
        plans.append(plan)
        wants.append(orc.pack([compact_bytes(t) for t in tensors], align))
        assert plan.payload_bytes == len(wants[-1]), (seed, tun)
        bufs.append(torch.full((plan.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu))
    torch.cuda.synchronize()
    batched = bool(rng.integers(0, 2))
    if batched:
        arr = (capi.Job * len(plans))()
        for i, (p, b) in enumerate(zip(plans, bufs)):
            arr[i] = capi.Job(p._h, 0, b.data_ptr(), p.payload_bytes, 0)
        capi.check(lib.axr_submit(arr, len(plans), stream))
    else:
        for p, b in zip(plans, bufs):
            p.pack(b.data_ptr(), p.payload_bytes, stream.value)
    capi.check(lib.axr_stream_synchronize(stream))
    for i, (p, b, w) in enumerate(zip(plans, bufs, wants)):
        got = b.cpu().numpy()
        assert np.array_equal(got[:p.payload_bytes], w), ("pack", seed, i, tun)
        assert (got[p.payload_bytes:] == POISON).all(), ("pack wrote past the payload", seed, i, tun)
    rplans, checks = [], []
    for views, p in zip(bundles, plans):
        made = [destination_like(v, base) for v, base in views]
        rplans.append(pkg.BundlePlan.from_header(p.header).bind([m[0] for m in made]))
        checks.append(made)
    torch.cuda.synchronize()
    if batched:       # the unpacks and, somewhere among them, a second pack of the first bundle
        again = torch.full((plans[0].payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu)
        jobs = [(rp, 1, b.data_ptr(), p.payload_bytes) for rp, p, b in zip(rplans, plans, bufs)]
        jobs.insert(int(rng.integers(0, len(jobs) + 1)), (plans[0], 0, again.data_ptr(), plans[0].payload_bytes))
        arr = (capi.Job * len(jobs))()
        for i, (p, unpack, ptr, nbytes) in enumerate(jobs):
            arr[i] = capi.Job(p._h, unpack, ptr, nbytes, 0)
        capi.check(lib.axr_submit(arr, len(jobs), stream))
        capi.check(lib.axr_stream_synchronize(stream))
        got = again.cpu().numpy()
        assert np.array_equal(got[:plans[0].payload_bytes], wants[0]), ("second pack", seed, tun)
        assert (got[plans[0].payload_bytes:] == POISON).all(), ("second pack wrote past the payload", seed, tun)
    else:
        for rp, p, b in zip(rplans, plans, bufs):
            rp.unpack(b.data_ptr(), p.payload_bytes, stream.value)
        capi.check(lib.axr_stream_synchronize(stream))
    for bi, made in enumerate(checks):
        for ti, (_, fresh, expect) in enumerate(made):
            v = bundles[bi][ti][0]
            assert torch.equal(fresh, expect), ("unpack", seed, bi, ti, tuple(v.shape), v.stride(), v.dtype, tun)
    for p in plans + rplans:
        p.close()


@pytest.mark.parametrize("block", range(8))
def test_random_bundles_under_random_tunables(pkg, orc, gpu, block):
    lib, capi = pkg._capi.load(), pkg._capi
    defaults = {}
    for k in TUNABLES:
        v = C.c_int64()
        capi.check(lib.axr_tune_get(k.encode(), C.byref(v)))
        defaults[k] = v.value
    stream = C.c_void_p()
    capi.check(lib.axr_stream_create(C.byref(stream)))
    try:
        for seed in range(block * 25, block * 25 + 25):
            one_scenario(pkg, orc, gpu, stream, seed, defaults)
    finally:
        pkg.tune(**defaults)
        capi.check(lib.axr_stream_synchronize(stream))
        capi.check(lib.axr_stream_destroy(stream))
