"""axr_submit (several bundles per launch), tensor address deltas and the head peel of
contiguous segments, against the CPU oracle and against axr_pack / axr_unpack, through
the C ABI.  Bit-exact: this is byte movement."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xCD


def chunk_of(t):
    import torch
    if isinstance(t, torch.Tensor):
        c = torch.empty(t.shape, dtype=t.dtype, device=t.device)
        c.copy_(t)
        return c.reshape(-1).view(torch.uint8).cpu().numpy()
    return np.ascontiguousarray(t).view(np.uint8).reshape(-1)


def random_tensors(rng, gpu, count, lo=16, hi=48 * 1024, strided_every=0, transposed_every=0):
    import torch
    dtypes = [torch.uint8, torch.float16, torch.float32, torch.int64]
    out = []
    for i in range(count):
        dt = dtypes[i % 4]
        item = torch.empty((), dtype=dt).element_size()
        if transposed_every and i % transposed_every == 1:
            r, c = int(rng.integers(40, 200)), int(rng.integers(40, 200))
            raw = torch.from_numpy(rng.integers(0, 256, size=r * c * item, dtype=np.uint8)).to(gpu)
            out.append(raw.view(dt).reshape(r, c).t())
        elif strided_every and i % strided_every == 0:
            rows, cols, pitch = int(rng.integers(2, 20)), int(rng.integers(1, 900)), 1024
            raw = torch.from_numpy(rng.integers(0, 256, size=rows * pitch * item, dtype=np.uint8)).to(gpu)
            out.append(raw.view(dt).reshape(rows, pitch)[:, :cols])
        else:
            n = max(1, int(np.exp(rng.uniform(np.log(lo), np.log(hi)))) // item)
            raw = torch.from_numpy(rng.integers(0, 256, size=n * item, dtype=np.uint8)).to(gpu)
            out.append(raw.view(dt))
    return out


def zeros_like_views(tensors):
    """Destinations with the same shapes and strides as the sources (views stay views)."""
    import torch
    outs = []
    for t in tensors:
        if t.is_contiguous():
            outs.append(torch.zeros_like(t))
        else:
            base = torch.zeros(t.untyped_storage().nbytes(), dtype=torch.uint8, device=t.device)
            outs.append(torch.as_strided(base.view(t.dtype), t.shape, t.stride(), t.storage_offset()))
    return outs


def job_array(capi, jobs):
    arr = (capi.Job * len(jobs))()
    for i, (plan, unpack, ptr, nbytes, delta) in enumerate(jobs):
        arr[i] = capi.Job(plan._h, unpack, ptr, nbytes, delta)
    return arr


@pytest.mark.parametrize("align", [1, 256])
def test_submit_matches_the_oracle_and_separate_calls(pkg, orc, gpu, align):
    """Six jobs in one call: packs and unpacks of bundles with plain tensors, strided
    views, transposed views (element kernels), a bundle small enough for inline tables,
    one with a host tensor (runs on its own) and one with another tile size."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(31 + align)
    stream = C.c_void_p()
    capi.check(lib.axr_stream_create(C.byref(stream)))
    bundles = [
        random_tensors(rng, gpu, 400),                                  # plain, pack
        random_tensors(rng, gpu, 300, strided_every=5),                 # run tiles + elements, pack
        random_tensors(rng, gpu, 5),                                    # tiny
        random_tensors(rng, gpu, 200, strided_every=4, transposed_every=6),
        random_tensors(rng, gpu, 64, lo=100000, hi=400000),            # larger tensors
    ]
    host = rng.integers(0, 256, size=70001, dtype=np.uint8)
    bundles.append([bundles[0][3], host, bundles[0][4]])                # host tensor inside
    torch.cuda.synchronize()
    plans, bufs, wants = [], [], []
    for tensors in bundles:
        plan = pkg.BundlePlan.create(tensors, align=align)
        plans.append(plan)
        bufs.append(torch.full((plan.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu))
        wants.append(orc.pack([chunk_of(t) for t in tensors], align))
    torch.cuda.synchronize()
    try:
        # all packs in one call
        arr = job_array(capi, [(p, 0, b.data_ptr(), p.payload_bytes, 0) for p, b in zip(plans, bufs)])
        capi.check(lib.axr_submit(arr, len(plans), stream))
        capi.check(lib.axr_stream_synchronize(stream))
        for p, b, w in zip(plans, bufs, wants):
            got = b.cpu().numpy()
            assert np.array_equal(got[:p.payload_bytes], w)
            assert (got[p.payload_bytes:] == POISON).all()
        # unpacks of bundles 0..4 together with a fresh pack of bundle 0's twin: mixed directions
        outs = [zeros_like_views(t) for t in bundles[:5]]
        rplans = [pkg.BundlePlan.from_header(p.header).bind(o) for p, o in zip(plans[:5], outs)]
        twin = pkg.BundlePlan.create(bundles[0], align=align)
        twin_buf = torch.full((twin.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu)
        torch.cuda.synchronize()
        jobs = [(rp, 1, b.data_ptr(), p.payload_bytes, 0) for rp, p, b in zip(rplans, plans, bufs)]
        jobs.insert(1, (twin, 0, twin_buf.data_ptr(), twin.payload_bytes, 0))
        arr = job_array(capi, jobs)
        capi.check(lib.axr_submit(arr, len(jobs), stream))
        capi.check(lib.axr_stream_synchronize(stream))
        for tensors, o in zip(bundles[:5], outs):
            for a, b in zip(tensors, o):
                assert np.array_equal(chunk_of(a), chunk_of(b))
        assert np.array_equal(twin_buf.cpu().numpy()[:twin.payload_bytes], wants[0])
        # the same through axr_pack: identical bytes
        ref = torch.full((plans[1].payload_bytes,), POISON, dtype=torch.uint8, device=gpu)
        solo = pkg.BundlePlan.create(bundles[1], align=align)
        solo.pack(ref.data_ptr(), solo.payload_bytes, stream.value)
        capi.check(lib.axr_stream_synchronize(stream))
        assert torch.equal(ref, bufs[1][:solo.payload_bytes])
        for p in rplans + [twin, solo]:
            p.close()
    finally:
        for p in plans:
            p.close()
        capi.check(lib.axr_stream_destroy(stream))


def test_payload_cache_hints_move_the_same_bytes(pkg, orc, gpu):
    """AXR_JOB_PAYLOAD_STREAMING / _CACHED only choose the cache treatment of the payload side."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(12)
    tensors = random_tensors(rng, gpu, 300, strided_every=6)
    want = orc.pack([chunk_of(t) for t in tensors], 256)
    torch.cuda.synchronize()
    for flags in (0, capi.JOB_PAYLOAD_STREAMING, capi.JOB_PAYLOAD_CACHED):
        plan = pkg.BundlePlan.create(tensors, align=256)
        buf = torch.full((plan.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu)
        outs = zeros_like_views(tensors)
        rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
        torch.cuda.synchronize()
        for _ in range(2):          # first launch (tables may ride in the arguments) and a later one
            arr = (capi.Job * 1)(capi.Job(plan._h, 0, buf.data_ptr(), plan.payload_bytes, 0, flags, 0))
            capi.check(lib.axr_submit(arr, 1, None))
            arr = (capi.Job * 1)(capi.Job(rplan._h, 1, buf.data_ptr(), plan.payload_bytes, 0, flags, 0))
            capi.check(lib.axr_submit(arr, 1, None))
            torch.cuda.synchronize()
            got = buf.cpu().numpy()
            assert np.array_equal(got[:want.size], want) and (got[want.size:] == POISON).all()
            for a, b in zip(tensors, outs):
                assert np.array_equal(chunk_of(a), chunk_of(b))
        arr = (capi.Job * 1)(capi.Job(plan._h, 0, buf.data_ptr(), plan.payload_bytes, 0, 3, 0))
        assert lib.axr_submit(arr, 1, None) == capi.AXR_ERR_INVALID      # both hints at once
        arr = (capi.Job * 1)(capi.Job(plan._h, 0, buf.data_ptr(), plan.payload_bytes, 0, 8, 0))
        assert lib.axr_submit(arr, 1, None) == capi.AXR_ERR_INVALID      # unknown bit
        plan.close()
        rplan.close()


def test_submit_refusals(pkg, gpu):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    x = torch.arange(4096, dtype=torch.uint8, device=gpu)
    plan = pkg.BundlePlan.create([x], align=1)
    buf = torch.zeros(4096, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    assert lib.axr_submit(None, 0, None) == 0
    assert lib.axr_submit(None, 1, None) == capi.AXR_ERR_INVALID
    arr = job_array(capi, [(plan, 0, buf.data_ptr(), 4095, 0)])
    assert lib.axr_submit(arr, 1, None) == capi.AXR_ERR_LENGTH
    arr = job_array(capi, [(plan, 0, buf.data_ptr(), 4096, 0), (plan, 0, buf.data_ptr(), 4096, 0)])
    assert lib.axr_submit(arr, 2, None) == capi.AXR_ERR_INVALID          # one plan twice
    host = np.arange(64, dtype=np.uint8)
    hplan = pkg.BundlePlan.create([host], align=1)
    arr = job_array(capi, [(hplan, 0, buf.data_ptr(), 64, 128)])
    assert lib.axr_submit(arr, 1, None) == capi.AXR_ERR_UNSUPPORTED      # host tensors cannot be rebased
    unbound = pkg.BundlePlan.from_header(plan.header)
    arr = job_array(capi, [(unbound, 1, buf.data_ptr(), 4096, 0)])
    assert lib.axr_submit(arr, 1, None) == capi.AXR_ERR_INVALID
    torch.cuda.synchronize()
    assert bool((buf == 0).all())                                        # nothing ran
    for p in (plan, hplan, unbound):
        p.close()


def test_tensor_delta_serves_chunks_of_one_geometry(pkg, orc, gpu):
    """One plan bound to chunk 0 of a pitched parent gathers chunks 1..3 through the
    delta, and one receiver plan scatters them into another parent."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(9)
    chunks, views, rows, cols, pitch = 4, 6, 40, 1000, 1536
    src = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, size=(chunks, views, rows, pitch),
                                        dtype=np.int16)).to(gpu)
    dst = torch.zeros_like(src)
    chunk_bytes = views * rows * pitch * 2

    def tensors_of(parent, k):
        return [parent[k, v, :, :cols] for v in range(views)]

    plan = pkg.BundlePlan.create(tensors_of(src, 0), align=256)
    rplan = pkg.BundlePlan.from_header(plan.header).bind(tensors_of(dst, 0))
    n = plan.payload_bytes
    bufs = [torch.full((n,), POISON, dtype=torch.uint8, device=gpu) for _ in range(chunks)]
    torch.cuda.synchronize()
    # every tensor of the bundle moves by the same number of bytes from chunk to chunk
    for k in range(chunks):
        arr = job_array(capi, [(plan, 0, bufs[k].data_ptr(), n, k * chunk_bytes)])
        capi.check(lib.axr_submit(arr, 1, None))
    torch.cuda.synchronize()
    view_bytes = rows * cols * 2
    for k in range(chunks):
        got = bufs[k].cpu().numpy()
        want = orc.pack([chunk_of(src[k, v, :, :cols]) for v in range(views)], 256)
        assert np.array_equal(got, want), k
    for k in range(chunks):
        arr = job_array(capi, [(rplan, 1, bufs[k].data_ptr(), n, k * chunk_bytes)])
        capi.check(lib.axr_submit(arr, 1, None))
    torch.cuda.synchronize()
    assert torch.equal(dst[:, :, :, :cols], src[:, :, :, :cols])
    assert bool((dst[:, :, :, cols:] == 0).all())
    assert view_bytes * views <= n
    # the delta also reaches the segments of a plan whose tables ride in the kernel arguments
    # on its first launch: a rebased first launch must not take that path with delta 0
    fresh = pkg.BundlePlan.create(tensors_of(src, 0), align=256)
    one = torch.full((n,), POISON, dtype=torch.uint8, device=gpu)
    arr = job_array(capi, [(fresh, 0, one.data_ptr(), n, 2 * chunk_bytes)])
    capi.check(lib.axr_submit(arr, 1, None))
    torch.cuda.synchronize()
    assert torch.equal(one, bufs[2])
    fresh.close()
    plan.close()
    rplan.close()


@pytest.mark.parametrize("head_align", [128, 16, 0])
def test_head_peel_every_misalignment(pkg, orc, gpu, head_align):
    """Contiguous tensors longer than a tile whose tensor address and payload offset take
    every residue modulo 128, in both directions and with plans used against their
    orientation (a sender's plan unpacking, a receiver's plan packing)."""
    import torch
    before = C.c_int64()
    pkg._capi.check(pkg._capi.load().axr_tune_get(b"head_align", C.byref(before)))
    pkg.tune(head_align=head_align)
    try:
        rng = np.random.default_rng(77)
        arena = torch.from_numpy(rng.integers(0, 256, size=4 << 20, dtype=np.uint8)).to(gpu)
        views, at = [], 0
        for k in range(140):
            n = int(rng.integers(2049, 9000)) if k % 3 else int(rng.integers(1, 2200))
            at += int(rng.integers(0, 3)) * 64 + (k % 128)              # every residue on the tensor side
            views.append(arena[at:at + n])
            at += n
        chunks = [chunk_of(v) for v in views]
        for align in (1, 4, 256):
            for shift in (0, 1, 77):                                      # payload base not aligned either
                plan = pkg.BundlePlan.create(views, align=align)
                n = plan.payload_bytes
                heads = [s["head"] for s in plan.segments()]
                assert max(heads) < max(head_align, 1)
                if head_align and align == 1:
                    assert max(heads) > 0                                 # the peel is in use
                buf = torch.full((n + shift + 64,), POISON, dtype=torch.uint8, device=gpu)
                plan.pack(buf.data_ptr() + shift, n)
                torch.cuda.synchronize()
                got = buf.cpu().numpy()
                assert np.array_equal(got[shift:shift + n], orc.pack(chunks, align)), (align, shift)
                assert (got[:shift] == POISON).all() and (got[shift + n:] == POISON).all()
                # receiver's plan (anchored on the tensor side) scatters
                out_arena = torch.full_like(arena, POISON)
                outs = [out_arena[v.data_ptr() - arena.data_ptr():][:v.numel()] for v in views]
                rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
                rplan.unpack(buf.data_ptr() + shift, n)
                torch.cuda.synchronize()
                mask = torch.zeros_like(arena, dtype=torch.bool)
                for v in views:
                    o = v.data_ptr() - arena.data_ptr()
                    mask[o:o + v.numel()] = True
                assert torch.equal(out_arena[mask], arena[mask])
                assert bool((out_arena[~mask] == POISON).all())           # nothing beside the tensors
                # against orientation: the receiver's plan packs, the sender's plan unpacks
                buf2 = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
                rplan.pack(buf2.data_ptr(), n)
                out2 = torch.full_like(arena, POISON)
                outs2 = [out2[v.data_ptr() - arena.data_ptr():][:v.numel()] for v in views]
                plan2 = pkg.BundlePlan.create(outs2, align=align)
                plan2.unpack(buf.data_ptr() + shift, n)
                torch.cuda.synchronize()
                assert np.array_equal(buf2.cpu().numpy()[:n], orc.pack(chunks, align))
                assert torch.equal(out2[mask], arena[mask]) and bool((out2[~mask] == POISON).all())
                for p in (plan, rplan, plan2):
                    p.close()
    finally:
        pkg.tune(head_align=before.value)


@pytest.mark.parametrize("align", [1, 256])
def test_tables_built_on_the_device_match_the_oracle(pkg, orc, gpu, align):
    """Bundles of contiguous device tensors whose tables a kernel expands from one record per
    tensor ("device_tables"): every count from one tensor to several per thread of the
    expanding workgroup, empty tensors in between, tensors of many thousand tiles, odd
    addresses; packed bytes against the oracle, unpack round trip, and the same plans with
    host-built tables."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    before = C.c_int64()
    capi.check(lib.axr_tune_get(b"device_tables", C.byref(before)))
    rng = np.random.default_rng(99 + align)
    arena = torch.from_numpy(rng.integers(0, 256, size=96 << 20, dtype=np.uint8)).to(gpu)
    cases = []
    for count, lo, hi in ((1, 5000, 5001), (3, 1, 40), (70, 1, 9000), (1023, 1, 3000), (1025, 1, 3000),
                          (2500, 1, 12000), (5, 3 << 20, 9 << 20), (40, 1, 1 << 20)):
        views, at = [], int(rng.integers(0, 64))
        for k in range(count):
            n = 0 if (count > 3 and k % 17 == 5) else int(rng.integers(lo, hi))
            at += int(rng.integers(0, 130))
            views.append(arena[at:at + n])
            at += n
        assert at <= arena.numel()
        cases.append(views)
    try:
        for views in cases:
            want = orc.pack([chunk_of(v) for v in views], align)
            for device_tables in (1, 0):
                pkg.tune(device_tables=device_tables)
                plan = pkg.BundlePlan.create(views, align=align)
                n = plan.payload_bytes
                buf = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
                for _ in range(2):      # the second launch reuses the tables
                    plan.pack(buf.data_ptr(), n)
                torch.cuda.synchronize()
                got = buf.cpu().numpy()
                assert np.array_equal(got[:n], want), (len(views), device_tables)
                assert (got[n:] == POISON).all()
                out_arena = torch.full_like(arena, POISON)
                outs = [out_arena[v.data_ptr() - arena.data_ptr():][:v.numel()] for v in views]
                rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
                rplan.unpack(buf.data_ptr(), n)
                torch.cuda.synchronize()
                mask = torch.zeros_like(arena, dtype=torch.bool)
                for v in views:
                    o = v.data_ptr() - arena.data_ptr()
                    mask[o:o + v.numel()] = True
                assert torch.equal(out_arena[mask], arena[mask])
                assert bool((out_arena[~mask] == POISON).all())
                # asking for the tables on the host afterwards gives the same launch geometry
                # and the next launch still moves the same bytes
                info = plan.launch_info()
                assert info["tiles"] > 0 or n == 0
                buf.fill_(POISON)
                plan.pack(buf.data_ptr(), n)
                torch.cuda.synchronize()
                assert np.array_equal(buf.cpu().numpy()[:n], want)
                plan.close()
                rplan.close()
        # a strided view among them: the host builds the tables, same result
        pkg.tune(device_tables=1)
        mixed = cases[2][:20] + [arena[:4096].view(torch.int16).reshape(32, 64)[:, :20]] + cases[2][20:40]
        plan = pkg.BundlePlan.create(mixed, align=align)
        buf = torch.full((plan.payload_bytes,), POISON, dtype=torch.uint8, device=gpu)
        plan.pack(buf.data_ptr(), plan.payload_bytes)
        torch.cuda.synchronize()
        assert np.array_equal(buf.cpu().numpy(), orc.pack([chunk_of(v) for v in mixed], align))
        plan.close()
    finally:
        pkg.tune(device_tables=before.value)


def test_many_small_bundles_in_one_call(pkg, orc, gpu):
    """Forty small bundles (the size of an RPC argument list) gathered by one axr_submit and
    scattered by another: sixteen jobs share a launch, so the call is three launches, and
    every bundle equals the oracle's pack and comes back whole."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(77)
    bundles = [random_tensors(rng, gpu, int(rng.integers(1, 9)), lo=64, hi=70000) for _ in range(40)]
    torch.cuda.synchronize()
    plans = [pkg.BundlePlan.create(t, align=256) for t in bundles]
    bufs = [torch.full((p.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu) for p in plans]
    outs = [zeros_like_views(t) for t in bundles]
    rplans = [pkg.BundlePlan.from_header(p.header).bind(o) for p, o in zip(plans, outs)]
    torch.cuda.synchronize()
    try:
        arr = job_array(capi, [(p, 0, b.data_ptr(), p.payload_bytes, 0) for p, b in zip(plans, bufs)])
        capi.check(lib.axr_submit(arr, len(plans), None))
        arr = job_array(capi, [(r, 1, b.data_ptr(), p.payload_bytes, 0) for r, p, b in zip(rplans, plans, bufs)])
        capi.check(lib.axr_submit(arr, len(plans), None))
        capi.check(lib.axr_device_synchronize())
        for tensors, p, b, o in zip(bundles, plans, bufs, outs):
            got = b.cpu().numpy()
            assert np.array_equal(got[:p.payload_bytes], orc.pack([chunk_of(t) for t in tensors], 256))
            assert (got[p.payload_bytes:] == POISON).all()
            for x, y in zip(tensors, o):
                assert np.array_equal(chunk_of(x), chunk_of(y))
    finally:
        for p in plans + rplans:
            p.close()


@pytest.mark.parametrize("device_tables", [1, 0])
def test_streaming_geometry_for_payloads_beyond_the_cache(pkg, gpu, device_tables):
    """A payload between 256 MiB and 1 GiB moves in 1 KiB tiles, one wavefront per workgroup
    (tables built on the device and on the host).  6000 contiguous tensors of odd lengths around
    64 KiB at odd addresses, tight layout: the packed bytes are the tensors' concatenation,
    compared on the device, and an unpack into fresh memory gives the tensors back with the
    bytes between them untouched."""
    import torch
    rng = np.random.default_rng(12)
    sizes = rng.integers(50_000, 80_000, size=6000)
    gaps = rng.integers(0, 100, size=6000)
    total = int(sizes.sum() + gaps.sum()) + 64
    g = torch.Generator(device=gpu)
    g.manual_seed(7)
    arena = torch.randint(0, 256, (total,), dtype=torch.uint8, device=gpu, generator=g)
    views, at = [], 3
    for n, gap in zip(sizes, gaps):
        at += int(gap)
        views.append(arena[at:at + int(n)])
        at += int(n)
    before = C.c_int64()
    pkg._capi.check(pkg._capi.load().axr_tune_get(b"device_tables", C.byref(before)))
    pkg.tune(device_tables=device_tables)
    try:
        plan = pkg.BundlePlan.create(views, align=1)
        n = plan.payload_bytes
        assert (256 << 20) < n <= (1 << 30) and n == int(sizes.sum())
        buf = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
        plan.pack(buf.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
        info = plan.launch_info()
        assert info["tile_bytes"] == 1024 and info["threads_per_workgroup"] == 64
        assert torch.equal(buf[:n], torch.cat(views)) and bool((buf[n:] == POISON).all())
        out_arena = torch.full_like(arena, POISON)
        outs = [out_arena[v.data_ptr() - arena.data_ptr():][:v.numel()] for v in views]
        rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
        rplan.unpack(buf.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
        assert rplan.launch_info()["tile_bytes"] == 1024
        mask = torch.zeros(total, dtype=torch.bool, device=gpu)
        for v in views:
            o = v.data_ptr() - arena.data_ptr()
            mask[o:o + v.numel()] = True
        assert torch.equal(out_arena[mask], arena[mask]) and bool((out_arena[~mask] == POISON).all())
        rplan.close()
        plan.close()
    finally:
        pkg.tune(device_tables=before.value)


@pytest.mark.parametrize("interleave", [2, 0])
def test_two_jobs_of_equal_grids_take_workgroups_in_turn(pkg, orc, gpu, interleave):
    """Two bundles of one geometry (the same sizes at other addresses) in one launch: the pack
    of one and the unpack of the other, payloads streaming, with the jobs' workgroups
    interleaved ("submit_interleave" = 2; by default only payloads beyond the cache size do
    that) and in one range each; the same bytes either way."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(77)
    sizes = [int(x) for x in np.exp(rng.uniform(np.log(16), np.log(90000), size=500))]
    sets = []
    for _ in range(2):
        sets.append([torch.from_numpy(rng.integers(0, 256, size=n, dtype=np.uint8)).to(gpu) for n in sizes])
    plans = [pkg.BundlePlan.create(s, align=256) for s in sets]
    n = plans[0].payload_bytes
    assert len({p.launch_info()["workgroups"] for p in plans}) == 1
    bufs = [torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu) for _ in range(2)]
    want = orc.pack([chunk_of(t) for t in sets[0]], 256)
    # the second bundle's payload is packed first, on its own, and unpacked inside the joint launch
    plans[1].pack(bufs[1].data_ptr(), n)
    outs = [torch.zeros_like(t) for t in sets[1]]
    rplan = pkg.BundlePlan.from_header(plans[1].header).bind(outs)
    torch.cuda.synchronize()
    before = C.c_int64()
    capi.check(lib.axr_tune_get(b"submit_interleave", C.byref(before)))
    pkg.tune(submit_interleave=interleave)
    try:
        arr = job_array(capi, [(plans[0], 0, bufs[0].data_ptr(), n, 0), (rplan, 1, bufs[1].data_ptr(), n, 0)])
        for k in range(2):          # interleaving is for payloads that stream: ask for that treatment
            arr[k].flags = capi.JOB_PAYLOAD_STREAMING
        capi.check(lib.axr_submit(arr, 2, None))
        torch.cuda.synchronize()
    finally:
        pkg.tune(submit_interleave=before.value)
    got = bufs[0].cpu().numpy()
    assert np.array_equal(got[:n], want) and (got[n:] == POISON).all()
    for o, t in zip(outs, sets[1]):
        assert torch.equal(o, t)
    for p in plans + [rplan]:
        p.close()


def test_two_jobs_whose_wavefronts_take_several_tiles(pkg, orc, gpu):
    """A launch of two jobs normally finds what it needs for its first table reads in the
    preloaded kernel arguments; plans whose wavefronts walk several tiles ("max_waves") read
    their descriptors instead.  Same bytes."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(78)
    before = C.c_int64()
    capi.check(lib.axr_tune_get(b"max_waves", C.byref(before)))
    pkg.tune(max_waves=96)
    try:
        sets = [random_tensors(rng, gpu, 300, strided_every=7) for _ in range(2)]
        plans = [pkg.BundlePlan.create(s, align=64) for s in sets]
        bufs = [torch.full((p.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu) for p in plans]
        plans[1].pack(bufs[1].data_ptr(), plans[1].payload_bytes)
        info = plans[0].launch_info()
        assert info["tiles"] > 96 * (info["threads_per_workgroup"] // 64) or info["workgroups"] * (info["threads_per_workgroup"] // 64) < info["tiles"]
        outs = zeros_like_views(sets[1])
        rplan = pkg.BundlePlan.from_header(plans[1].header).bind(outs)
        torch.cuda.synchronize()
        arr = job_array(capi, [(plans[0], 0, bufs[0].data_ptr(), plans[0].payload_bytes, 0),
                               (rplan, 1, bufs[1].data_ptr(), plans[1].payload_bytes, 0)])
        capi.check(lib.axr_submit(arr, 2, None))
        torch.cuda.synchronize()
    finally:
        pkg.tune(max_waves=before.value)
    n = plans[0].payload_bytes
    got = bufs[0].cpu().numpy()
    assert np.array_equal(got[:n], orc.pack([chunk_of(t) for t in sets[0]], 64)) and (got[n:] == POISON).all()
    for o, t in zip(outs, sets[1]):
        assert np.array_equal(chunk_of(o), chunk_of(t))      # bytes: the random bit patterns hold NaNs
    for p in plans + [rplan]:
        p.close()


def test_a_joint_launch_in_a_hip_graph(pkg, orc, gpu):
    """axr_submit under stream capture: the pack of one bundle and the unpack of another share
    one captured launch (the step a worker repeats).  Plans that were not prepared are refused
    and record nothing; the graph is replayed several times with eager work and
    synchronisations in between, every replay checked against the oracle."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(404)
    a = random_tensors(rng, gpu, 300)
    b = random_tensors(rng, gpu, 300)
    b_out = zeros_like_views(b)
    plan_a = pkg.BundlePlan.create(a, align=256)
    plan_b = pkg.BundlePlan.create(b, align=256)
    rplan_b = pkg.BundlePlan.from_header(plan_b.header).bind(b_out)
    buf_a = torch.full((plan_a.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu)
    buf_b = torch.full((plan_b.payload_bytes + 64,), POISON, dtype=torch.uint8, device=gpu)
    side = torch.cuda.Stream()
    jobs = job_array(capi, [(plan_a, 0, buf_a.data_ptr(), plan_a.payload_bytes, 0),
                            (rplan_b, 1, buf_b.data_ptr(), plan_b.payload_bytes, 0)])
    refused = torch.cuda.CUDAGraph()
    with torch.cuda.graph(refused, stream=side):
        rc = lib.axr_submit(jobs, 2, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == capi.AXR_ERR_INVALID
    del refused
    plan_a.prepare()
    rplan_b.prepare()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        capi.check(lib.axr_submit(jobs, 2, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    try:
        for replay in range(4):
            for t in a:
                t.view(torch.uint8).add_(replay + 1)
            for t in b:
                t.view(torch.uint8).add_(2 * replay + 1)
            for o in b_out:
                o.zero_()
            buf_a.fill_(POISON)
            plan_b.pack(buf_b.data_ptr(), plan_b.payload_bytes)          # eager, on the default stream
            torch.cuda.synchronize()
            want_a = orc.pack([chunk_of(t) for t in a], 256)
            graph.replay()
            torch.cuda.synchronize()
            got = buf_a.cpu().numpy()
            assert np.array_equal(got[:plan_a.payload_bytes], want_a), replay
            assert (got[plan_a.payload_bytes:] == POISON).all(), replay
            for o, t in zip(b_out, b):
                assert np.array_equal(chunk_of(o), chunk_of(t)), replay
    finally:
        del graph
        for p in (plan_a, plan_b, rplan_b):
            p.close()
