"""Short tensors that share wavefronts (group tiles) against the CPU oracle, through the C ABI.

A bundle of many short contiguous tensors is moved by wavefronts that each take several
whole tensors.  Bit-exact against the oracle's pack / unpack in both layouts, with every
length from 1 byte up, odd source and destination offsets, a shifted payload base, and
nothing written outside the tensors and the payload."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xCD


def short_tensors(rng, gpu, sizes, max_gap=33):
    """Byte tensors of the given sizes carved out of one arena at arbitrary byte offsets."""
    import torch
    total = sum(sizes) + max_gap * len(sizes) + 64
    arena = torch.from_numpy(rng.integers(0, 256, size=total, dtype=np.uint8)).to(gpu)
    host = arena.cpu().numpy()
    tensors, chunks, at = [], [], 0
    for n in sizes:
        at += int(rng.integers(0, max_gap))
        tensors.append(arena[at:at + n])
        chunks.append(host[at:at + n])
        at += n
    return arena, tensors, chunks


def pack_checked(pkg, tensors, align, gpu, shift=0, plan=None):
    import torch
    plan = plan or pkg.BundlePlan.create(tensors, align=align)
    n = plan.payload_bytes
    buf = torch.full((n + shift + 64,), POISON, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    plan.pack(buf.data_ptr() + shift, n, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert (host[:shift] == POISON).all() and (host[shift + n:] == POISON).all()
    return host[shift:shift + n], plan, buf


def unpack_checked(pkg, plan_header, payload_ptr, payload_bytes, sizes, chunks, rng, gpu, rplan=None):
    """Unpack into destinations at fresh odd offsets; bytes between them must stay untouched."""
    import torch
    dst_arena = torch.full((sum(sizes) + 40 * len(sizes) + 64,), 0xEE, dtype=torch.uint8, device=gpu)
    outs, spans, at = [], [], 0
    for n in sizes:
        at += int(rng.integers(0, 33))
        outs.append(dst_arena[at:at + n])
        spans.append((at, n))
        at += n
    if rplan is None:
        rplan = pkg.BundlePlan.from_header(plan_header).bind(outs)
    else:
        rplan.bind(outs)
    torch.cuda.synchronize()
    rplan.unpack(payload_ptr, payload_bytes)
    torch.cuda.synchronize()
    got = dst_arena.cpu().numpy()
    expect = np.full(got.size, 0xEE, np.uint8)
    for (o, n), c in zip(spans, chunks):
        expect[o:o + n] = c
    assert np.array_equal(got, expect)
    return rplan


@pytest.mark.parametrize("seed", [0, 1])
def test_every_short_length_in_every_layout(pkg, orc, gpu, seed):
    rng = np.random.default_rng(seed)
    sizes = list(range(0, 130)) + [int(x) for x in rng.integers(1, 520, size=900)] + [700, 1023, 1024, 5000, 3, 1]
    rng.shuffle(sizes)
    arena, tensors, chunks = short_tensors(rng, gpu, sizes)
    for align, shift in ((1, 0), (1, 5), (2, 0), (16, 3), (64, 0), (256, 0), (256, 9), (4096, 0)):
        got, plan, buf = pack_checked(pkg, tensors, align, gpu, shift)
        assert np.array_equal(got, orc.pack(chunks, align)), (align, shift)
        modes = {s["mode"] for s in plan.segments()}
        assert (6 in modes) == (align != 4096)
        unpack_checked(pkg, plan.header, buf.data_ptr() + shift, plan.payload_bytes, sizes, chunks, rng, gpu)


def test_groups_off_gives_the_same_bytes(pkg, orc, gpu):
    rng = np.random.default_rng(5)
    sizes = [int(x) for x in rng.integers(1, 400, size=3000)]
    arena, tensors, chunks = short_tensors(rng, gpu, sizes)
    got, plan, _ = pack_checked(pkg, tensors, 1, gpu)
    pkg.tune(group_bytes=0)
    try:
        plain, plan0, _ = pack_checked(pkg, tensors, 1, gpu)
        assert plan0.launch_info()["tiles"] == 3000
    finally:
        pkg.tune(group_bytes=512)
    assert plan.launch_info()["tiles"] < 3000 // 4
    assert np.array_equal(got, plain) and np.array_equal(got, orc.pack(chunks, 1))


def test_sender_plan_unpacks_and_receiver_plan_packs(pkg, orc, gpu):
    """The zero slots behind a member belong to the pack direction only: a plan made by
    axr_plan_create also scatters, a plan made from a header also gathers (gaps zeroed)."""
    import torch
    rng = np.random.default_rng(6)
    sizes = [int(x) for x in rng.integers(1, 300, size=500)]
    arena, tensors, chunks = short_tensors(rng, gpu, sizes)
    got, plan, buf = pack_checked(pkg, tensors, 256, gpu)
    want = orc.pack(chunks, 256)
    assert np.array_equal(got, want)
    # scatter with the sender's own plan, rebound to new destinations
    unpack_checked(pkg, None, buf.data_ptr(), plan.payload_bytes, sizes, chunks, rng, gpu,
                   rplan=pkg.BundlePlan.create(tensors, align=256))
    # gather with a plan decoded from the header
    rplan = pkg.BundlePlan.from_header(plan.header).bind(tensors)
    again, _, _ = pack_checked(pkg, tensors, 256, gpu, plan=rplan)
    assert np.array_equal(again, want)


@pytest.mark.parametrize("align", [256, 1])
def test_small_segment_workload_full(pkg, orc, gpu, align):
    """65,536 contiguous tensors of 8 to 512 bytes in five dtypes (about 8 MB)."""
    import torch
    from execution_ucx_amd import workloads
    spec = workloads.mixed_bundle(n=65536, lo=8, hi=512, seed=3)
    arena, _ = workloads.materialize_mixed(spec, gpu, seed=3)
    host = arena.cpu().numpy()
    chunks = [host[s.arena_offset:s.arena_offset + s.nbytes] for s in spec.segments]
    views = workloads.mixed_views(spec, arena.data_ptr())
    plan = pkg.BundlePlan.create(views, align=align)
    got, plan, buf = pack_checked(pkg, None, align, gpu, plan=plan)
    want = orc.pack(chunks, align)
    assert np.array_equal(got, want)
    info = plan.launch_info()
    assert info["tiles"] < 65536 // 4          # wavefronts follow the payload, not the tensor count
    dst = torch.zeros_like(arena)
    rplan = pkg.BundlePlan.from_header(plan.header).bind(workloads.mixed_views(spec, dst.data_ptr()))
    torch.cuda.synchronize()
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    back = dst.cpu().numpy()
    expect = np.zeros_like(back)
    for s, c in zip(spec.segments, chunks):
        expect[s.arena_offset:s.arena_offset + s.nbytes] = c
    assert np.array_equal(back, expect)


def test_grouped_plans_in_submit_with_deltas_and_without_allocation(pkg, orc, gpu):
    """Group tiles through axr_submit (two jobs in one launch, one of them moved by a tensor
    address delta) and through axr_pack_noalloc (tables in the static area)."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(8)
    sizes = [int(x) for x in rng.integers(1, 500, size=2000)]
    total = sum(sizes) + 33 * len(sizes) + 64
    two = torch.from_numpy(rng.integers(0, 256, size=2 * total, dtype=np.uint8)).to(gpu)
    host = two.cpu().numpy()
    tensors, chunks_a, chunks_b, at = [], [], [], 0
    for n in sizes:
        at += int(rng.integers(0, 33))
        tensors.append(two[at:at + n])
        chunks_a.append(host[at:at + n])
        chunks_b.append(host[total + at:total + at + n])
        at += n
    plan_a = pkg.BundlePlan.create(tensors, align=16)
    plan_b = pkg.BundlePlan.create(tensors, align=16)
    n = plan_a.payload_bytes
    pay = torch.full((2, n + 64), POISON, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    jobs = (capi.Job * 2)(capi.Job(plan_a._h, 0, pay[0].data_ptr(), n, 0),
                          capi.Job(plan_b._h, 0, pay[1].data_ptr(), n, total))
    capi.check(lib.axr_submit(jobs, 2, None))
    torch.cuda.synchronize()
    got = pay.cpu().numpy()
    assert np.array_equal(got[0, :n], orc.pack(chunks_a, 16))
    assert np.array_equal(got[1, :n], orc.pack(chunks_b, 16))
    assert (got[:, n:] == POISON).all()
    # no allocation: 2000 members do not fit the kernel arguments, the static area takes them
    assert plan_a.launch_info()["table_bytes"] > 3584
    out = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    capi.check(lib.axr_pack_noalloc(plan_a._h, out.data_ptr(), n, None))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy()[:n], orc.pack(chunks_a, 16))


@pytest.mark.parametrize("seed", range(6))
def test_random_mixtures_of_short_long_strided_and_empty_tensors(pkg, orc, gpu, seed):
    """Group tiles next to ordinary and strided segments in random order: short (1-1099 B),
    long (1.1-40 KB), pitched 2-D views and empty tensors at odd offsets, a random alignment
    and a shifted payload base; pack against the oracle, unpack into fresh tensors."""
    import torch
    rng = np.random.default_rng(10_000 + seed)
    tensors, chunks = [], []
    for k in rng.integers(0, 10, size=int(rng.integers(50, 400))):
        if k < 8:
            nb = int(rng.integers(1, 1100)) if k < 6 else int(rng.integers(1100, 40000))
            raw = torch.from_numpy(rng.integers(0, 256, size=nb + 32, dtype=np.uint8)).to(gpu)
            o = int(rng.integers(0, 32))
            t = raw[o:o + nb]
        elif k == 8:
            rows, cols, pitch = int(rng.integers(1, 20)), int(rng.integers(1, 3000)), 3100
            raw = torch.from_numpy(rng.integers(0, 256, size=rows * pitch, dtype=np.uint8)).to(gpu)
            t = raw.reshape(rows, pitch)[:, :cols]
        else:
            t = torch.empty(0, dtype=torch.uint8, device=gpu)
        tensors.append(t)
        chunks.append(t.contiguous().reshape(-1).cpu().numpy())
    align = int(rng.choice([1, 2, 16, 64, 256, 1024]))
    shift = int(rng.integers(0, 16))
    got, plan, buf = pack_checked(pkg, tensors, align, gpu, shift=shift)
    assert np.array_equal(got, orc.pack(chunks, align))
    outs = [torch.full_like(t, 0xEE) if t.is_contiguous() else
            torch.full((t.shape[0], 3100), 0xEE, dtype=torch.uint8, device=gpu)[:, :t.shape[1]] for t in tensors]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    torch.cuda.synchronize()
    rplan.unpack(buf.data_ptr() + shift, plan.payload_bytes)
    torch.cuda.synchronize()
    for o, c in zip(outs, chunks):
        assert np.array_equal(o.contiguous().reshape(-1).cpu().numpy(), c)
    rplan.close()
    plan.close()


@pytest.mark.parametrize("align", [1, 64])
def test_more_than_a_million_tensors(pkg, gpu, align):
    """1.2 million tensors of 0-48 bytes (and a few of 100 KB) in one bundle: beyond the 2^20
    tensors up to which the device builds the tables, with tensor, tile and table counts that no
    longer fit 16 or 20 bits anywhere.  The expected payload is built with numpy index
    arithmetic (offset rule of the aligned layout: every tensor starts at the next multiple of
    `align`), the descriptors are written as one numpy record array, through the C ABI."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    record = np.dtype([("data", "<u8"), ("device_type", "<i4"), ("device_id", "<i4"), ("ndim", "<i4"),
                       ("code", "u1"), ("bits", "u1"), ("lanes", "<u2"), ("shape", "<u8"),
                       ("strides", "<u8"), ("byte_offset", "<u8")])
    assert record.itemsize == C.sizeof(capi.Tensor)
    n = 1_200_000
    rng = np.random.default_rng(align)
    sizes = rng.integers(1, 49, size=n).astype(np.int64)
    sizes[::150_000] = rng.integers(50_000, 200_000, size=len(sizes[::150_000]))
    sizes[rng.integers(0, n, size=n // 50)] = 0
    starts = np.cumsum(sizes + rng.integers(0, 3, size=n) * 7) - sizes
    arena_bytes = int(starts[-1] + sizes[-1] + 64)
    src = torch.randint(0, 256, (arena_bytes,), dtype=torch.uint8, device=gpu)
    dst = torch.full((arena_bytes,), 0x55, dtype=torch.uint8, device=gpu)

    def descriptors(base):
        d = np.zeros(n, record)
        d["data"], d["device_type"], d["ndim"], d["code"], d["bits"], d["lanes"] = base + starts, 10, 1, 1, 8, 1
        d["shape"] = sizes.ctypes.data + 8 * np.arange(n, dtype=np.uint64)
        return d, C.cast(C.c_void_p(d.ctypes.data), C.POINTER(capi.Tensor))

    _keep_s, sd = descriptors(src.data_ptr())
    _keep_d, dd = descriptors(dst.data_ptr())
    plan, rplan = C.c_void_p(), C.c_void_p()
    capi.check(lib.axr_plan_create(sd, n, align, 0, C.byref(plan)))
    try:
        nbytes = C.c_uint64()
        capi.check(lib.axr_plan_payload_bytes(plan, C.byref(nbytes)))
        padded = (sizes + align - 1) & ~(align - 1)
        offsets = np.cumsum(padded) - padded
        total = int(offsets[-1] + sizes[-1])
        assert nbytes.value == total
        payload = torch.full((total + 64,), POISON, dtype=torch.uint8, device=gpu)
        torch.cuda.synchronize()
        capi.check(lib.axr_pack(plan, payload.data_ptr(), total, None))
        header, header_bytes = C.c_void_p(), C.c_size_t()
        capi.check(lib.axr_plan_header(plan, C.byref(header), C.byref(header_bytes)))
        capi.check(lib.axr_plan_from_header_bind(header, header_bytes.value, dd, n, C.byref(rplan)))
        capi.check(lib.axr_unpack(rplan, payload.data_ptr(), total, None))
        torch.cuda.synchronize()
        host = src.cpu().numpy()
        filled = sizes > 0
        within = np.arange(int(sizes.sum())) - np.repeat(np.cumsum(sizes[filled]) - sizes[filled], sizes[filled])
        from_arena = np.repeat(starts[filled], sizes[filled]) + within
        to_payload = np.repeat(offsets[filled], sizes[filled]) + within
        want = np.zeros(total, np.uint8)
        want[to_payload] = host[from_arena]
        got = payload.cpu().numpy()
        assert np.array_equal(got[:total], want)
        assert (got[total:] == POISON).all()
        expect = np.full(arena_bytes, 0x55, np.uint8)
        expect[from_arena] = host[from_arena]
        assert np.array_equal(dst.cpu().numpy(), expect)
    finally:
        capi.check(lib.axr_plan_free(plan))
        if rplan:
            capi.check(lib.axr_plan_free(rplan))
