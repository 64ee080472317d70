"""Parity of the HIP pack/unpack path with the CPU oracle, through the C ABI.

Bit-exact is the bar everywhere: this is byte movement.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xCD


def tbytes(t):
    """Bytes of a torch tensor's C-order element sequence, as numpy uint8."""
    import torch
    if t.numel() == 0:
        return np.zeros(0, np.uint8)
    c = torch.empty(t.shape, dtype=t.dtype, device=t.device)   # compact even when contiguous() is a no-op
    c.copy_(t)
    return c.reshape(-1).view(torch.uint8).cpu().numpy()


def device_bytes(n, gpu, fill=POISON):
    import torch
    return torch.full((max(n, 1),), fill, dtype=torch.uint8, device=gpu)


def run_pack(pkg, tensors, align, gpu, base_shift=0):
    """Pack and return (payload bytes as numpy, plan)."""
    import torch
    plan = pkg.BundlePlan.create(tensors, align=align)
    n = plan.payload_bytes
    buf = device_bytes(n + base_shift + 64, gpu)
    # on the stream that produced the tensors: ordered by the stream itself, and the copy to
    # the host below waits for it
    plan.pack(buf.data_ptr() + base_shift, n, torch.cuda.current_stream().cuda_stream)
    host = buf.cpu().numpy()
    # nothing outside [shift, shift + n) may be written
    assert (host[:base_shift] == POISON).all() and (host[base_shift + n:] == POISON).all()
    return host[base_shift:base_shift + n], plan, buf


def rand_bytes_tensor(rng, nbytes, gpu):
    import torch
    return torch.from_numpy(rng.integers(0, 256, size=nbytes, dtype=np.uint8)).to(gpu)


# ------------------------------------------------------------------ reference KATs on device

@pytest.mark.parametrize("lens", [(256, 512, 300), (512 * 1024, 256 * 1024, 800 * 1024)])
def test_iov_to_contig_kat(pkg, orc, gpu, lens):
    import torch
    segs, cursor = [], 0
    for n in lens:
        segs.append(((np.arange(n) + cursor) % 256).astype(np.uint8))
        cursor += n
    dev = [torch.from_numpy(s).to(gpu) for s in segs]
    got, plan, buf = run_pack(pkg, dev, 1, gpu)
    expected = (np.arange(sum(lens)) % 256).astype(np.uint8)
    assert np.array_equal(got, expected)
    assert np.array_equal(got, orc.pack(segs, 1))
    # iov -> iov: scatter into receiver buffers of the same lengths
    outs = [torch.zeros(n, dtype=torch.uint8, device=gpu) for n in lens]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    for s, o in zip(segs, outs):
        assert np.array_equal(o.cpu().numpy(), s)


def test_process_round_trip_kat(pkg, orc, gpu):
    # send float(i % 256), divide by two on the device, expect (i % 256) / 2 exactly
    import torch
    lib = pkg._capi.load()
    for n in (32, 1 << 20):
        x = torch.from_numpy((np.arange(4 * n) % 256).astype(np.float32)).to(gpu)
        parts = list(x.chunk(4))
        got, plan, buf = run_pack(pkg, parts, 1, gpu)
        assert np.array_equal(got.view(np.float32), (np.arange(4 * n) % 256).astype(np.float32))
        pkg._capi.check(lib.axr_divide_by_two(buf.data_ptr(), 4 * n, None))
        torch.cuda.synchronize()
        back = buf.cpu().numpy()[:16 * n].view(np.float32)
        assert np.array_equal(back, (np.arange(4 * n) % 256).astype(np.float32) / 2)
        assert np.array_equal(back, orc.divide_by_two((np.arange(4 * n) % 256).astype(np.float32)))


def test_buffer_to_vec_kat(pkg, gpu):
    # fp32[2048] = i split four ways keeps the global index (axon_worker_test.cpp:1656-1774)
    import torch
    f = torch.arange(2048, dtype=torch.float32, device=gpu)
    outs = [torch.zeros(512, dtype=torch.float32, device=gpu) for _ in range(4)]
    plan = pkg.BundlePlan.create(outs, align=1)
    assert plan.payload_bytes == 8192
    plan.unpack(f.data_ptr(), 8192)
    torch.cuda.synchronize()
    for k, o in enumerate(outs):
        assert torch.equal(o, torch.arange(512 * k, 512 * (k + 1), dtype=torch.float32, device=gpu))
    views = plan.split(f.data_ptr(), 8192)
    assert views == [(f.data_ptr() + 2048 * k, 2048) for k in range(4)]


def test_golden_small_bundle(pkg, gpu):
    """Committed vectors (tests/golden/small_bundle_v1.json): chunks -> packed bytes."""
    import json
    import os
    import torch
    fx = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "small_bundle_v1.json")))
    chunks = [np.frombuffer(bytes.fromhex(h), dtype=np.uint8) for h in fx["chunks_hex"]]
    dev = [torch.from_numpy(c.copy()).to(gpu) for c in chunks]
    for align, hexed in fx["packed"].items():
        got, plan, buf = run_pack(pkg, dev, int(align), gpu)
        assert got.tobytes().hex() == hexed
        outs = [torch.full((c.size,), 0x11, dtype=torch.uint8, device=gpu) for c in chunks]
        pkg.BundlePlan.from_header(plan.header).bind(outs).unpack(buf.data_ptr(), plan.payload_bytes)
        torch.cuda.synchronize()
        for o, c in zip(outs, chunks):
            assert np.array_equal(o.cpu().numpy(), c)


# ------------------------------------------------------------------ config 1: host tensors

def test_c1_host_bundle(pkg, orc, gpu):
    import torch
    from execution_ucx_amd import workloads
    srcs = workloads.host_bundle_c1(seed=0)
    got, plan, buf = run_pack(pkg, srcs, 1, gpu)
    assert plan.payload_bytes == 4 << 20
    want = orc.pack([s.view(np.uint8) for s in srcs], 1)
    assert np.array_equal(got, want)
    outs = [np.zeros_like(s) for s in srcs]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    info = rplan.launch_info()
    assert info["host_copies"] == 64 and info["host_chunks"] == 1    # one staged device copy
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    for a, b in zip(srcs, outs):
        assert a.tobytes() == b.tobytes()


def test_host_tensors_staged_with_device_tensors(pkg, orc, gpu):
    """Host (kDLCPU) tensors interleaved with device tensors: neighbouring host
    pieces share one staged device copy, a 20 MiB host tensor is cut over several
    staging blocks, strided host views move piece by piece; the plan is used twice
    so that the staging blocks are reused while their last copy may be in flight."""
    import torch
    rng = np.random.default_rng(11)
    big = rng.integers(0, 256, size=20 * (1 << 20) + 12345, dtype=np.uint8)
    mat = rng.integers(0, 2 ** 31, size=(64, 300), dtype=np.int32)
    small = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in (1, 255, 256, 70000)]
    dev = [rand_bytes_tensor(rng, n, gpu) for n in (4096, 100, 3 << 20)]
    tensors = [small[0], dev[0], small[1], small[2], big, dev[1], mat[::2, 10:250], small[3], dev[2]]

    def chunk_of(t):
        return tbytes(t) if isinstance(t, torch.Tensor) else np.ascontiguousarray(t).view(np.uint8).reshape(-1)

    chunks = [chunk_of(t) for t in tensors]
    for align in (256, 1):
        plan = pkg.BundlePlan.create(tensors, align=align)
        info = plan.launch_info()
        assert info["host_copies"] == 4 + 3 + 32                 # 20 MiB in three pieces, 32 matrix rows
        assert 3 <= info["host_chunks"] < info["host_copies"]
        n = plan.payload_bytes
        for repeat in range(2):
            buf = device_bytes(n + 64, gpu)
            plan.pack(buf.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            host = buf.cpu().numpy()
            assert np.array_equal(host[:n], orc.pack(chunks, align)), (align, repeat)
            assert (host[n:] == POISON).all()
        outs = []
        for t in tensors:
            if isinstance(t, torch.Tensor):
                outs.append(torch.zeros_like(t))
            else:
                outs.append(np.zeros(t.shape, dtype=t.dtype))
        rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
        for repeat in range(2):
            for o in outs:
                if isinstance(o, torch.Tensor):
                    o.zero_()
                else:
                    o[...] = 0
            rplan.unpack(buf.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            for o, c in zip(outs, chunks):
                assert np.array_equal(chunk_of(o), c), (align, repeat)


# ------------------------------------------------------------------ config 2: mixed small tensors

@pytest.mark.parametrize("align", [256, 1])
def test_c2_mixed_bundle_full(pkg, orc, gpu, align):
    import torch
    from execution_ucx_amd import workloads
    spec = workloads.mixed_bundle()
    assert len(spec.segments) == 4096
    arena, tensors = workloads.materialize_mixed(spec, gpu, seed=0)
    host_arena = arena.cpu().numpy()
    chunks = [host_arena[s.arena_offset:s.arena_offset + s.nbytes] for s in spec.segments]
    got, plan, buf = run_pack(pkg, tensors, align, gpu)           # through 4096 DLPack capsules
    assert plan.data_bytes == spec.data_bytes
    want = orc.pack(chunks, align)
    assert got.size == want.size
    assert np.array_equal(got, want)
    offs, sizes = plan.layout()
    assert (offs, plan.payload_bytes) == orc.layout(sizes, align)
    # header carries dtype and shape of every tensor
    metas = plan.metas()
    for m, s in zip(metas, spec.segments):
        assert m.dtype == s.dtype and m.nbytes == s.nbytes and m.device[0] == 10
    # unpack into fresh tensors
    outs = [torch.zeros_like(t) for t in tensors]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    back = orc.unpack(want, sizes, align)
    for o, b in zip(outs, back):
        assert np.array_equal(tbytes(o), b)


# ------------------------------------------------------------------ config 3: Llama layer

def test_c3_llama_layer_full(pkg, orc, gpu):
    import torch
    from execution_ucx_amd import workloads
    tensors = workloads.materialize_llama_layer(gpu, seed=0)
    chunks = [tbytes(t) for t in tensors]
    got, plan, buf = run_pack(pkg, tensors, 256, gpu)
    assert plan.data_bytes == 404_766_720 == workloads.llama_layer_bytes()
    assert np.array_equal(got, orc.pack(chunks, 256))
    outs = [torch.empty_like(t).zero_() for t in tensors]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    for a, b in zip(tensors, outs):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


# ------------------------------------------------------------------ alignment torture

@pytest.mark.parametrize("seed", [0, 1, 2])
def test_arbitrary_alignment(pkg, orc, gpu, seed):
    """Odd sizes, odd source offsets, tight layout, shifted payload base."""
    import torch
    rng = np.random.default_rng(seed)
    edge = [0, 1, 2, 3, 15, 16, 17, 31, 33, 255, 256, 257, 1023, 1024, 1025, 4095, 4097,
            8191, 8192, 8193, 16383, 16385, 3 * 8192 + 5]
    sizes = edge + [int(x) for x in rng.integers(1, 40000, size=40)]
    rng.shuffle(sizes)
    arena = rand_bytes_tensor(rng, sum(sizes) + 64 * len(sizes) + 64, gpu)
    host = arena.cpu().numpy()
    tensors, chunks, at = [], [], 0
    for n in sizes:
        at += int(rng.integers(0, 33))           # any byte offset
        tensors.append(arena[at:at + n])
        chunks.append(host[at:at + n])
        at += n
    for align, shift in ((1, 0), (1, 7), (16, 3), (256, 0), (4096, 1)):
        got, plan, buf = run_pack(pkg, tensors, align, gpu, base_shift=shift)
        want = orc.pack(chunks, align)
        assert np.array_equal(got, want), (align, shift)
        # unpack into destinations at fresh odd offsets
        dst_arena = device_bytes(sum(sizes) + 64 * len(sizes) + 64, gpu, fill=0xEE)
        outs, spans, dat = [], [], 0
        for n in sizes:
            dat += int(rng.integers(0, 33))
            outs.append(dst_arena[dat:dat + n])
            spans.append((dat, n))
            dat += n
        rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
        rplan.unpack(buf.data_ptr() + shift, plan.payload_bytes)
        torch.cuda.synchronize()
        hd = dst_arena.cpu().numpy()
        expect = np.full(hd.size, 0xEE, np.uint8)
        for (o, n), c in zip(spans, chunks):
            expect[o:o + n] = c
        assert np.array_equal(hd, expect), (align, shift)       # bytes between tensors untouched


@pytest.mark.parametrize("rows", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("threads", [64, 256, 1024])
def test_every_kernel_instantiation(pkg, orc, gpu, rows, threads):
    """Each tile size / workgroup size / temporal variant against the oracle,
    with several tiles per wave forced as well."""
    import torch
    rng = np.random.default_rng(rows * 1000 + threads)
    sizes = [0, 5, 16, 17, 1000, 1024, 1025, 2048, 4097, 16384, 16400, 70001, 3 * 16384 + 100]
    sizes += [int(x) for x in rng.integers(1, 60000, size=20)]
    streaming = [rand_bytes_tensor(rng, n, gpu) for n in sizes]
    mat = rand_bytes_tensor(rng, 200 * 3000, gpu).reshape(200, 3000)
    streaming += [mat[::2, 16:2064]]                        # run tiles
    # short runs and a transposition select the kernels that decode elements
    # (their workgroups hold at most 256 threads)
    general = streaming + [mat.t()[5:9], mat[:, 7:107], mat.t()]
    try:
        for tensors, thread_cap in ((streaming, 1024), (general, 256)):
            chunks = [tbytes(t) for t in tensors]
            for nt, max_waves in ((3, 1 << 20), (0, 1 << 20), (1, 7), (2, 1 << 20)):
                pkg.tune(tile_rows=rows, threads=threads, nontemporal=nt, max_waves=max_waves)
                for align in (1, 256):
                    got, plan, buf = run_pack(pkg, tensors, align, gpu)
                    info = plan.launch_info()
                    assert info["tile_bytes"] == rows * 1024
                    got_threads = info["threads_per_workgroup"]
                    if tensors is streaming:
                        assert got_threads == threads
                    else:                       # also bounded by the LDS the byte transposition needs
                        assert got_threads in (min(threads, 192), min(threads, thread_cap))
                    assert np.array_equal(got, orc.pack(chunks, align)), (nt, max_waves, align)
                    outs = [torch.zeros_like(t, memory_format=torch.contiguous_format) for t in tensors]
                    pkg.BundlePlan.from_header(plan.header).bind(outs).unpack(buf.data_ptr(),
                                                                               plan.payload_bytes)
                    torch.cuda.synchronize()
                    for o, c in zip(outs, chunks):
                        assert np.array_equal(tbytes(o), c), (nt, max_waves, align)
    finally:
        pkg.tune(tile_rows=0, threads=0, nontemporal=-1, max_waves=1 << 20)


# ------------------------------------------------------------------ strided views

def random_torch_view(rng, parent, max_dims):
    """A random strided view of a torch tensor (slices, steps, permutes)."""
    ndim = parent.dim()
    index = []
    for d in range(ndim):
        n = parent.shape[d]
        lo = int(rng.integers(0, n))
        hi = int(rng.integers(lo + 1, n + 1))
        step = int(rng.choice([1, 1, 1, 2, 3]))
        index.append(slice(lo, hi, step))
    v = parent[tuple(index)]
    if rng.random() < 0.6:
        v = v.permute(*[int(i) for i in rng.permutation(ndim)])
    return v


def random_numpy_view(rng, parent):
    """A view of `parent` with forward and backward steps and permuted dimensions."""
    index = []
    for n in parent.shape:
        lo = int(rng.integers(0, n))
        hi = int(rng.integers(lo + 1, n + 1))
        step = int(rng.choice([1, 1, 2, 3, -1, -1, -2]))
        index.append(slice(lo, hi, step) if step > 0 else slice(hi - 1, lo - 1 if lo else None, step))
    v = parent[tuple(index)]
    if rng.random() < 0.6:
        v = v.transpose(*[int(i) for i in rng.permutation(parent.ndim)])
    return v


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_views_with_negative_strides(pkg, orc, gpu, seed):
    """numpy exports views that walk memory backwards (`a[::-1]`); torch never does, so
    these are described by hand over a device copy of the same bytes.  Gather against
    the oracle, then scatter into a poisoned twin and compare the whole twin."""
    import torch
    rng = np.random.default_rng(100 + seed)
    dtypes = [(np.uint8, (1, 8, 1)), (np.int16, (0, 16, 1)), (np.float32, (2, 32, 1)),
              (np.float64, (2, 64, 1)), (np.complex128, (5, 128, 1))]
    memory = rng.integers(0, 256, size=1 << 23, dtype=np.uint8)
    device = torch.from_numpy(memory).to(gpu)
    base = memory.__array_interface__["data"][0]
    for trial in range(10):
        described, chunks, at = [], [], 0
        for _ in range(int(rng.integers(1, 5))):
            np_dt, dl_dt = dtypes[int(rng.integers(0, len(dtypes)))]
            item = np.dtype(np_dt).itemsize
            ndim = int(rng.integers(1, 5))
            cap = 300 if ndim == 1 else (90 if ndim == 2 else (30 if ndim == 3 else 12))
            shape = [int(x) for x in rng.integers(1, cap + 1, size=ndim)]
            if rng.random() < 0.3:
                shape = [min(n, 6) for n in shape[:-1]] + [int(rng.integers(100, 3000))]
            nbytes = int(np.prod(shape)) * item
            at = (at + 15) // 16 * 16 + int(rng.choice([0, 0, item]))
            if at + nbytes > memory.size:
                break                                       # this trial has enough tensors
            v = random_numpy_view(rng, memory[at:at + nbytes].view(np_dt).reshape(shape))
            start = v.__array_interface__["data"][0] - base
            strides = tuple(st // item for st in v.strides)
            described.append((start, dl_dt, tuple(v.shape), strides, item))
            chunks.append(np.ascontiguousarray(v).view(np.uint8).reshape(-1))
            at += nbytes

        def views_over(tensor):
            return [pkg.TensorView(data=tensor.data_ptr() + start, device_type=10, device_id=0, dtype=dl_dt,
                                   shape=shape, strides=strides)
                    for start, dl_dt, shape, strides, _ in described]
        if not described:
            continue
        align = int(rng.choice([1, 64, 256]))
        want = orc.pack(chunks, align)
        plan = pkg.BundlePlan.create(views_over(device), align=align)
        n = plan.payload_bytes
        assert n == want.size
        payload = device_bytes(n, gpu)
        plan.pack(payload.data_ptr(), n)
        torch.cuda.synchronize()
        assert np.array_equal(payload.cpu().numpy()[:n], want), (seed, trial)
        twin = device_bytes(memory.size, gpu, fill=0x77)
        back = pkg.BundlePlan.from_header(plan.header).bind(views_over(twin))
        back.unpack(payload.data_ptr(), n)
        torch.cuda.synchronize()
        expect = np.full(memory.size, 0x77, np.uint8)
        for (start, _, shape, strides, item), c in zip(described, chunks):
            orc.scatter_strided(c, expect, start, shape, strides, item)
        assert np.array_equal(twin.cpu().numpy(), expect), (seed, trial)
        plan.close()
        back.close()


@pytest.mark.parametrize("dtype_name", ["uint8", "bfloat16", "float32", "float64", "complex128"])
def test_strided_gather_scatter_random(pkg, orc, gpu, dtype_name):
    import torch
    dt = getattr(torch, dtype_name)
    item = torch.empty((), dtype=dt).element_size()
    rng = np.random.default_rng(item)
    for trial in range(12):
        ndim = int(rng.integers(1, 6))
        shape = [int(x) for x in rng.integers(1, 9, size=ndim)]
        shape[-1] = int(rng.integers(1, 400))                # sometimes long inner runs
        nbytes = int(np.prod(shape)) * item
        parent = rand_bytes_tensor(rng, nbytes, gpu).view(dt).reshape(shape)
        views = [random_torch_view(rng, parent, ndim) for _ in range(3)]
        views.append(parent)                                  # a compact one in between
        host_parent = parent.reshape(-1).view(torch.uint8).cpu().numpy()
        chunks = []
        for v in views:
            start = (v.data_ptr() - parent.data_ptr())
            chunks.append(orc.gather_strided(host_parent, start, tuple(v.shape), tuple(v.stride()), item))
            assert np.array_equal(chunks[-1], tbytes(v))       # oracle == .contiguous()
        for align in (1, 256):
            got, plan, buf = run_pack(pkg, views, align, gpu)
            assert np.array_equal(got, orc.pack(chunks, align)), (trial, align)
            # scatter into a poisoned twin of the parent at the same views
            twin = device_bytes(nbytes, gpu, fill=0x77).view(dt).reshape(shape)
            tviews = [twin.as_strided(v.shape, v.stride(), v.storage_offset()) for v in views[:-1]]
            rplan = pkg.BundlePlan.from_header(plan.header)
            metas = rplan.metas()[:-1]
            # unpack only the strided ones: rebuild a header-compatible plan for them
            sub = pkg.BundlePlan.create(views[:-1], align=align)
            sub_payload = device_bytes(sub.payload_bytes, gpu)
            sub.pack(sub_payload.data_ptr(), sub.payload_bytes)
            rsub = pkg.BundlePlan.from_header(sub.header).bind(tviews)
            rsub.unpack(sub_payload.data_ptr(), sub.payload_bytes)
            torch.cuda.synchronize()
            expect = np.full(nbytes, 0x77, np.uint8)
            for v, c in zip(views[:-1], chunks[:-1]):
                orc.scatter_strided(c, expect, v.data_ptr() - parent.data_ptr(), tuple(v.shape),
                                    tuple(v.stride()), item)
            assert np.array_equal(twin.reshape(-1).view(torch.uint8).cpu().numpy(), expect), (trial, align)
            assert len(metas) == len(views) - 1


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_strided_views_larger_extents(pkg, orc, gpu, seed):
    """Random slices and permutations of 2- to 4-d parents with extents up to 90:
    large enough for transposed blocks with batch dimensions, ragged edges and
    misaligned bases, mixed in one bundle with element mode and run tiles."""
    import torch
    rng = np.random.default_rng(1000 + seed)
    names = ["uint8", "int16", "float32", "float64", "complex128"]
    for trial in range(10):
        cases = []
        for _ in range(int(rng.integers(1, 5))):
            dt = getattr(torch, names[int(rng.integers(0, len(names)))])
            item = torch.empty((), dtype=dt).element_size()
            ndim = int(rng.integers(2, 5))
            shape = [int(x) for x in rng.integers(1, 91 if ndim < 4 else 25, size=ndim)]
            parent = rand_bytes_tensor(rng, int(np.prod(shape)) * item, gpu).view(dt).reshape(shape)
            cases.append((parent, random_torch_view(rng, parent, ndim), item))
        views = [v for _, v, _ in cases]
        chunks = []
        for parent, v, item in cases:
            host_parent = parent.reshape(-1).view(torch.uint8).cpu().numpy()
            chunks.append(orc.gather_strided(host_parent, v.data_ptr() - parent.data_ptr(),
                                             tuple(v.shape), tuple(v.stride()), item))
        align = int(rng.choice([1, 16, 256]))
        got, plan, buf = run_pack(pkg, views, align, gpu)
        assert np.array_equal(got, orc.pack(chunks, align)), (seed, trial)
        twins, tviews = [], []
        for parent, v, item in cases:
            twin = device_bytes(parent.numel() * item, gpu, fill=0x77).view(parent.dtype).reshape(parent.shape)
            twins.append(twin)
            tviews.append(twin.as_strided(v.shape, v.stride(), v.storage_offset()))
        pkg.BundlePlan.from_header(plan.header).bind(tviews).unpack(buf.data_ptr(), plan.payload_bytes)
        torch.cuda.synchronize()
        for (parent, v, item), twin, c in zip(cases, twins, chunks):
            e = np.full(parent.numel() * item, 0x77, np.uint8)
            orc.scatter_strided(c, e, v.data_ptr() - parent.data_ptr(), tuple(v.shape),
                                tuple(v.stride()), item)
            assert np.array_equal(twin.reshape(-1).view(torch.uint8).cpu().numpy(), e), (seed, trial)


@pytest.mark.parametrize("dtype_name", ["uint8", "bfloat16", "float32", "float64", "complex128"])
def test_transposed_views(pkg, orc, gpu, dtype_name):
    """Views whose packed-inner dimension is strided while another dimension is
    contiguous in the tensor move as square blocks through LDS: whole aligned
    blocks, ragged edges, misaligned bases and batched permutations, against the
    oracle's element-by-element gather and scatter."""
    import torch
    dt = getattr(torch, dtype_name)
    item = torch.empty((), dtype=dt).element_size()
    t = (128 if item <= 4 else 256) // item                    # block edge in elements
    rng = np.random.default_rng(100 + item)

    def parent_of(shape):
        nbytes = int(np.prod(shape)) * item
        return rand_bytes_tensor(rng, nbytes, gpu).view(dt).reshape(shape)

    m2 = parent_of([2 * t, 3 * t])
    m3 = parent_of([t + 5, 2 * t + 3])
    m4 = parent_of([3, 20, 2, 24])
    m5 = parent_of([2, 9, 70])
    m6 = parent_of([4, 3, 20, 30])                              # NCHW
    m7 = parent_of([4, 20, 30, 3])                              # NHWC
    m8 = parent_of([3000, 2])
    cases = [
        (m6, m6.permute(0, 2, 3, 1)),                          # channels last: 3 x 600 rectangles
        (m7, m7.permute(0, 3, 1, 2)),                          # and back
        (m8, m8.t()),                                          # interleaved pairs to two planes
        (m8, m8[5:2900:1].t()),
        (m2, m2.t()),                                          # whole aligned blocks only
        (m3, m3.t()),                                          # ragged in both directions
        (m3, m3[1:, 3:].t()),                                  # base off the 16-byte grid
        (m3, m3[::2, 1::3].t()),                               # strided on both sides: element mode
        (m4, m4.permute(2, 0, 3, 1)),                          # two batch dims around the block
        (m4, m4[:, 2:19].permute(0, 2, 3, 1)),
        (m5, m5.permute(2, 0, 1)),                             # [70, 2*9] after merging
        (m5, m5.permute(1, 2, 0)),
    ]
    views = [v for _, v in cases]
    plan = pkg.BundlePlan.create(views, align=256)
    modes = [s["mode"] for s in plan.segments()]
    assert modes.count(5) >= 9, modes
    chunks = []
    for parent, v in cases:
        host_parent = parent.reshape(-1).view(torch.uint8).cpu().numpy()
        chunks.append(orc.gather_strided(host_parent, v.data_ptr() - parent.data_ptr(),
                                         tuple(v.shape), tuple(v.stride()), item))
    for align in (256, 1):
        got, plan, buf = run_pack(pkg, views, align, gpu)
        assert np.array_equal(got, orc.pack(chunks, align)), align
        # scatter back through the same views of poisoned twins
        twins, tviews, expects = [], [], []
        for (parent, v), c in zip(cases, chunks):
            twin = device_bytes(parent.numel() * item, gpu, fill=0x77).view(dt).reshape(parent.shape)
            twins.append(twin)
            tviews.append(twin.as_strided(v.shape, v.stride(), v.storage_offset()))
            e = np.full(parent.numel() * item, 0x77, np.uint8)
            orc.scatter_strided(c, e, v.data_ptr() - parent.data_ptr(), tuple(v.shape),
                                tuple(v.stride()), item)
            expects.append(e)
        pkg.BundlePlan.from_header(plan.header).bind(tviews).unpack(buf.data_ptr(), plan.payload_bytes)
        torch.cuda.synchronize()
        for i, (twin, e) in enumerate(zip(twins, expects)):
            assert np.array_equal(twin.reshape(-1).view(torch.uint8).cpu().numpy(), e), (align, i)
    # the element-by-element path gives the same bytes
    pkg.tune(transpose=0)
    try:
        got0, plan0, _ = run_pack(pkg, views, 256, gpu)
        assert 5 not in {s["mode"] for s in plan0.segments()}
        assert np.array_equal(got0, orc.pack(chunks, 256))
    finally:
        pkg.tune(transpose=1)


def test_transposed_large_matrix_round_trip(pkg, gpu):
    """A 4096 x 4096 bf16 transposition (32 MiB) against torch's own
    contiguous copy, and back into a transposed destination."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    x = torch.randint(-2 ** 15, 2 ** 15, (4096, 4096), device="cuda", generator=g,
                      dtype=torch.int16).view(torch.bfloat16)
    plan = pkg.BundlePlan.create([x.t()], align=256)
    assert [s["mode"] for s in plan.segments()] == [5]
    buf = device_bytes(plan.payload_bytes, gpu)
    plan.pack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    want = x.t().contiguous().view(torch.int16).reshape(-1)
    assert torch.equal(buf[:want.numel() * 2].view(torch.int16), want)
    y = torch.zeros_like(x)
    pkg.BundlePlan.from_header(plan.header).bind([y.t()]).unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), x.view(torch.int16))


def test_strided_many_dims_and_long_runs(pkg, orc, gpu):
    """More strided outer dimensions than the device table holds (peeled on the
    host), runs that span several tiles, and a transposed matrix."""
    import torch
    rng = np.random.default_rng(42)
    p8 = rand_bytes_tensor(rng, 3 * 4 * 3 * 4 * 3 * 4 * 3 * 4 * 40 * 2, gpu).view(torch.int16)
    p8 = p8.reshape(3, 4, 3, 4, 3, 4, 3, 4, 40)
    v8 = p8[:2, 1:3, :2, ::2, 1:, :3, ::2, 1:3, 4:36]          # 8 strided dims + 64 B runs
    big = rand_bytes_tensor(rng, 64 * 40000, gpu).view(torch.float32).reshape(64, 10000)
    vlong = big[::2, 17:9000]                                   # 35,932 B runs, 4-byte aligned only
    mat = rand_bytes_tensor(rng, 300 * 500 * 2, gpu).view(torch.bfloat16).reshape(300, 500)
    views = [v8, vlong, mat.t(), mat[:, 100:164]]
    chunks = [tbytes(v) for v in views]
    plan = pkg.BundlePlan.create(views, align=256)
    modes = {s["mode"] for s in plan.segments()}
    assert {1, 2, 5} <= modes                  # run tiles, element mode and transposed blocks all used
    got, plan, buf = run_pack(pkg, views, 256, gpu)
    assert np.array_equal(got, orc.pack(chunks, 256))
    outs = [torch.zeros_like(v, memory_format=torch.contiguous_format) for v in views]
    pkg.BundlePlan.from_header(plan.header).bind(outs).unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    for v, o in zip(views, outs):
        assert np.array_equal(tbytes(o), tbytes(v))


def test_c4_kv_gather_reduced_vs_oracle(pkg, orc, gpu):
    import torch
    from execution_ucx_amd import workloads
    spec = workloads.kv_gather(layers=4, blocks=64, picks=16, seed=0)
    n = int(np.prod(spec.cache_shape))
    a = torch.randn(n, device=gpu).to(torch.bfloat16)
    b = torch.zeros(n, dtype=torch.bfloat16, device=gpu)
    src = [workloads.kv_block_view(a.data_ptr(), spec, int(i)) for i in spec.src_index]
    dst = [workloads.kv_block_view(b.data_ptr(), spec, int(i)) for i in spec.dst_index]
    host_a = a.view(torch.uint8).cpu().numpy()
    chunks = [orc.gather_strided(host_a, v.data - a.data_ptr(), v.shape, v.strides, 2) for v in src]
    got, plan, buf = run_pack(pkg, src, 256, gpu)
    assert plan.payload_bytes == spec.payload_bytes
    assert np.array_equal(got, orc.pack(chunks, 256))
    seg = plan.segments()[0]
    assert (seg["mode"], seg["run_bytes"], seg["shape"]) == (1, spec.block_elems * 2, (spec.layers * 2,))
    pkg.BundlePlan.from_header(plan.header).bind(dst).unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    expect = np.zeros(n * 2, np.uint8)
    for v, c in zip(dst, chunks):
        orc.scatter_strided(c, expect, v.data - b.data_ptr(), v.shape, v.strides, 2)
    assert np.array_equal(b.view(torch.uint8).cpu().numpy(), expect)


def test_c4_kv_gather_full_size_properties(pkg, gpu):
    """8 GiB caches, 1 GiB payload: checked with size-independent properties on
    the device (moved blocks equal, everything else untouched)."""
    import torch
    from execution_ucx_amd import workloads
    spec = workloads.kv_gather()
    shape = spec.cache_shape
    a = torch.empty(shape, dtype=torch.bfloat16, device=gpu)
    a.view(torch.int16).random_(-32768, 32767)
    b = torch.zeros(shape, dtype=torch.bfloat16, device=gpu)
    src = [workloads.kv_block_view(a.data_ptr(), spec, int(i)) for i in spec.src_index]
    dst = [workloads.kv_block_view(b.data_ptr(), spec, int(i)) for i in spec.dst_index]
    plan = pkg.BundlePlan.create(src, align=256)
    assert plan.payload_bytes == 1 << 30 == spec.payload_bytes
    payload = torch.empty(1 << 30, dtype=torch.uint8, device=gpu)
    plan.pack(payload.data_ptr(), 1 << 30)
    torch.cuda.synchronize()
    si = torch.from_numpy(spec.src_index).to(gpu)
    di = torch.from_numpy(spec.dst_index).to(gpu)
    # payload == [block j][layer][kv] order == A[:, :, src].permute(2, 0, 1, ...)
    want = a.view(torch.int16)[:, :, si].permute(2, 0, 1, 3, 4, 5).contiguous()
    assert torch.equal(payload.view(torch.int16), want.reshape(-1))
    del want
    pkg.BundlePlan.from_header(plan.header).bind(dst).unpack(payload.data_ptr(), 1 << 30)
    torch.cuda.synchronize()
    assert torch.equal(b.view(torch.int16)[:, :, di], a.view(torch.int16)[:, :, si])
    mask = torch.ones(spec.blocks, dtype=torch.bool, device=gpu)
    mask[di] = False
    assert int(b.view(torch.int16)[:, :, mask].ne(0).sum()) == 0


def test_c5_pitched_chunk(pkg, orc, gpu):
    """One 256 MiB chunk of 64 pitched 2-D views, and a small one against the oracle."""
    import torch
    from execution_ucx_amd import workloads
    small = workloads.pitched_chunk(views=3, rows=5, cols=64)
    big = workloads.pitched_chunk()
    assert big.payload_bytes == 256 << 20
    for spec, use_oracle in ((small, True), (big, False)):
        parents = torch.empty(spec.views, spec.rows, spec.pitch, dtype=torch.bfloat16, device=gpu)
        parents.view(torch.int16).random_(-32768, 32767)
        views = workloads.pitched_views(parents.data_ptr(), spec)
        plan = pkg.BundlePlan.create(views, align=256)
        assert plan.data_bytes == spec.payload_bytes
        nbytes = plan.payload_bytes                      # small views leave alignment gaps
        payload = device_bytes(nbytes, gpu)
        plan.pack(payload.data_ptr(), nbytes)
        torch.cuda.synchronize()
        if use_oracle:
            host = parents.view(torch.uint8).reshape(-1).cpu().numpy()
            chunks = [orc.gather_strided(host, v.data - parents.data_ptr(), v.shape, v.strides, 2)
                      for v in views]
            assert np.array_equal(payload.cpu().numpy()[:nbytes], orc.pack(chunks, 256))
        else:
            assert nbytes == spec.payload_bytes
            want = parents[:, :, :spec.cols].contiguous()
            assert torch.equal(payload[:nbytes].view(torch.int16), want.view(torch.int16).reshape(-1))
        twin = torch.zeros_like(parents)
        tv = workloads.pitched_views(twin.data_ptr(), spec)
        pkg.BundlePlan.from_header(plan.header).bind(tv).unpack(payload.data_ptr(), nbytes)
        torch.cuda.synchronize()
        assert torch.equal(twin.view(torch.int16)[:, :, :spec.cols],
                           parents.view(torch.int16)[:, :, :spec.cols])   # bit patterns: NaNs compare equal
        assert int(twin[:, :, spec.cols:].view(torch.int16).ne(0).sum()) == 0     # pitch gap untouched


@pytest.mark.parametrize("zero_copy", [True, False])
def test_c5_streamed_pipeline(pkg, gpu, zero_copy):
    """Double-buffered pack -> loopback send -> unpack over two streams: small
    chunks (eager and rendezvous sizes by the reference's threshold) and the full
    stream of 32 chunks of 256 MiB (8 GiB), all chunks of a stream served by one
    sender plan and one receiver plan.  With the receiver borrowing the sender's slot
    (zero copy) and with a copy into a receive slot."""
    import torch
    from execution_ucx_amd import workloads
    for spec, chunks in ((workloads.pitched_chunk(views=3, rows=4, cols=64), 7),
                         (workloads.pitched_chunk(views=5, rows=64, cols=256), 9),
                         (workloads.pitched_chunk(), 32)):
        src = torch.empty(chunks, spec.views, spec.rows, spec.pitch, dtype=torch.bfloat16, device=gpu)
        src.view(torch.int16).random_(-32768, 32767)
        dst = torch.zeros_like(src)
        torch.cuda.synchronize()
        slot = (spec.view_bytes + 255) // 256 * 256 * spec.views
        st = pkg.StreamedTransfer(slot_bytes=slot, streams=2, zero_copy=zero_copy)
        per_chunk = spec.views * spec.parent_elems * 2
        for k in range(chunks):
            st.submit(workloads.pitched_views(src.data_ptr() + k * per_chunk, spec),
                      workloads.pitched_views(dst.data_ptr() + k * per_chunk, spec))
        assert st._plans is not None and len(st._keep) == chunks     # one pair of plans for the stream
        st.finish()
        s16, d16 = src.view(torch.int16), dst.view(torch.int16)
        assert torch.equal(d16[..., :spec.cols], s16[..., :spec.cols])
        assert int(d16[..., spec.cols:].ne(0).sum()) == 0
        st.close()
        assert pkg.DevicePool.default().stats()["live_blocks"] == 0
        del src, dst, s16, d16
        torch.cuda.empty_cache()


def test_streamed_host_chunks_plan_anew(pkg, gpu):
    """Chunks of host (numpy) tensors of one geometry at different addresses: a bundle with
    host tensors cannot be rebased by an address delta, so every chunk at a new base gets
    fresh plans (and the result is right from the second chunk on)."""
    import torch
    rng = np.random.default_rng(21)
    chunks = 4
    srcs = [[rng.integers(0, 256, size=n, dtype=np.uint8) for n in (70000, 33, 4096)] for _ in range(chunks)]
    outs = [[np.zeros_like(a) for a in c] for c in srcs]
    st = pkg.StreamedTransfer(slot_bytes=1 << 20, streams=2)
    plans_seen = set()
    for c, o in zip(srcs, outs):
        st.submit(c, o)
        plans_seen.add(id(st._plans[4]))
    st.finish()
    for c, o in zip(srcs, outs):
        for a, b in zip(c, o):
            assert np.array_equal(a, b)
    assert len(plans_seen) == chunks                     # no plan was moved by a delta
    # the same chunk again reuses its plans (same base: delta 0)
    st.submit(srcs[-1], outs[-1])
    assert id(st._plans[4]) in plans_seen
    st.finish()
    st.close()
    # device chunks of one geometry still share one pair of plans
    dev = torch.from_numpy(rng.integers(0, 256, size=(3, 5000), dtype=np.uint8)).to(gpu)
    back = torch.zeros_like(dev)
    st = pkg.StreamedTransfer(slot_bytes=1 << 20, streams=1)
    ids = set()
    for k in range(3):
        st.submit([dev[k, :3000], dev[k, 3000:]], [back[k, :3000], back[k, 3000:]])
        ids.add(id(st._plans[4]))
    st.finish()
    assert len(ids) == 1 and torch.equal(dev, back)
    st.close()


def test_streamed_transfer_through_the_c_abi(pkg, orc, gpu):
    """axr_transfer_* with plans the caller keeps: chunks of one geometry at growing
    deltas, one, two and three lanes, a change of geometry, and the refusals."""
    import ctypes as C
    import torch
    from execution_ucx_amd import workloads
    lib, capi = pkg._capi.load(), pkg._capi
    spec = workloads.pitched_chunk(views=4, rows=33, cols=200)
    chunks = 11
    per_chunk = spec.views * spec.parent_elems * 2
    rng = np.random.default_rng(3)
    src = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, size=(chunks, spec.views, spec.rows, spec.pitch),
                                        dtype=np.int16)).to(gpu).view(torch.bfloat16)
    send = pkg.BundlePlan.create(workloads.pitched_views(src.data_ptr(), spec), align=256)
    slot = send.payload_bytes
    for lanes, streams, zero_copy in ((1, 1, 1), (2, 2, 1), (2, 1, 0), (3, 2, 0), (2, 2, 0), (3, 2, 1)):
        dst = torch.zeros_like(src)
        recv = pkg.BundlePlan.from_header(send.header).bind(workloads.pitched_views(dst.data_ptr(), spec))
        torch.cuda.synchronize()
        t = C.c_void_p()
        assert lib.axr_transfer_create(None, slot, lanes, lanes + 1, C.byref(t)) == capi.AXR_ERR_INVALID
        capi.check(lib.axr_transfer_create(None, slot, lanes, streams, C.byref(t)))
        capi.check(lib.axr_transfer_set_zero_copy(t, zero_copy))
        # chunks in a scrambled order: deltas need not grow
        order = [int(k) for k in rng.permutation(chunks)]
        for k in order:
            capi.check(lib.axr_transfer_submit(t, send._h, k * per_chunk, recv._h, k * per_chunk))
        capi.check(lib.axr_transfer_finish(t))
        s16, d16 = src.view(torch.int16), dst.view(torch.int16)
        assert torch.equal(d16[..., :spec.cols], s16[..., :spec.cols])
        assert int(d16[..., spec.cols:].ne(0).sum()) == 0
        # refusals: a receiver plan of another header; a chunk beyond the slot
        other = pkg.BundlePlan.create([torch.zeros(64, dtype=torch.uint8, device=gpu)], align=256)
        assert lib.axr_transfer_submit(t, send._h, 0, other._h, 0) == capi.AXR_ERR_MISMATCH
        big = torch.zeros(slot + 256, dtype=torch.uint8, device=gpu)
        bigplan = pkg.BundlePlan.create([big], align=256)
        bigrecv = pkg.BundlePlan.from_header(bigplan.header).bind([torch.zeros_like(big)])
        assert lib.axr_transfer_submit(t, bigplan._h, 0, bigrecv._h, 0) == capi.AXR_ERR_LENGTH
        # a chunk that fails after its send was queued (injected: the message "does not match"):
        # the send is withdrawn, the lane comes back idle, and good chunks follow on every lane
        dst.zero_()
        torch.cuda.synchronize()
        capi.check(lib.axr_transfer_submit(t, send._h, 0, recv._h, 0))
        pkg.tune(transfer_fail_after_send=1)
        assert lib.axr_transfer_submit(t, send._h, per_chunk, recv._h, per_chunk) == capi.AXR_ERR_MISMATCH
        assert b"does not match" in lib.axr_last_error()
        for k in range(2, 2 + 2 * lanes):
            capi.check(lib.axr_transfer_submit(t, send._h, k * per_chunk, recv._h, k * per_chunk))
        capi.check(lib.axr_transfer_finish(t))
        d16 = dst.view(torch.int16)
        moved = [0] + list(range(2, 2 + 2 * lanes))
        assert torch.equal(d16[moved][..., :spec.cols], s16[moved][..., :spec.cols])
        assert int(d16[1].ne(0).sum()) == 0                       # the failed chunk moved nothing
        # the mode cannot change under chunks in flight
        capi.check(lib.axr_transfer_submit(t, send._h, 0, recv._h, 0))
        assert lib.axr_transfer_set_zero_copy(t, 1 - zero_copy) == capi.AXR_ERR_BUSY
        capi.check(lib.axr_transfer_finish(t))
        capi.check(lib.axr_transfer_set_zero_copy(t, zero_copy))
        # another geometry through the same transfer (smaller than a slot)
        a = torch.from_numpy(rng.integers(0, 256, size=5000, dtype=np.uint8)).to(gpu)
        b = torch.zeros_like(a)
        p1 = pkg.BundlePlan.create([a[:3000], a[3000:]], align=1)
        p2 = pkg.BundlePlan.from_header(p1.header).bind([b[:3000], b[3000:]])
        torch.cuda.synchronize()
        capi.check(lib.axr_transfer_submit(t, p1._h, 0, p2._h, 0))
        capi.check(lib.axr_transfer_finish(t))
        assert torch.equal(a, b)
        # an empty bundle is a chunk without a message
        e1 = pkg.BundlePlan.create([a[:0]], align=1)
        e2 = pkg.BundlePlan.from_header(e1.header).bind([b[:0]])
        capi.check(lib.axr_transfer_submit(t, e1._h, 0, e2._h, 0))
        capi.check(lib.axr_transfer_destroy(t))
        for p in (recv, other, bigplan, bigrecv, p1, p2, e1, e2):
            p.close()
        assert pkg.DevicePool.default().stats()["live_blocks"] == 0
    send.close()


# ------------------------------------------------------------------ checksums, compare

def test_checksum_of_checksums(pkg, orc, gpu):
    import torch
    lib = pkg._capi.load()
    rng = np.random.default_rng(1)
    tensors = [rand_bytes_tensor(rng, int(n), gpu) for n in rng.integers(1, 200000, size=30)]
    got, plan, buf = run_pack(pkg, tensors, 256, gpu)
    offs, sizes = plan.layout()
    total = C.c_uint64()
    pkg._capi.check(lib.axr_checksum(buf.data_ptr(), plan.payload_bytes, 0, C.byref(total)))
    assert total.value == orc.checksum(got, 0)
    acc = 0
    for t, o in zip(tensors, offs):
        s = C.c_uint64()
        pkg._capi.check(lib.axr_checksum(t.data_ptr(), t.numel(), o, C.byref(s)))
        acc = (acc + s.value) % (1 << 64)
    assert acc == total.value                    # zero gaps add nothing
    mism = C.c_uint64(99)
    twin = buf.clone()
    pkg._capi.check(lib.axr_compare(buf.data_ptr(), twin.data_ptr(), plan.payload_bytes, C.byref(mism)))
    assert mism.value == 0
    twin[5] ^= 1
    twin[plan.payload_bytes - 1] ^= 0x80
    pkg._capi.check(lib.axr_compare(buf.data_ptr(), twin.data_ptr(), plan.payload_bytes, C.byref(mism)))
    assert mism.value == 2


# ------------------------------------------------------------------ DLPack in and out

def test_dlpack_rocm_capsules_and_zero_copy_receive(pkg, gpu):
    import torch
    srcs = [torch.randn(1000, device=gpu), torch.randn(7, 33, device=gpu).to(torch.bfloat16),
            torch.arange(50, device=gpu, dtype=torch.int32)]
    view = pkg.extract(srcs[1])
    assert view.device_type == 10 and view.dtype == (4, 16, 1) and view.shape == (7, 33)
    stream = torch.cuda.current_stream().cuda_stream
    packed = pkg.pack_bundle(srcs, align=256, stream=stream)
    assert packed.payload.memory_type == 3                      # ucx_memory_type::ROCM
    outs = pkg.unpack_bundle(packed.header, packed.payload, stream=stream,
                             from_dlpack_fn=torch.from_dlpack)
    torch.cuda.synchronize()
    for a, b in zip(srcs, outs):
        assert b.device.type == "cuda" and b.dtype == a.dtype and b.shape == a.shape
        assert torch.equal(a, b)
    base = packed.payload.data
    assert [o.data_ptr() - base for o in outs] == packed.plan.layout()[0]   # views, not copies


def test_torch_device_tensors_through_the_short_export_route(pkg, orc, gpu):
    """GPU tensors are exported from C with to_dlpack while torch runs on its default
    stream, and through Tensor.__dlpack__ (which orders the streams) on any other;
    both routes describe the same memory and pack the oracle's bytes."""
    import torch
    from execution_ucx_amd import dlpack
    rng = np.random.default_rng(33)
    tensors = [rand_bytes_tensor(rng, n, gpu) for n in (4096, 10, 70002, 0, 512)]
    tensors[2] = tensors[2][2:70002].view(torch.int16).reshape(100, 350)[:, 3:77]
    fast = dlpack._torch_exporter()
    assert fast and fast[2] == torch.cuda.current_device()
    short = dlpack.TensorArray.from_objects(tensors).views
    plain = dlpack.extract_many(tensors)
    assert [(x.data, x.device_type, x.shape, x.strides, x.dtype) for x in short] == \
        [(x.data, x.device_type, x.shape, x.strides, x.dtype) for x in plain]
    # the reader that makes no capsules took them (device and pinned host tensors alike), and
    # declines GPU tensors when asked for another device than theirs
    direct = dlpack._native_torch()
    assert direct is not None, "build lib/_axr_torch*.so with `make -C execution-ucx_amd`"
    with_pinned = tensors + [torch.arange(12, dtype=torch.float32).pin_memory().view(3, 4)[:, 1:]]
    described = direct.describe(with_pinned, fast[2])
    assert described is not None and described[2] == with_pinned
    again = dlpack._native().describe(with_pinned, *fast)
    count = len(with_pinned)
    ta = (dlpack._capi.Tensor * count).from_buffer(described[0])
    tb = (dlpack._capi.Tensor * count).from_buffer(again[0])
    for i in range(count):
        for f in ("data", "device_type", "device_id", "ndim", "dtype_code", "dtype_bits", "dtype_lanes",
                  "byte_offset"):
            assert getattr(ta[i], f) == getattr(tb[i], f), (i, f)
    del ta, tb
    assert bytes(described[1]) == bytes(again[1])
    assert direct.describe(tensors, fast[2] + 1) is None and direct.describe(tensors, -1) is None
    want = orc.pack([tbytes(t) for t in tensors], 64)
    got, plan, _ = run_pack(pkg, tensors, 64, gpu)
    assert np.array_equal(got, want)
    plan.close()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert dlpack._torch_exporter() == ()
        got, plan, _ = run_pack(pkg, tensors, 64, gpu)       # packs on `side`
    assert np.array_equal(got, want)
    plan.close()


def test_bundle_to_host_for_checkpointing(pkg, orc, gpu):
    """A packed device bundle staged to host byte arrays, one per tensor (what the
    reference's checkpoint writer builds with one memcpy per buffer,
    avro_serialization.cpp:478-523): 300 tensors and 40 MiB cross in 8 MiB blocks."""
    import torch
    rng = np.random.default_rng(21)
    sizes = [int(x) for x in rng.integers(0, 280000, size=300)]
    tensors = [rand_bytes_tensor(rng, n, gpu)[:n] for n in sizes]
    tensors[7] = rand_bytes_tensor(rng, 6000, gpu).view(torch.float32).reshape(30, 50).t()   # strided source
    bundle = pkg.pack_bundle(tensors, align=256)
    torch.cuda.synchronize()
    info = pkg.BundlePlan.from_header(bundle.header)
    arrays = pkg.bundle_to_host(bundle.header, bundle.payload, bundle.payload_bytes)
    assert len(arrays) == len(tensors)
    for a, t in zip(arrays, tensors):
        assert np.array_equal(a, tbytes(t))
    # few device copies for many tensors
    metas = info.metas()
    assert metas[7].shape == (50, 30)
    info.close()
    bundle.plan.close()
    bundle.payload.release()


def test_pinned_host_destination(pkg, orc, gpu):
    """Scatter a device payload straight into pinned host tensors (the staging a
    checkpoint writer needs) and gather from them: the kernel addresses pinned
    memory like device memory."""
    import torch
    rng = np.random.default_rng(8)
    srcs = [rand_bytes_tensor(rng, n, gpu) for n in (70000, 33, 4096, 123457)]
    got, plan, buf = run_pack(pkg, srcs, 256, gpu)
    pinned = [torch.zeros(t.numel(), dtype=torch.uint8).pin_memory() for t in srcs]
    views = [pkg.TensorView(data=p.data_ptr(), device_type=11, device_id=0, dtype=(1, 8, 1),
                            shape=(p.numel(),), strides=None, owner=p) for p in pinned]
    rplan = pkg.BundlePlan.from_header(plan.header).bind(views)
    assert rplan.launch_info()["host_copies"] == 0           # no staged copies: one kernel
    rplan.unpack(buf.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    for p, t in zip(pinned, srcs):
        assert np.array_equal(p.numpy(), t.cpu().numpy())
    got2, plan2, _ = run_pack(pkg, views, 256, gpu)          # and back: pinned sources
    assert np.array_equal(got2, got)


# ------------------------------------------------------------------ plan reuse, streams, errors

def test_plan_reuse_rebind_and_streams(pkg, orc, gpu):
    import torch
    lib = pkg._capi.load()
    rng = np.random.default_rng(2)
    a = [rand_bytes_tensor(rng, n, gpu) for n in (5000, 70000, 33)]
    b = [rand_bytes_tensor(rng, n, gpu) for n in (5000, 70000, 33)]
    plan = pkg.BundlePlan.create(a, align=256)
    n = plan.payload_bytes
    s1, s2 = C.c_void_p(), C.c_void_p()
    pkg._capi.check(lib.axr_stream_create(C.byref(s1)))
    pkg._capi.check(lib.axr_stream_create(C.byref(s2)))
    p1, p2 = device_bytes(n, gpu), device_bytes(n, gpu)
    torch.cuda.synchronize()
    plan.pack(p1.data_ptr(), n, s1.value)
    plan.pack(p2.data_ptr(), n, s2.value)          # second stream waits for the table upload
    pkg._capi.check(lib.axr_stream_synchronize(s1))
    pkg._capi.check(lib.axr_stream_synchronize(s2))
    want = orc.pack([tbytes(t) for t in a], 256)
    assert np.array_equal(p1.cpu().numpy()[:n], want)
    assert np.array_equal(p2.cpu().numpy()[:n], want)
    plan.bind(b)
    plan.pack(p1.data_ptr(), n, s1.value)
    pkg._capi.check(lib.axr_stream_synchronize(s1))
    assert np.array_equal(p1.cpu().numpy()[:n], orc.pack([tbytes(t) for t in b], 256))
    ev0, ev1 = C.c_void_p(), C.c_void_p()
    pkg._capi.check(lib.axr_event_create(C.byref(ev0)))
    pkg._capi.check(lib.axr_event_create(C.byref(ev1)))
    pkg._capi.check(lib.axr_event_record(ev0, s1))
    plan.pack(p1.data_ptr(), n, s1.value)
    pkg._capi.check(lib.axr_event_record(ev1, s1))
    pkg._capi.check(lib.axr_event_synchronize(ev1))
    ms = C.c_float()
    pkg._capi.check(lib.axr_event_elapsed_ms(ev0, ev1, C.byref(ms)))
    assert ms.value > 0
    for h in (ev0, ev1):
        pkg._capi.check(lib.axr_event_destroy(h))
    plan.close()
    for s in (s1, s2):
        pkg._capi.check(lib.axr_stream_destroy(s))


def test_block_cache_gives_memory_back_after_a_burst(pkg, orc, gpu):
    """Forty live plans with 9 MiB of host tensors hold two pinned staging blocks each (4 and
    8 MiB: 480 MiB, more than the 256 MiB the recycling list keeps); freeing them returns the
    excess to the driver, and planning goes on as before."""
    import torch
    rng = np.random.default_rng(3)
    host = [rng.integers(0, 256, size=3 << 20, dtype=np.uint8) for _ in range(3)]
    dev = rand_bytes_tensor(rng, 5000, gpu)
    tensors = [host[0], dev, host[1], host[2]]
    want = orc.pack([np.ascontiguousarray(t).reshape(-1) if isinstance(t, np.ndarray) else tbytes(t)
                     for t in tensors], 256)
    plans, payloads = [], []
    for _ in range(40):
        plan = pkg.BundlePlan.create(tensors, align=256)
        buf = device_bytes(plan.payload_bytes, gpu)
        plan.pack(buf.data_ptr(), plan.payload_bytes)
        plans.append(plan)
        payloads.append(buf)
    torch.cuda.synchronize()
    for plan, buf in zip(plans, payloads):
        assert np.array_equal(buf.cpu().numpy()[:plan.payload_bytes], want)
        plan.close()
    for _ in range(3):                                       # blocks come from the list again
        got, plan, _ = run_pack(pkg, tensors, 256, gpu)
        assert np.array_equal(got, want)
        plan.close()


def test_plan_outlives_a_stream_it_ran_on(pkg, orc, gpu):
    """A plan drains the streams it ran on before its tables are rewritten or
    released.  A stream destroyed with axr_stream_destroy in the meantime must not
    be touched again: rebinding and freeing such a plan used to crash the process."""
    lib = pkg._capi.load()
    rng = np.random.default_rng(9)
    a = [rand_bytes_tensor(rng, n, gpu) for n in (70000, 33, 4096)]
    b = [rand_bytes_tensor(rng, n, gpu) for n in (70000, 33, 4096)]
    want_a = orc.pack([tbytes(t) for t in a], 256)
    want_b = orc.pack([tbytes(t) for t in b], 256)
    for then in ("free", "rebind"):
        plan = pkg.BundlePlan.create(a, align=256)
        n = plan.payload_bytes
        out = device_bytes(n, gpu)
        s = C.c_void_p()
        pkg._capi.check(lib.axr_stream_create(C.byref(s)))
        plan.pack(out.data_ptr(), n, s.value)
        pkg._capi.check(lib.axr_stream_synchronize(s))
        assert np.array_equal(out.cpu().numpy()[:n], want_a)
        pkg._capi.check(lib.axr_stream_destroy(s))
        if then == "rebind":
            plan.bind(b)
            plan.pack(out.data_ptr(), n, None)
            pkg._capi.check(lib.axr_device_synchronize())
            assert np.array_equal(out.cpu().numpy()[:n], want_b)
        plan.close()


def test_small_bundles_with_tables_in_the_kernel_arguments(pkg, orc, gpu):
    """Small bundles travel with their tables inside the kernel arguments; the same
    bundles with that switched off use an uploaded table block.  Both must give the
    oracle's bytes: plain tensors with pads, strided rows, short strided runs,
    transposed views, and a mix with a host tensor.  A plan launched this way can be
    captured in a graph without axr_plan_prepare, and freed once the capture has ended."""
    import torch
    rng = np.random.default_rng(55)

    def rb(n):
        return rand_bytes_tensor(rng, n, gpu)
    mat = rb(2 * 96 * 80).view(torch.int16).reshape(96, 80)
    rows = rb(4 * 40 * 1024).view(torch.float32).reshape(40, 1024)
    cases = {
        "plain": [rb(5000), rb(1), rb(70001), rb(0), rb(4096)],
        "strided rows": [rows[:, :600], rb(33)],                      # 2400-byte runs: run tiles
        "short runs": [rows[:, 5:45], mat[::2, 3:70]],                # element mode
        "transposed": [mat.t(), rows[:, :64].t(), rb(100)],
        "with a host tensor": [rb(3000), torch.from_numpy(rng.integers(0, 256, 5000, dtype=np.uint8)), rb(17)],
    }
    for name, tensors in cases.items():
        want = orc.pack([tbytes(t) for t in tensors], 256)
        for inline in (16384, 0):
            pkg.tune(inline_tables=inline)
            try:
                plan = pkg.BundlePlan.create(tensors, align=256)
                assert plan.launch_info()["inline_tables"] == (1 if inline else 0), name
                n, header = plan.payload_bytes, plan.header
                payload = device_bytes(n, gpu)
                plan.pack(payload.data_ptr(), n)
                plan.close()                                           # waits for the launch
                torch.cuda.synchronize()
                assert np.array_equal(payload.cpu().numpy()[:n], want), (name, inline)
                outs = [torch.zeros(t.shape, dtype=t.dtype, device=t.device) for t in tensors]
                back = pkg.BundlePlan.from_header(header).bind(outs)
                assert back.launch_info()["inline_tables"] == (1 if inline else 0), name
                back.unpack(payload.data_ptr(), n)
                torch.cuda.synchronize()
                back.close()
                for o, t in zip(outs, tensors):
                    assert np.array_equal(tbytes(o), tbytes(t)), (name, inline)
            finally:
                pkg.tune(inline_tables=16384)

    # capture without prepare: the launch carries everything it needs
    tensors = cases["short runs"] + cases["plain"]
    want = orc.pack([tbytes(t) for t in tensors], 256)
    plan = pkg.BundlePlan.create(tensors, align=256)
    assert plan.launch_info()["inline_tables"] == 1
    n = plan.payload_bytes
    payload = device_bytes(n, gpu)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        plan.pack(payload.data_ptr(), n, side.cuda_stream)
    plan.close()                                                       # the graph keeps its own copy
    for _ in range(3):
        payload.fill_(POISON)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(payload.cpu().numpy()[:n], want)


def test_pack_and_unpack_in_a_hip_graph(pkg, orc, gpu):
    """A prepared plan's pack and unpack are single kernel launches that stream
    capture can record.  The graph is replayed several times with eager work and
    synchronisations in between, and every replay is checked against the oracle
    for the tensors' contents at that moment."""
    import torch
    rng = np.random.default_rng(77)
    sizes = [int(x) for x in rng.integers(1, 50000, size=120)]
    tensors = [rand_bytes_tensor(rng, n, gpu) for n in sizes]
    mat = rand_bytes_tensor(rng, 2 * 200 * 136, gpu).view(torch.int16).reshape(200, 136)
    tensors += [mat.t(), mat[:, 8:72]]                       # transposed blocks (LDS) and short runs
    outs = [torch.zeros_like(t, memory_format=torch.contiguous_format) for t in tensors]
    plan = pkg.BundlePlan.create(tensors, align=256)
    n = plan.payload_bytes
    buf = device_bytes(n, gpu)
    rplan = pkg.BundlePlan.from_header(plan.header).bind(outs)
    side = torch.cuda.Stream()

    # an unprepared plan refuses to be captured and records nothing
    g0 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g0, stream=side):
        with pytest.raises(pkg.AxonRocmError):
            plan.pack(buf.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    del g0

    plan.prepare()
    rplan.prepare()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        handle = torch.cuda.current_stream().cuda_stream
        plan.pack(buf.data_ptr(), n, handle)
        rplan.unpack(buf.data_ptr(), n, handle)
    for replay in range(4):
        # eager work between replays: new contents, poisoned payload and outputs
        for t in tensors[:120]:
            t.add_(replay + 1)
        mat.add_(replay + 3)
        buf.fill_(POISON)
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        chunks = [tbytes(t) for t in tensors]
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(buf.cpu().numpy()[:n], orc.pack(chunks, 256)), replay
        for o, c in zip(outs, chunks):
            assert np.array_equal(tbytes(o), c), replay
    # the same plans still work eagerly afterwards
    buf.fill_(POISON)
    plan.pack(buf.data_ptr(), n)
    torch.cuda.synchronize()
    assert np.array_equal(buf.cpu().numpy()[:n], orc.pack([tbytes(t) for t in tensors], 256))
    del graph
    plan.close()
    rplan.close()


def test_error_paths(pkg, gpu):
    import torch
    a = [torch.zeros(100, device=gpu), torch.zeros(7, device=gpu)]
    plan = pkg.BundlePlan.create(a, align=256)
    buf = device_bytes(1024, gpu)
    with pytest.raises(pkg.LengthError):
        plan.pack(buf.data_ptr(), plan.payload_bytes - 1)
    with pytest.raises(pkg.LengthError):
        plan.split(buf.data_ptr(), 10)
    r = pkg.BundlePlan.from_header(plan.header)
    with pytest.raises(pkg.AxonRocmError):
        r.unpack(buf.data_ptr(), plan.payload_bytes)              # nothing bound yet
    with pytest.raises(pkg.MismatchError):
        r.bind([torch.zeros(100, device=gpu)])
    with pytest.raises(pkg.MismatchError):
        r.bind([torch.zeros(100, device=gpu), torch.zeros(8, device=gpu)])
    with pytest.raises(pkg.AxonRocmError):                        # overlapping destination
        r.bind([torch.zeros(1, device=gpu).expand(100), torch.zeros(7, device=gpu)])
        r.unpack(buf.data_ptr(), plan.payload_bytes)
    hdr = bytearray(plan.header)
    hdr[0] ^= 0xFF
    with pytest.raises(pkg.HeaderError):
        pkg.BundlePlan.from_header(bytes(hdr))
    # empty bundles are legal and move nothing
    empty = pkg.BundlePlan.create([], align=1)
    assert empty.payload_bytes == 0
    empty.pack(0, 0)
    zero = pkg.BundlePlan.create([torch.zeros(0, device=gpu), torch.zeros((), device=gpu)], align=256)
    assert zero.payload_bytes == 0 and zero.layout() == ([0, 0], [0, 0])
    zero.pack(0, 0)


def test_tensor_larger_than_4_gib(pkg, gpu):
    """64-bit offsets end to end: one 5 GiB tensor next to small ones."""
    import torch
    n = 5 * (1 << 30) + 12345
    big = torch.empty(n, dtype=torch.uint8, device=gpu)
    big[: n // 8 * 8].view(torch.int64).random_()
    big[n - 12345:] = 7
    small = torch.arange(1000, device=gpu, dtype=torch.int32)
    plan = pkg.BundlePlan.create([small, big, small], align=256)
    info = plan.launch_info()
    assert info["tiles"] * info["tile_bytes"] >= n and info["tile_bytes"] > 2048
    payload = torch.empty(plan.payload_bytes, dtype=torch.uint8, device=gpu)
    plan.pack(payload.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    offs, sizes = plan.layout()
    assert sizes[1] == n and offs[2] == offs[1] + (n + 255) // 256 * 256
    assert torch.equal(payload[offs[1]:offs[1] + n], big)
    assert torch.equal(payload[offs[2]:offs[2] + 4000].view(torch.int32), small)
    out_big = torch.zeros_like(big)
    outs = [torch.zeros_like(small), out_big, torch.zeros_like(small)]
    pkg.BundlePlan.from_header(plan.header).bind(outs).unpack(payload.data_ptr(), plan.payload_bytes)
    torch.cuda.synchronize()
    assert torch.equal(out_big, big) and torch.equal(outs[0], small) and torch.equal(outs[2], small)


def test_concurrent_host_threads(pkg, orc, gpu):
    """Plans, packs and pool traffic from several host threads at once (the UCX
    worker thread, thread-pool threads and Python threads all use one manager)."""
    import threading
    import torch
    lib = pkg._capi.load()
    errors = []

    def worker(seed):
        try:
            rng = np.random.default_rng(seed)
            s = C.c_void_p()
            pkg._capi.check(lib.axr_stream_create(C.byref(s)))
            for it in range(25):
                sizes = [int(x) for x in rng.integers(1, 50000, size=30)]
                host = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in sizes]
                with torch.cuda.stream(torch.cuda.ExternalStream(s.value)):
                    tensors = [torch.from_numpy(a).to(gpu, non_blocking=False) for a in host]
                packed = pkg.pack_bundle(tensors, align=256, stream=s.value)
                pkg._capi.check(lib.axr_stream_synchronize(s))
                back = np.zeros(packed.payload_bytes, np.uint8)
                pkg._capi.check(lib.axr_memcpy(0, back.ctypes.data, 3, packed.payload.data, back.size))
                if not np.array_equal(back, orc.pack(host, 256)):
                    errors.append(f"thread {seed} iteration {it}: payload differs")
                packed.plan.close()
                packed.payload.release()
            pkg._capi.check(lib.axr_stream_destroy(s))
        except Exception as ex:   # noqa: BLE001
            errors.append(repr(ex))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


# ------------------------------------------------------------------ memory resource

def test_large_copy_to_pageable_host_memory(pkg, gpu):
    """axr_memcpy between the device and pageable memory goes through pinned staging
    blocks from 16 MiB on, in both directions: three whole blocks and an odd tail,
    and the sizes around the switch."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    for n in ((16 << 20) - 1, 16 << 20, (24 << 20) + 12345, (40 << 20) + 7):
        dev = torch.randint(0, 256, (n,), dtype=torch.uint8, device=gpu)
        host = np.full(n + 64, 0xEE, dtype=np.uint8)
        capi.check(lib.axr_memcpy(capi.MEM_HOST, host.ctypes.data + 32, capi.MEM_ROCM, dev.data_ptr(), n))
        assert np.array_equal(host[32:32 + n], dev.cpu().numpy()), n
        assert (host[:32] == 0xEE).all() and (host[32 + n:] == 0xEE).all()
        # and back from pageable memory, staged from the same size on
        back = torch.full((n + 64,), 0x11, dtype=torch.uint8, device=gpu)
        capi.check(lib.axr_memcpy(capi.MEM_ROCM, back.data_ptr() + 32, capi.MEM_HOST, host.ctypes.data + 32, n))
        got = back.cpu().numpy()
        assert np.array_equal(got[32:32 + n], host[32:32 + n]), n
        assert (got[:32] == 0x11).all() and (got[32 + n:] == 0x11).all()


def test_pool_and_copy_table(pkg, gpu):
    import torch
    registered = []
    pool = pkg.DevicePool(device=0, slab_bytes=4 << 20)
    pool.set_registrar(lambda addr, n: (registered.append((addr, n)) or 0xABC0 + len(registered)),
                       lambda h: registered.append(("unreg", h)))
    x = pool.alloc(1000)
    y = pool.alloc(3 << 20, alignment=4096)
    z = pool.alloc(8 << 20)                                       # larger than a slab: own slab
    assert x.data % 256 == 0 and y.data % 4096 == 0
    assert x.mem_h == 0xABC1 and y.mem_h == 0xABC1 and z.mem_h == 0xABC2
    st = pool.stats()
    assert st["slabs"] == 2 and st["live_blocks"] == 3
    x_addr = x.data
    x.release()
    x2 = pool.alloc(1000)
    assert x2.data == x_addr                                      # freed block is reused
    for blk in (x2, y, z):
        blk.release()
    assert pool.stats()["allocated_bytes"] == 0
    pool.trim()
    assert pool.stats()["slabs"] == 0
    assert sorted(r for r in registered if r[0] == "unreg") == [("unreg", 0xABC1), ("unreg", 0xABC2)]
    pool.close()

    mr = pkg.RocmMemoryResourceManager()
    HOST, ROCM, PINNED = 0, 3, 4
    src = np.arange(100000, dtype=np.uint8)
    d = mr.allocate(ROCM, src.size)
    p = mr.allocate(PINNED, src.size)
    back = np.zeros_like(src)
    mr.memcpy(ROCM, d, HOST, src.ctypes.data, src.size)          # H2D
    mr.memcpy(PINNED, p, ROCM, d, src.size)                      # D2H into pinned
    mr.memcpy(HOST, back.ctypes.data, PINNED, p, src.size)       # H2H
    assert np.array_equal(src, back)
    d2 = mr.allocate(ROCM, src.size)
    mr.memcpy(ROCM, d2, ROCM, d, src.size)                        # D2D
    back[:] = 0
    mr.memcpy(HOST, back.ctypes.data, ROCM, d2, src.size)
    assert np.array_equal(src, back)
    with pytest.raises(pkg.UnsupportedMemoryError):
        mr.allocate(1, 16)                                        # ucx_memory_type::CUDA
    with pytest.raises(pkg.UnsupportedMemoryError):
        mr.memcpy(1, d, HOST, src.ctypes.data, 16)
    for t, ptr in ((ROCM, d), (ROCM, d2), (PINNED, p)):
        mr.deallocate(t, ptr, src.size)
    with pkg.rocm(0).activate() as devobj:
        assert devobj.get_type_string() == "rocm" and devobj.get_context_handle() == 0


def test_shaped_copy_reference_kernel(pkg, gpu):
    """The calibration copy in every wavefront shape copies exactly its range and refuses
    shapes and sizes it does not cover."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    n = 3 * 4096 * 37
    src = torch.randint(0, 256, (n + 64,), dtype=torch.uint8, device=gpu)
    for threads in (64, 128, 256, 1024):
        for kib in (1, 2, 4):
            for nt in (0, 1):
                dst = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
                torch.cuda.synchronize()
                capi.check(lib.axr_copy_reference_shaped(dst.data_ptr(), src.data_ptr(), n, threads, kib, nt, None))
                torch.cuda.synchronize()
                assert torch.equal(dst[:n], src[:n]) and bool((dst[n:] == POISON).all()), (threads, kib, nt)
    for bad in ((n, 96, 1), (n, 64, 3), (n + 1024, 64, 4), (n, 2048, 1)):
        assert lib.axr_copy_reference_shaped(dst.data_ptr(), src.data_ptr(), bad[0], bad[1], bad[2], 1, None) == capi.AXR_ERR_INVALID
    assert lib.axr_copy_reference_shaped(dst.data_ptr(), src.data_ptr(), 0, 64, 1, 1, None) == 0


@pytest.mark.parametrize("nontemporal", [0, 3])
def test_rows_reference_kernel(pkg, gpu, nontemporal):
    """The plain row gather / scatter kernel (the calibration reference of the strided modes)
    against numpy slicing: ragged and exact row lengths, rows that fill their pitch, and a
    scatter that leaves every byte between the rows alone."""
    import torch
    lib, check = pkg._capi.load(), pkg._capi.check
    rng = np.random.default_rng(17)
    for run, pitch, rows in ((100, 256, 1000), (250, 1024, 333), (16, 16, 7), (4096, 4100, 5),
                             (48, 64, 129), (17, 33, 1025), (2049, 2304, 3), (128, 128, 4097)):
        host = rng.integers(0, 256, size=rows * pitch, dtype=np.uint8)
        strided = torch.from_numpy(host).to(gpu)
        packed = device_bytes(rows * run + 32, gpu)
        check(lib.axr_rows_reference(strided.data_ptr(), pitch, packed.data_ptr(), run, rows, 0, nontemporal, None))
        torch.cuda.synchronize()
        want = host.reshape(rows, pitch)[:, :run].reshape(-1)
        got = packed.cpu().numpy()
        assert np.array_equal(got[:rows * run], want), (run, pitch, rows)
        assert (got[rows * run:] == POISON).all()
        twin = device_bytes(rows * pitch, gpu, fill=0xAB)
        check(lib.axr_rows_reference(twin.data_ptr(), pitch, packed.data_ptr(), run, rows, 1, nontemporal, None))
        torch.cuda.synchronize()
        expect = np.full(rows * pitch, 0xAB, np.uint8)
        expect.reshape(rows, pitch)[:, :run] = want.reshape(rows, run)
        assert np.array_equal(twin.cpu().numpy(), expect), (run, pitch, rows)
    with pytest.raises(Exception):
        check(lib.axr_rows_reference(strided.data_ptr(), 8, packed.data_ptr(), 16, 1, 0, 0, None))


@pytest.mark.parametrize("nontemporal", [-1, 3, 0])
def test_short_rows_of_every_length(pkg, orc, gpu, nontemporal):
    """Element mode over its whole range of run lengths: every length from 16 to 160 bytes and
    a few up to the crossover with run tiles, enough rows for several work units (so that units
    begin inside a run whenever the lane slots per run do not divide 512), with one and with two
    strided dimensions, bases and pitches on and off the 16-byte grid, and every cache-hint
    setting.  Gather against numpy slicing (the oracle for a sample), scatter into poisoned twins."""
    import torch
    rng = np.random.default_rng(31 + nontemporal)
    lengths = list(range(16, 161)) + [250, 500, 1001, 1279]
    pkg.tune(nontemporal=nontemporal)
    try:
        for batch in range(0, len(lengths), 25):
            cases = []
            for run in lengths[batch:batch + 25]:
                pitch = run + int(rng.choice([0, 1, 7, 16, 100, 256 - run % 256]))
                rows = int(rng.integers(600, 1400))
                lead = int(rng.choice([0, 1, 3, 16]))
                if rng.random() < 0.4:                       # two strided dimensions: [planes, rows, run]
                    planes = int(rng.integers(2, 5))
                    host = rng.integers(0, 256, size=lead + planes * (rows + 3) * pitch, dtype=np.uint8)
                    dev = torch.from_numpy(host).to(gpu)
                    view = dev[lead:].reshape(planes, rows + 3, pitch)[:, 1:rows + 1, :run]
                    want = host[lead:].reshape(planes, rows + 3, pitch)[:, 1:rows + 1, :run]
                else:
                    host = rng.integers(0, 256, size=lead + rows * pitch, dtype=np.uint8)
                    dev = torch.from_numpy(host).to(gpu)
                    view = dev[lead:].reshape(rows, pitch)[:, :run]
                    want = host[lead:].reshape(rows, pitch)[:, :run]
                cases.append((host, dev, view, np.ascontiguousarray(want).reshape(-1)))
            views = [c[2] for c in cases]
            chunks = [c[3] for c in cases]
            host0, _, v0, c0 = cases[0]
            assert np.array_equal(c0, orc.gather_strided(host0, v0.storage_offset(), tuple(v0.shape),
                                                         tuple(v0.stride()), 1))
            for align in (1, 256):
                got, plan, buf = run_pack(pkg, views, align, gpu)
                modes = [s["mode"] for s in plan.segments()]      # pitch == run: one contiguous run
                assert set(modes) <= {0, 1, 2} and modes.count(2) >= len(modes) // 2, modes
                assert np.array_equal(got, orc.pack(chunks, align)), (batch, align)
                twins = [device_bytes(c[1].numel(), gpu, fill=0x5C) for c in cases]
                tviews = [t.as_strided(c[2].shape, c[2].stride(), c[2].storage_offset())
                          for t, c in zip(twins, cases)]
                pkg.BundlePlan.from_header(plan.header).bind(tviews).unpack(buf.data_ptr(), plan.payload_bytes)
                torch.cuda.synchronize()
                for twin, (host, _, view, chunk) in zip(twins, cases):
                    expect = np.full(host.size, 0x5C, np.uint8)
                    orc.scatter_strided(chunk, expect, view.storage_offset(), tuple(view.shape),
                                        tuple(view.stride()), 1)
                    assert np.array_equal(twin.cpu().numpy(), expect), (batch, align, tuple(view.shape))
    finally:
        pkg.tune(nontemporal=-1)


@pytest.mark.parametrize("dtype_name", ["uint8", "int16", "float32", "float64", "complex128"])
def test_transposed_views_of_random_extents(pkg, orc, gpu, dtype_name):
    """Transposed matrices whose extents fall anywhere around the block edge: shorter than a
    block, one element past a whole number of blocks, one short of it (the last block of such
    a dimension is moved back over its neighbour and stays on the vector path), with row
    pitches and bases off every power-of-two grid.  Gather against the oracle, scatter into
    poisoned twins."""
    import torch
    dt = getattr(torch, dtype_name)
    item = torch.empty((), dtype=dt).element_size()
    t = (128 if item <= 4 else 256) // item
    rng = np.random.default_rng(500 + item)
    extents = [1, 2, t - 1, t, t + 1, 2 * t - 1, 2 * t + 1, 3 * t - 5, int(rng.integers(1, 3 * t)),
               int(rng.integers(1, 3 * t))]
    cases = []
    for _ in range(14):
        rows, cols = int(rng.choice(extents)), int(rng.choice(extents))
        pad_r, pad_c = int(rng.integers(0, 3)), int(rng.integers(0, 4))
        parent = rand_bytes_tensor(rng, (rows + pad_r) * (cols + pad_c) * item, gpu).view(dt).reshape(rows + pad_r, cols + pad_c)
        cases.append((parent, parent[pad_r:, pad_c:].t()))
    b = rand_bytes_tensor(rng, 3 * (t + 3) * (2 * t + 1) * item, gpu).view(dt).reshape(3, t + 3, 2 * t + 1)
    cases.append((b, b.transpose(1, 2)))                       # a batch of ragged transposes
    views = [v for _, v in cases]
    chunks = []
    for parent, v in cases:
        host_parent = parent.reshape(-1).view(torch.uint8).cpu().numpy()
        chunks.append(orc.gather_strided(host_parent, (v.data_ptr() - parent.data_ptr()),
                                         tuple(v.shape), tuple(v.stride()), item))
    for align in (256, 1):
        got, plan, buf = run_pack(pkg, views, align, gpu)
        assert np.array_equal(got, orc.pack(chunks, align)), align
        twins = [device_bytes(p.numel() * item, gpu, fill=0x3B).view(dt).reshape(p.shape) for p, _ in cases]
        tviews = [tw.as_strided(v.shape, v.stride(), v.storage_offset()) for tw, (_, v) in zip(twins, cases)]
        pkg.BundlePlan.from_header(plan.header).bind(tviews).unpack(buf.data_ptr(), plan.payload_bytes)
        torch.cuda.synchronize()
        for tw, (parent, v), c in zip(twins, cases, chunks):
            expect = np.full(parent.numel() * item, 0x3B, np.uint8)
            orc.scatter_strided(c, expect, v.data_ptr() - parent.data_ptr(), tuple(v.shape), tuple(v.stride()), item)
            assert np.array_equal(tw.reshape(-1).view(torch.uint8).cpu().numpy(), expect), (align, tuple(v.shape))


def test_polled_stream_wait(pkg, orc, gpu):
    """axr_stream_synchronize with "spin_wait_us": the wait that polls a word of pinned memory
    returns only when the stream's work is done (a pack's payload is complete right after it),
    a budget too short for the kernel falls back to the runtime's wait with the same result,
    and plans freed afterwards do not trip over the notify kernels."""
    import torch
    lib, check = pkg._capi.load(), pkg._capi.check
    rng = np.random.default_rng(12)
    stream = C.c_void_p()
    check(lib.axr_stream_create(C.byref(stream)))
    big = [rand_bytes_tensor(rng, 64 << 20, gpu) for _ in range(4)]        # a launch of ~100 us
    small = [rand_bytes_tensor(rng, int(n), gpu) for n in rng.integers(1, 5000, size=9)]
    want_big = orc.pack([t.cpu().numpy() for t in big], 256)
    want_small = orc.pack([t.cpu().numpy() for t in small], 256)
    torch.cuda.synchronize()
    try:
        for budget in (200, 1, 0):
            pkg.tune(spin_wait_us=budget)
            for tensors, want in ((big, want_big), (small, want_small)):
                for _ in range(3):
                    plan = pkg.BundlePlan.create(tensors, align=256)
                    buf = device_bytes(plan.payload_bytes, gpu)
                    torch.cuda.synchronize()
                    plan.pack(buf.data_ptr(), plan.payload_bytes, stream.value)
                    check(lib.axr_stream_synchronize(stream))
                    host = torch.empty(plan.payload_bytes, dtype=torch.uint8).pin_memory()
                    host.copy_(buf)                            # a blocking copy on another stream: no extra wait for ours
                    plan.close()
                    assert np.array_equal(host.numpy(), want), (budget, len(tensors))
        # A scatter into pinned host tensors: the kernel writes host memory, which the runtime's
        # wait makes visible and the polled wait does not promise to; the stream's next wait is
        # therefore the runtime's, whatever the budget, and the CPU reads the data at once.
        pkg.tune(spin_wait_us=200)
        plan = pkg.BundlePlan.create(small, align=256)
        buf = device_bytes(plan.payload_bytes, gpu)
        torch.cuda.synchronize()
        plan.pack(buf.data_ptr(), plan.payload_bytes, stream.value)
        pinned = [torch.zeros(t.numel(), dtype=torch.uint8).pin_memory() for t in small]
        views = [pkg.TensorView(data=p.data_ptr(), device_type=11, device_id=0, dtype=(1, 8, 1),
                                shape=(p.numel(),), strides=None, owner=p) for p in pinned]
        rplan = pkg.BundlePlan.from_header(plan.header).bind(views)
        assert {s["mode"] for s in rplan.segments()} <= {0, 6}        # device segments: the kernel writes them
        for _ in range(5):
            for t in pinned:
                t.zero_()
            rplan.unpack(buf.data_ptr(), plan.payload_bytes, stream.value)
            check(lib.axr_stream_synchronize(stream))
            for t, src in zip(pinned, small):
                assert np.array_equal(t.numpy(), src.cpu().numpy())
        rplan.close()
        plan.close()
    finally:
        pkg.tune(spin_wait_us=0)
        check(lib.axr_stream_destroy(stream))


def test_die_contiguous_tile_ranges(pkg, orc, gpu):
    """"xcd_remap": every die walks one contiguous share of the tiles.  Forced on for a mixed
    bundle, and chosen automatically for a bundle of transposed views whose rows straddle
    128-byte lines (there the grid is rounded up to a multiple of the eight dies); both
    against the oracle, pack and unpack."""
    import torch
    rng = np.random.default_rng(808)
    mixed = [rand_bytes_tensor(rng, int(n), gpu) for n in rng.integers(1, 40000, size=700)]
    mixed.append(rand_bytes_tensor(rng, 300 * 1000, gpu).reshape(300, 1000)[:, :333])      # element mode
    odd = [rand_bytes_tensor(rng, 700 * 650 * 2, gpu).view(torch.int16).reshape(700, 650).t() for _ in range(2)]
    for views, tune, expect_rounded in ((mixed, 1, True), (odd, -1, True), (odd, 0, False)):
        pkg.tune(xcd_remap=tune)
        try:
            chunks = [tbytes(v) for v in views]
            got, plan, buf = run_pack(pkg, views, 256, gpu)
            info = plan.launch_info()
            assert info["workgroups"] >= 32
            assert (info["workgroups"] % 8 == 0) == expect_rounded or not expect_rounded, info
            assert np.array_equal(got, orc.pack(chunks, 256)), tune
            twins = [torch.zeros_like(v._base if v._base is not None else v) for v in views]
            tviews = [tw.as_strided(v.shape, v.stride(), v.storage_offset()) for tw, v in zip(twins, views)]
            pkg.BundlePlan.from_header(plan.header).bind(tviews).unpack(buf.data_ptr(), plan.payload_bytes)
            torch.cuda.synchronize()
            for v, tv_ in zip(views, tviews):
                assert np.array_equal(tbytes(v), tbytes(tv_)), tune
        finally:
            pkg.tune(xcd_remap=-1)


def test_zero_dim_tensors_take_no_payload_bytes(pkg, orc, gpu):
    """The reference's size rule gives a 0-d tensor no bytes (rpc_core/utils/tensor_meta.hpp:91-104):
    it gets an offset and a header record, nothing is moved for it, a destination bound for it
    stays as it was, and a zero-copy view of it reads a zero of its own, not what follows its
    offset in the payload (here: the end of the payload)."""
    import torch
    a = torch.arange(64, dtype=torch.float32, device=gpu)
    scalar = torch.tensor(7.5, device=gpu)
    tensors = [a, scalar]
    for align in (1, 256):
        got, plan, buf = run_pack(pkg, tensors, align, gpu)
        assert plan.payload_bytes == 256 and np.array_equal(got, orc.pack([tbytes(a), np.zeros(0, np.uint8)], align))
        metas = plan.metas()
        assert metas[1].shape == () and metas[1].nbytes == 0 and metas[1].offset == 256
        outs = [torch.zeros_like(a), torch.tensor(-1.0, device=gpu)]
        rplan = pkg.unpack_bundle(plan.header, buf.data_ptr(), payload_bytes=plan.payload_bytes, out=outs)
        rplan.close()
        assert torch.equal(outs[0], a) and float(outs[1]) == -1.0
        views = pkg.unpack_bundle(plan.header, buf.data_ptr(), payload_bytes=plan.payload_bytes,
                                  from_dlpack_fn=torch.from_dlpack)
        assert torch.equal(views[0], a) and views[1].shape == () and float(views[1]) == 0.0
        del views
        plan.close()


def test_read_only_host_sources(pkg, orc, gpu):
    """Host arrays that may not be written (over bytes, broadcast) are packed like any other
    source and come back in writable destinations."""
    frozen = np.frombuffer(bytes(range(200)) * 50, dtype=np.uint8)
    spread = np.broadcast_to(np.arange(5, dtype=np.float32), (7, 5))
    plain = np.arange(33, dtype=np.int16)
    sources = [plain, frozen, spread]
    bundle = pkg.pack_bundle(sources, align=256)
    chunks = [np.ascontiguousarray(x).view(np.uint8).reshape(-1) for x in sources]
    payload = pkg.bundle_to_host(bundle.header, bundle.payload, payload_bytes=bundle.payload_bytes)
    for got, want in zip(payload, chunks):
        assert np.array_equal(got, want)
    outs = [np.zeros_like(plain), np.zeros(frozen.shape, np.uint8), np.zeros((7, 5), np.float32)]
    plan = pkg.unpack_bundle(bundle.header, bundle.payload, payload_bytes=bundle.payload_bytes, out=outs)
    plan.close()
    for out, src in zip(outs, sources):
        assert np.array_equal(out, src)
    with pytest.raises(BufferError, match="read-only"):
        pkg.unpack_bundle(bundle.header, bundle.payload, payload_bytes=bundle.payload_bytes,
                          out=[np.zeros_like(plain), frozen, np.zeros((7, 5), np.float32)])
    bundle.close()
