"""axr_pack_noalloc (the pack entry point that allocates nothing) against axr_pack,
through the C ABI: byte-identical payloads on two calls in a row on one stream,
the second with a smaller bundle, so that the second call's tables overwrite the
first call's in the shared static table area while nothing waits in between.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xCD


def make_bundle(gpu, rng, count, strided_every):
    """`count` device tensors of 16 B .. 24 KiB in four dtypes; every
    `strided_every`-th one is a pitched 2-D view (strided segments add Dims records)."""
    import torch
    dtypes = [torch.uint8, torch.float16, torch.float32, torch.int64]
    tensors = []
    for i in range(count):
        dt = dtypes[i % 4]
        item = torch.empty((), dtype=dt).element_size()
        if strided_every and i % strided_every == 0:
            rows, cols, pitch = int(rng.integers(2, 9)), int(rng.integers(1, 400)), 512
            raw = torch.from_numpy(rng.integers(0, 256, size=rows * pitch * item, dtype=np.uint8)).to(gpu)
            tensors.append(raw.view(dt).reshape(rows, pitch)[:, :cols])
        else:
            n = max(1, int(np.exp(rng.uniform(np.log(16), np.log(24 * 1024)))) // item)
            raw = torch.from_numpy(rng.integers(0, 256, size=n * item, dtype=np.uint8)).to(gpu)
            tensors.append(raw.view(dt))
    return tensors


def host_chunks(tensors):
    import torch
    out = []
    for t in tensors:
        c = torch.empty(t.shape, dtype=t.dtype, device=t.device)
        c.copy_(t)
        out.append(c.reshape(-1).view(torch.uint8).cpu().numpy())
    return out


@pytest.mark.parametrize("align", [1, 256])
def test_two_calls_in_a_row_match_axr_pack(pkg, orc, gpu, align):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(2024 + align)
    big = make_bundle(gpu, rng, 1500, strided_every=7)
    small = make_bundle(gpu, rng, 300, strided_every=5)
    stream = C.c_void_p()
    capi.check(lib.axr_stream_create(C.byref(stream)))
    plans, bufs = [], []
    try:
        for tensors in (big, small):
            plan = pkg.BundlePlan.create(tensors, align=align)
            info = plan.launch_info()
            # both bundles are past what the kernel arguments hold: the static area is used
            assert info["inline_tables"] == 0 and 3584 < info["table_bytes"] <= (1 << 20)
            n = plan.payload_bytes
            buf = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
            plans.append(plan)
            bufs.append(buf)
        # the inputs and the poisoned buffers were produced on torch's stream: the launch stream
        # is ordered behind it with an event (no host wait), then two calls back to back
        assert pkg.streams.order_behind_producers(stream.value)
        for plan, buf in zip(plans, bufs):
            capi.check(lib.axr_pack_noalloc(plan._h, buf.data_ptr(), plan.payload_bytes, stream))
        capi.check(lib.axr_stream_synchronize(stream))
        for tensors, plan, buf in zip((big, small), plans, bufs):
            n = plan.payload_bytes
            got = buf.cpu().numpy()
            assert (got[n:] == POISON).all()
            # the existing entry point, on a plan of its own
            ref_plan = pkg.BundlePlan.create(tensors, align=align)
            ref = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
            ref_plan.pack(ref.data_ptr(), n, stream.value)
            capi.check(lib.axr_stream_synchronize(stream))
            assert np.array_equal(got[:n], ref.cpu().numpy()[:n])
            assert np.array_equal(got[:n], orc.pack(host_chunks(tensors), align))
            ref_plan.close()
        # a third call on the first plan again: the area holds the small bundle's tables by now
        bufs[0].fill_(POISON)
        torch.cuda.synchronize()
        capi.check(lib.axr_pack_noalloc(plans[0]._h, bufs[0].data_ptr(), plans[0].payload_bytes, stream))
        capi.check(lib.axr_stream_synchronize(stream))
        n = plans[0].payload_bytes
        assert np.array_equal(bufs[0].cpu().numpy()[:n], orc.pack(host_chunks(big), align))
        # calls on TWO streams share the one table area: the second stream is made to wait for
        # the first one's launch on the device, so alternating calls without any host wait
        # still give each bundle its own tables
        other = C.c_void_p()
        capi.check(lib.axr_stream_create(C.byref(other)))
        for buf in bufs:
            buf.fill_(POISON)
        assert pkg.streams.order_behind_producers(stream.value)
        assert pkg.streams.order_behind_producers(other.value)
        for _ in range(4):
            capi.check(lib.axr_pack_noalloc(plans[0]._h, bufs[0].data_ptr(), plans[0].payload_bytes, stream))
            capi.check(lib.axr_pack_noalloc(plans[1]._h, bufs[1].data_ptr(), plans[1].payload_bytes, other))
        capi.check(lib.axr_stream_synchronize(stream))
        capi.check(lib.axr_stream_synchronize(other))
        for tensors, plan, buf in zip((big, small), plans, bufs):
            n = plan.payload_bytes
            got = buf.cpu().numpy()
            assert np.array_equal(got[:n], orc.pack(host_chunks(tensors), align)) and (got[n:] == POISON).all()
        capi.check(lib.axr_stream_destroy(other))
    finally:
        for plan in plans:
            plan.close()
        capi.check(lib.axr_stream_destroy(stream))


def test_small_bundle_and_limits(pkg, orc, gpu):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(5)
    # a handful of tensors: the tables ride in the kernel arguments, no area involved
    few = make_bundle(gpu, rng, 6, strided_every=3)
    plan = pkg.BundlePlan.create(few, align=64)
    n = plan.payload_bytes
    buf = torch.full((n + 64,), POISON, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    for _ in range(2):               # also on a second launch of the same plan
        capi.check(lib.axr_pack_noalloc(plan._h, buf.data_ptr(), n, None))
        torch.cuda.synchronize()
        got = buf.cpu().numpy()
        assert np.array_equal(got[:n], orc.pack(host_chunks(few), 64)) and (got[n:] == POISON).all()
    # too small a payload buffer
    assert lib.axr_pack_noalloc(plan._h, buf.data_ptr(), n - 1, None) == capi.AXR_ERR_LENGTH
    plan.close()
    # tables beyond the static area: refused with a clear error, nothing launched
    arena = torch.zeros(100000 * 16, dtype=torch.uint8, device=gpu)
    views = [pkg.TensorView(data=arena.data_ptr() + 16 * i, device_type=10, device_id=0, dtype=(1, 8, 1),
                            shape=(16,), strides=None) for i in range(100000)]
    plan = pkg.BundlePlan.create(views, align=1)
    assert plan.launch_info()["table_bytes"] > (1 << 20)
    out = torch.full((plan.payload_bytes,), POISON, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    assert lib.axr_pack_noalloc(plan._h, out.data_ptr(), plan.payload_bytes, None) == capi.AXR_ERR_LENGTH
    assert b"static table area" in lib.axr_last_error()
    torch.cuda.synchronize()
    assert bool((out == POISON).all())
    plan.pack(out.data_ptr(), plan.payload_bytes)      # the allocating entry point still serves it
    torch.cuda.synchronize()
    assert bool((out == 0).all())
    plan.close()
    # host tensors need staging blocks: refused
    host = np.arange(64, dtype=np.uint8)
    plan = pkg.BundlePlan.create([host], align=1)
    assert lib.axr_pack_noalloc(plan._h, out.data_ptr(), 64, None) == capi.AXR_ERR_UNSUPPORTED
    plan.close()
