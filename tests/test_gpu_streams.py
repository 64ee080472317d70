"""Stream ordering between the tensor framework and the bundle kernels, on a GPU.

The pack and unpack kernels may run on a stream that does not synchronise with the stream
the tensors were produced on.  These tests put a long-running kernel in front of the
producer and never synchronise the host between producing the tensors and packing them: the
result is only right when the launch was ordered behind the producer's stream."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def delay(torch, milliseconds=30):
    """Keeps torch's current stream busy for about `milliseconds`."""
    sleep = getattr(torch.cuda, "_sleep", None)
    if sleep is not None:
        sleep(int(milliseconds * 2.0e6))      # cycles at roughly 2 GHz
        return
    a = torch.randn(4096, 4096, device="cuda")
    for _ in range(int(milliseconds * 4)):
        a = a @ a
        a = a / a.abs().max()


def make_stream(pkg):
    s = C.c_void_p()
    pkg._capi.check(pkg._capi.load().axr_stream_create(C.byref(s)))
    return s.value


def test_pack_waits_for_the_producers_without_a_host_synchronisation(pkg, orc, gpu):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(11)
    host = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in (100000, 33, 4096, 700001, 8, 250)]
    staged = [torch.from_numpy(h).pin_memory() for h in host]
    srcs = [torch.zeros(h.size, dtype=torch.uint8, device=gpu) for h in host]
    stream = make_stream(pkg)
    torch.cuda.synchronize()
    # the producers: a long kernel, then the copies that give the tensors their values
    delay(torch)
    for s, st in zip(srcs, staged):
        s.copy_(st, non_blocking=True)
    # packed at once on another (non-blocking) stream; nothing has waited on the host
    bundle = pkg.pack_bundle(srcs, align=256, stream=stream)
    capi.check(lib.axr_stream_synchronize(stream))
    got = torch.empty(bundle.payload_bytes, dtype=torch.uint8, device=gpu)
    capi.check(lib.axr_memcpy(capi.MEM_ROCM, got.data_ptr(), capi.MEM_ROCM, bundle.payload.data, bundle.payload_bytes))
    assert np.array_equal(got.cpu().numpy(), orc.pack(host, 256))
    # the same through a kept plan and BundlePlan.pack
    plan = pkg.BundlePlan.create(srcs, align=1)
    buf = torch.zeros(plan.payload_bytes, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    delay(torch)
    for s, st in zip(srcs, staged):
        s.copy_(st.flip(0), non_blocking=True)
    plan.pack(buf.data_ptr(), plan.payload_bytes, stream)
    capi.check(lib.axr_stream_synchronize(stream))
    assert np.array_equal(buf.cpu().numpy(), orc.pack([h[::-1] for h in host], 1))
    # without the ordering the kernel overtakes the producers (this is what the wait prevents)
    torch.cuda.synchronize()
    for s in srcs:
        s.zero_()
    torch.cuda.synchronize()
    delay(torch)
    for s, st in zip(srcs, staged):
        s.copy_(st, non_blocking=True)
    plan.pack(buf.data_ptr(), plan.payload_bytes, stream, order=False)
    capi.check(lib.axr_stream_synchronize(stream))
    early = buf.cpu().numpy()                 # (this copy waits for torch's stream, the pack did not)
    assert not early.any()
    plan.close()
    bundle.close()
    capi.check(lib.axr_stream_destroy(stream))


def test_unpack_is_ordered_both_ways(pkg, orc, gpu):
    """The scatter waits for the framework's writes to the destinations (zeroing them behind a
    long kernel), and the framework's next kernel waits for the scatter."""
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(12)
    host = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in (50000, 17, 300, 1 << 20)]
    srcs = [torch.from_numpy(h).to(gpu) for h in host]
    stream = make_stream(pkg)
    bundle = pkg.pack_bundle(srcs, align=256, stream=stream)
    capi.check(lib.axr_stream_synchronize(stream))
    outs = [torch.empty_like(s) for s in srcs]
    torch.cuda.synchronize()
    delay(torch)
    for o in outs:
        o.fill_(0xAB)                          # still queued behind the long kernel
    plan = pkg.unpack_bundle(bundle.header, bundle.payload, out=outs, stream=stream)
    sums = [o.to(torch.int64).sum() for o in outs]     # torch's stream: must see the scattered data
    torch.cuda.synchronize()
    assert [int(s) for s in sums] == [int(h.astype(np.int64).sum()) for h in host]
    for o, h in zip(outs, host):
        assert np.array_equal(o.cpu().numpy(), h)      # and the late fill did not overwrite it
    plan.close()
    bundle.close()
    capi.check(lib.axr_stream_destroy(stream))


class ForeignProducer:
    """A DLPack producer that is not a torch tensor: records the stream it is asked for and
    does its half of the handshake (here by delegating to the tensor it wraps)."""

    def __init__(self, tensor):
        self.tensor = tensor
        self.asked = []

    def __dlpack_device__(self):
        return self.tensor.__dlpack_device__()

    def __dlpack__(self, stream=None, **kwargs):
        self.asked.append(stream)
        # (1 names the legacy default stream in the protocol; this torch spells it None)
        return self.tensor.__dlpack__(stream=None if stream in (None, 1) else stream)


def test_foreign_producers_are_told_the_consumer_stream(pkg, orc, gpu):
    import torch
    lib, capi = pkg._capi.load(), pkg._capi
    rng = np.random.default_rng(13)
    host = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in (4096, 100, 70000)]
    staged = [torch.from_numpy(h).pin_memory() for h in host]
    tensors = [torch.zeros(h.size, dtype=torch.uint8, device=gpu) for h in host]
    producers = [ForeignProducer(t) for t in tensors]
    stream = make_stream(pkg)
    torch.cuda.synchronize()
    delay(torch)
    for t, st in zip(tensors, staged):
        t.copy_(st, non_blocking=True)
    bundle = pkg.pack_bundle(producers, align=64, stream=stream)
    capi.check(lib.axr_stream_synchronize(stream))
    # asked once each, with the consumer's stream handle (never 0 on a ROCm device)
    assert all(p.asked == [stream] for p in producers)
    got = torch.empty(bundle.payload_bytes, dtype=torch.uint8, device=gpu)
    capi.check(lib.axr_memcpy(capi.MEM_ROCM, got.data_ptr(), capi.MEM_ROCM, bundle.payload.data, bundle.payload_bytes))
    assert np.array_equal(got.cpu().numpy(), orc.pack(host, 64))
    # no stream named: asked the plain way, and the default stream is spelled 1 when it is named
    q = ForeignProducer(tensors[0])
    pkg.BundlePlan.create([q], align=1).close()
    assert q.asked == [None]
    q = ForeignProducer(tensors[0])
    pkg.BundlePlan.create([q], align=1, stream=0).close()
    assert q.asked == [1]
    bundle.close()
    capi.check(lib.axr_stream_destroy(stream))
