#!/usr/bin/env python3
"""Benchmark of the tensor-bundle pack+unpack path on one MI355X.

A step is one pack plus one unpack of the 4,096-tensor mixed bundle
(4096 1-D tensors of 256 B-64 KiB in five dtypes); inputs are resident in HBM before the timed region.
`value` = 4 * P / t  (P = sum of tensor bytes; pack reads P and writes P, unpack
reads P and writes P), in GB/s, timed with HIP events on the stream the kernels
are launched on.  The steps rotate over several independent copies of the bundle so
that the working set exceeds the 256 MB last-level cache, and they are software
pipelined the way a worker with traffic in both directions runs them: step i hands
the pack of bundle i+1 and the unpack of bundle i to axr_submit, which serves both
with ONE kernel launch on one stream (every bundle is still packed once and
unpacked once per step, and bundle i's unpack reads what the previous step's launch
packed).  The same steps as two separate launches (axr_pack, axr_unpack) are
reported next to it.  The K timed steps are repeated in batches until at least
50 ms have been timed and the median batch is reported.

Prints ONE JSON line.  Only one GPU is used: --gpus above 1 is refused.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--rotate", type=int, default=4,
                    help="independent bundle copies cycled through by the steps (1 = cache resident)")
    ap.add_argument("--workload", default="c2", choices=["c2", "c3", "c4", "c5", "small", "transposed", "rows100", "rows250", "rows512",
                             "stepped", "odd_transposed"])
    ap.add_argument("--align", type=int, default=256, help="pack alignment of the c2 and small workloads")
    ap.add_argument("--direction", default="both", choices=["both", "pack", "unpack"],
                    help="with --separate-launches: time only the packs or only the unpacks")
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--separate-launches", action="store_true",
                    help="time axr_pack + axr_unpack as two launches per step instead of one axr_submit")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--tune", default="", help="comma separated key=value kernel tunables")
    ap.add_argument("--ceilings", action="store_true",
                    help="print what the plain copy, fill and row kernels reach on this device and exit")
    ap.add_argument("--small-segments", action="store_true",
                    help="print the report of the many-short-tensors workload (65,536 tensors of 8-512 B) and exit")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="N",
                    help="also run N plain 256 MiB device copies (axr_copy_reference) so that "
                         "profiler counters can be scaled by a kernel of known traffic")
    return ap.parse_args()


class Harness:
    def __init__(self, pkg):
        import torch
        self.torch = torch
        self.pkg = pkg
        self.capi = pkg._capi
        self.lib = pkg._capi.load()
        s = C.c_void_p()
        self.capi.check(self.lib.axr_stream_create(C.byref(s)))
        self.stream = s.value
        self.ev0, self.ev1 = C.c_void_p(), C.c_void_p()
        self.capi.check(self.lib.axr_event_create(C.byref(self.ev0)))
        self.capi.check(self.lib.axr_event_create(C.byref(self.ev1)))

    def sync(self):
        self.capi.check(self.lib.axr_stream_synchronize(self.stream))
        self.torch.cuda.synchronize()

    MIN_TIMED_MS = 50.0
    MAX_BATCHES = 400

    def time_steps(self, step_fn, steps, warmup):
        """Runs step_fn(i) `warmup` times, then batches of `steps` calls, each batch
        between two HIP events on the launch stream, until MIN_TIMED_MS have been
        timed; returns the median batch in milliseconds (and leaves the batch count
        in self.batches)."""
        i = 0
        for _ in range(warmup):
            step_fn(i)
            i += 1
        self.sync()
        times, total = [], 0.0
        while total < self.MIN_TIMED_MS and len(times) < self.MAX_BATCHES:
            self.capi.check(self.lib.axr_event_record(self.ev0, self.stream))
            for _ in range(steps):
                step_fn(i)
                i += 1
            self.capi.check(self.lib.axr_event_record(self.ev1, self.stream))
            self.capi.check(self.lib.axr_event_synchronize(self.ev1))
            ms = C.c_float()
            self.capi.check(self.lib.axr_event_elapsed_ms(self.ev0, self.ev1, C.byref(ms)))
            times.append(float(ms.value))
            total += times[-1]
        self.sync()
        self.batches = len(times)
        times.sort()
        return times[len(times) // 2]


class BundleSet:
    """One independent copy of a workload: source views, payload, destination views, two plans.

    `check` compares source and destination on the device after a round trip."""

    def __init__(self, h: Harness, src_views, dst_views, align, keep, check=None, clear=None):
        pkg = h.pkg
        self.keep = keep
        self.check = check
        self.clear = clear
        self.pack_plan = pkg.BundlePlan.create(src_views, align=align)
        self.nbytes = self.pack_plan.payload_bytes
        self.data_bytes = self.pack_plan.data_bytes
        self.payload = h.torch.empty(max(self.nbytes, 1), dtype=h.torch.uint8, device="cuda")
        self.unpack_plan = pkg.BundlePlan.from_header(self.pack_plan.header).bind(dst_views)
        self.pp, self.up = self.pack_plan._h, self.unpack_plan._h
        self.ptr = self.payload.data_ptr()


def run_sets(h: Harness, sets, steps, warmup):
    lib, stream = h.lib, h.stream
    n = len(sets)
    calls = [(s.pp, s.up, s.ptr, s.nbytes) for s in sets]

    def step(i):
        pp, up, ptr, nb = calls[i % n]
        rc = lib.axr_pack(pp, ptr, nb, stream)
        rc |= lib.axr_unpack(up, ptr, nb, stream)
        if rc:
            h.capi.check(rc)

    ms = h.time_steps(step, steps, warmup)
    return ms


def run_sets_one_direction(h: Harness, sets, steps, warmup, unpack):
    """Only the packs (unpack == False) or only the unpacks of the rotating sets, one launch
    per step: what a sender and a receiver in different processes each see.  The payloads
    must hold packed data before the unpacks are timed."""
    lib, stream = h.lib, h.stream
    n = len(sets)
    calls = [(s.up if unpack else s.pp, s.ptr, s.nbytes) for s in sets]
    fn = lib.axr_unpack if unpack else lib.axr_pack

    def step(i):
        plan, ptr, nb = calls[i % n]
        rc = fn(plan, ptr, nb, stream)
        if rc:
            h.capi.check(rc)

    return h.time_steps(step, steps, warmup)


def half_rates(h: Harness, sets, steps, warmup):
    """Pack-only and unpack-only figures of a workload: GB/s over the 2P bytes one
    direction reads and writes, fraction of the HBM peak, microseconds per launch."""
    P = sets[0].data_bytes
    out = {}
    for name, unpack in (("pack_only", False), ("unpack_only", True)):
        ms = run_sets_one_direction(h, sets, steps, warmup, unpack)
        us = ms * 1e3 / steps
        gbps = 2.0 * P / (us * 1e-6) / 1e9
        out[name] = {"GBps_2P": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "avg_launch_us": round(us, 3)}
    return out


def run_sets_one_launch(h: Harness, sets, steps, warmup, width=1):
    """Step i = axr_submit({packs of the next `width` sets, unpacks of the `width` sets packed
    by the step before}): one kernel launch that moves `width` bundles each way."""
    lib, stream, capi = h.lib, h.stream, h.capi
    n = len(sets)
    if n < 2 * width or n % width:
        raise ValueError("the pipelined steps need two groups of bundle copies")
    groups = n // width
    jobs = []
    for g in range(groups):
        arr = (capi.Job * (2 * width))()
        for k in range(width):
            a, b = sets[((g + 1) % groups) * width + k], sets[g * width + k]
            arr[k] = capi.Job(a.pp, 0, a.ptr, a.nbytes, 0)
            arr[width + k] = capi.Job(b.up, 1, b.ptr, b.nbytes, 0)
        jobs.append(arr)
    for k in range(width):      # fills the pipeline
        capi.check(lib.axr_pack(sets[k].pp, sets[k].ptr, sets[k].nbytes, stream))

    def step(i):
        rc = lib.axr_submit(jobs[i % groups], 2 * width, stream)
        if rc:
            capi.check(rc)

    return h.time_steps(step, steps, warmup)


def run_sets_two_streams(h: Harness, sets, steps, warmup):
    """The same steps with the bundles alternating between two streams, so that one
    bundle's pack overlaps another's unpack (a sender with several bundles in flight).
    Host clock around a synchronisation of both streams; returns milliseconds."""
    lib, check = h.lib, h.capi.check
    second = C.c_void_p()
    check(lib.axr_stream_create(C.byref(second)))
    streams = (h.stream, second.value)
    n = len(sets)
    calls = [(s.pp, s.up, s.ptr, s.nbytes) for s in sets]

    def step(i):
        pp, up, ptr, nb = calls[i % n]
        stream = streams[i % 2]
        rc = lib.axr_pack(pp, ptr, nb, stream)
        rc |= lib.axr_unpack(up, ptr, nb, stream)
        if rc:
            check(rc)

    def drain():
        for stream in streams:
            check(lib.axr_stream_synchronize(stream))

    for i in range(warmup):
        step(i)
    drain()
    times, total = [], 0.0
    while total < h.MIN_TIMED_MS and len(times) < h.MAX_BATCHES:
        t0 = time.perf_counter()
        for i in range(steps):
            step(i)
        drain()
        times.append((time.perf_counter() - t0) * 1e3)
        total += times[-1]
    check(lib.axr_stream_destroy(second))
    times.sort()
    return times[len(times) // 2]


def run_sets_one_direction_two_streams(h: Harness, sets, steps, warmup, unpack):
    """Only the packs (or only the unpacks) of the rotating sets, alternating between two
    streams: a sender (or a receiver) with several independent bundles in flight, whose launches
    need no order among themselves.  Host clock around a synchronisation of both streams;
    returns milliseconds.  The payloads must hold packed data before the unpacks are timed."""
    lib, check = h.lib, h.capi.check
    second = C.c_void_p()
    check(lib.axr_stream_create(C.byref(second)))
    streams = (h.stream, second.value)
    n = len(sets)
    calls = [((s.up if unpack else s.pp), s.ptr, s.nbytes) for s in sets]
    fn = lib.axr_unpack if unpack else lib.axr_pack

    def step(i):
        plan, ptr, nb = calls[i % n]
        rc = fn(plan, ptr, nb, streams[i % 2])
        if rc:
            check(rc)

    def drain():
        for stream in streams:
            check(lib.axr_stream_synchronize(stream))

    for i in range(warmup):
        step(i)
    drain()
    times, total = [], 0.0
    while total < h.MIN_TIMED_MS and len(times) < h.MAX_BATCHES:
        t0 = time.perf_counter()
        for i in range(steps):
            step(i)
        drain()
        times.append((time.perf_counter() - t0) * 1e3)
        total += times[-1]
    check(lib.axr_stream_destroy(second))
    times.sort()
    return times[len(times) // 2]


def tensor_byte_mask(h, spec):
    """Boolean device tensor over the arena: True for bytes that belong to a tensor."""
    import numpy as np
    edges = np.zeros(spec.arena_bytes + 1, dtype=np.int32)
    starts = np.fromiter((s.arena_offset for s in spec.segments), dtype=np.int64, count=len(spec.segments))
    sizes = np.fromiter((s.nbytes for s in spec.segments), dtype=np.int64, count=len(spec.segments))
    np.add.at(edges, starts, 1)
    np.add.at(edges, starts + sizes, -1)
    return h.torch.from_numpy(np.cumsum(edges[:-1]) > 0).cuda()


def make_c2_sets(h, count, seed=0, align=256, spec=None):
    from execution_ucx_amd import workloads
    if spec is None:
        spec = workloads.mixed_bundle(seed=seed)
    sets = []
    mask = tensor_byte_mask(h, spec)
    for k in range(count):
        arena, _ = workloads.materialize_mixed(spec, "cuda", seed=seed + k)
        arena.mul_(mask)      # bytes between tensors are not part of the bundle: zero them
        dst = h.torch.zeros_like(arena)
        sv = workloads.mixed_views(spec, arena.data_ptr())
        dv = workloads.mixed_views(spec, dst.data_ptr())
        sets.append(BundleSet(h, sv, dv, align, (arena, dst),
                              check=lambda a=arena, d=dst: bool(h.torch.equal(a, d)),
                              clear=lambda d=dst: d.zero_()))
    return spec, sets


def make_c3_sets(h, count, seed=0):
    from execution_ucx_amd import workloads
    sets = []
    for k in range(count):
        src = workloads.materialize_llama_layer("cuda", seed=seed + k)
        dst = [h.torch.empty_like(t) for t in src]
        sets.append(BundleSet(
            h, workloads.views_of_torch(src), workloads.views_of_torch(dst), 256, (src, dst),
            check=lambda s=src, d=dst: all(bool(h.torch.equal(x.view(h.torch.int16), y.view(h.torch.int16)))
                                           for x, y in zip(s, d))))
    return sets


def make_c4_set(h, seed=0):
    from execution_ucx_amd import workloads
    spec = workloads.kv_gather(seed=seed)
    a = h.torch.empty(spec.cache_shape, dtype=h.torch.bfloat16, device="cuda")
    a.view(h.torch.int16).random_(-32768, 32767)
    b = h.torch.zeros(spec.cache_shape, dtype=h.torch.bfloat16, device="cuda")
    sv = [workloads.kv_block_view(a.data_ptr(), spec, int(i)) for i in spec.src_index]
    dv = [workloads.kv_block_view(b.data_ptr(), spec, int(i)) for i in spec.dst_index]
    si = h.torch.from_numpy(spec.src_index).cuda()
    di = h.torch.from_numpy(spec.dst_index).cuda()

    def check():
        ai, bi = a.view(h.torch.int16), b.view(h.torch.int16)
        return bool(h.torch.equal(bi[:, :, di], ai[:, :, si]))
    return BundleSet(h, sv, dv, 256, (a, b), check=check)


def make_c5_sets(h, count):
    from execution_ucx_amd import workloads
    spec = workloads.pitched_chunk()
    sets = []
    for _ in range(count):
        src = h.torch.empty(spec.views, spec.rows, spec.pitch, dtype=h.torch.bfloat16, device="cuda")
        src.view(h.torch.int16).random_(-32768, 32767)
        dst = h.torch.zeros_like(src)
        sets.append(BundleSet(
            h, workloads.pitched_views(src.data_ptr(), spec),
            workloads.pitched_views(dst.data_ptr(), spec), 256, (src, dst),
            check=lambda s=src, d=dst, c=spec.cols: bool(h.torch.equal(
                s.view(h.torch.int16)[:, :, :c], d.view(h.torch.int16)[:, :, :c]))))
    return sets


def make_transposed_sets(h, count, seed=0, n=8, edge=4096):
    """n transposed [edge, edge] bf16 matrices per bundle (x.t() views), scattered
    back through the same transposition."""
    import torch
    from execution_ucx_amd import workloads
    sets = []
    for k in range(count):
        g = torch.Generator(device="cuda")
        g.manual_seed(seed + k)
        src = [torch.randint(-2 ** 15, 2 ** 15, (edge, edge), device="cuda", generator=g,
                             dtype=torch.int16).view(torch.bfloat16) for _ in range(n)]
        dst = [torch.zeros_like(x) for x in src]
        sets.append(BundleSet(
            h, workloads.views_of_torch([x.t() for x in src]),
            workloads.views_of_torch([y.t() for y in dst]), 256, (src, dst),
            check=lambda src=src, dst=dst: all(bool(torch.equal(x.view(torch.int16), y.view(torch.int16)))
                                               for x, y in zip(src, dst))))
    return sets


def _random_storage(torch, shape, dtype, seed):
    """Random bytes viewed as `dtype` (every bit pattern occurs, NaNs included: the path moves bytes)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    item = torch.empty((), dtype=dtype).element_size()
    n = 1
    for e in shape:
        n *= e
    return torch.randint(0, 256, (n * item,), dtype=torch.uint8, device="cuda", generator=g).view(dtype).reshape(shape)


# Strided views: name -> (description, function(torch, seed) -> list of views of fresh storage)
VIEW_WORKLOADS = {
    "rows100": ("fp32 [2M, 64][:, :25]: rows of 100 B at a 256 B pitch (element mode, ragged 16-byte granules)",
                lambda t, seed: [_random_storage(t, (1 << 21, 64), t.float32, seed)[:, :25]]),
    "rows250": ("bf16 [1M, 512][:, :125]: rows of 250 B at a 1 KiB pitch (element mode, ragged 16-byte granules)",
                lambda t, seed: [_random_storage(t, (1 << 20, 512), t.bfloat16, seed)[:, :125]]),
    "rows512": ("bf16 [512K, 512][:, :256]: rows of 512 B at a 1 KiB pitch (element mode, 16-byte granules)",
                lambda t, seed: [_random_storage(t, (1 << 19, 512), t.bfloat16, seed)[:, :256]]),
    "stepped": ("fp32 [16M, 8][:, ::2]: every second element (element mode, 4-byte granules)",
                lambda t, seed: [_random_storage(t, (1 << 24, 8), t.float32, seed)[:, ::2]]),
    "odd_transposed": ("4 transposed 4097 x 4099 bf16 matrices (x.t() views; rows straddle 128-byte lines)",
                       lambda t, seed: [_random_storage(t, (4097, 4099), t.bfloat16, seed + k).t() for k in range(4)]),
}


def make_view_sets(h, count, workload, seed=0):
    """Bundles of strided torch views, scattered back into views of the same geometry over
    zeroed storage; the check compares the elements the views address."""
    import torch
    from execution_ucx_amd import workloads
    make = VIEW_WORKLOADS[workload][1]
    sets = []
    for k in range(count):
        src = make(torch, seed + 100 * k)
        twins = [torch.zeros_like(v._base if v._base is not None else v) for v in src]
        dst = [tw.as_strided(v.shape, v.stride(), v.storage_offset()) for tw, v in zip(twins, src)]

        def check(src=src, dst=dst):
            return all(bool(torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8)))
                       for a, b in zip(src, dst))
        sets.append(BundleSet(h, workloads.views_of_torch(src), workloads.views_of_torch(dst), 256,
                              (src, twins, dst), check=check))
    return sets


def verify_set(h, s):
    """One pack + unpack, then destination == source on the device."""
    h.sync()      # inputs were produced on torch's stream, the bundle kernels run on ours
    h.capi.check(h.lib.axr_pack(s.pp, s.ptr, s.nbytes, h.stream))
    h.capi.check(h.lib.axr_unpack(s.up, s.ptr, s.nbytes, h.stream))
    h.sync()
    if s.check is not None and not s.check():
        raise SystemExit("bench.py: round trip did not reproduce the source tensors")


def check_sets(h, sets, what):
    h.sync()
    for s in sets:
        if s.check is not None and not s.check():
            raise SystemExit(f"bench.py: {what} did not reproduce the source tensors")


def clear_sets(h, sets):
    for s in sets:
        if s.clear is not None:
            s.clear()
    h.sync()


def rate(data_bytes, ms, steps):
    """GB/s of read+write traffic for `steps` pack+unpack round trips."""
    return 4.0 * data_bytes * steps / (ms * 1e-3) / 1e9


def end_to_end_us(h, spec, steps=20):
    """Wall time of plan -> pack -> sync -> plan from header and destination tensors
    (axr_plan_from_header_bind) -> unpack -> sync for a fresh 4,096-tensor bundle, C ABI only
    (tensor descriptors prebuilt)."""
    from execution_ucx_amd import workloads
    from execution_ucx_amd.dlpack import TensorArray
    lib, capi = h.lib, h.capi
    arena, _ = workloads.materialize_mixed(spec, "cuda", seed=99)
    dst = h.torch.zeros_like(arena)
    mask = h.torch.zeros(spec.arena_bytes, dtype=h.torch.bool, device="cuda")
    for s in spec.segments:
        mask[s.arena_offset:s.arena_offset + s.nbytes] = True
    sa = TensorArray(workloads.mixed_views(spec, arena.data_ptr()))
    da = TensorArray(workloads.mixed_views(spec, dst.data_ptr()))
    probe = h.pkg.BundlePlan.create(sa.views, align=256)
    nbytes = probe.payload_bytes
    probe.close()
    payload = h.torch.empty(nbytes, dtype=h.torch.uint8, device="cuda")
    times, plan_times = [], []
    for it in range(steps + 3):
        h.sync()
        t0 = time.perf_counter()
        p = C.c_void_p()
        capi.check(lib.axr_plan_create(sa.pointer(), sa.count, 256, 0, C.byref(p)))
        hp, hn = C.c_void_p(), C.c_size_t()
        capi.check(lib.axr_plan_header(p, C.byref(hp), C.byref(hn)))
        t1 = time.perf_counter()
        capi.check(lib.axr_pack(p, payload.data_ptr(), nbytes, h.stream))
        capi.check(lib.axr_stream_synchronize(h.stream))
        r = C.c_void_p()
        capi.check(lib.axr_plan_from_header_bind(hp, hn.value, da.pointer(), da.count, C.byref(r)))
        capi.check(lib.axr_unpack(r, payload.data_ptr(), nbytes, h.stream))
        capi.check(lib.axr_stream_synchronize(h.stream))
        t2 = time.perf_counter()
        capi.check(lib.axr_plan_free(p))
        capi.check(lib.axr_plan_free(r))
        if it >= 3:
            times.append(t2 - t0)
            plan_times.append(t1 - t0)
    # the bytes between the tensors are not part of the bundle and stay zero
    if not (bool(h.torch.equal(arena[mask], dst[mask])) and bool((dst[~mask] == 0).all())):
        raise SystemExit("bench.py: fresh-bundle round trip did not reproduce the tensors")
    times.sort()
    plan_times.sort()
    n_k = len(spec.segments) / 1000.0
    return {"us_per_1k_tensors": times[len(times) // 2] * 1e6 / n_k,
            "plan_us_per_1k_tensors": plan_times[len(plan_times) // 2] * 1e6 / n_k,
            "round_trip_us": times[len(times) // 2] * 1e6}


def end_to_end_from_cpp():
    """The same fresh-bundle round trip timed inside a C++ caller of the C ABI
    (execution-ucx_amd/lib/fresh_bundle_bench, built by `make`): no ctypes calls in the timed
    region.  It checks its own result and prints one JSON line."""
    import subprocess
    exe = os.path.join(ROOT, "execution-ucx_amd", "lib", "fresh_bundle_bench")
    if not os.path.exists(exe):
        return "not measured: lib/fresh_bundle_bench is not built"
    out = subprocess.run([exe, "100"], capture_output=True, text=True, timeout=120)
    if out.returncode != 0:
        raise SystemExit("bench.py: fresh_bundle_bench failed: " + out.stderr.strip()[-400:])
    return json.loads(out.stdout.strip().splitlines()[-1])


def fresh_small_round_trip(h, tensors=4, each=64 * 1024, steps=200):
    """Wall time of plan -> pack -> sync -> plan-from-header -> bind -> unpack -> sync for a
    fresh bundle of a few tensors (the size of a typical RPC argument list), C ABI only."""
    from execution_ucx_amd.dlpack import TensorArray
    lib, capi, torch = h.lib, h.capi, h.torch
    src = [torch.randint(0, 255, (each,), dtype=torch.uint8, device="cuda") for _ in range(tensors)]
    dst = [torch.zeros_like(t) for t in src]
    sa, da = TensorArray.from_objects(src), TensorArray.from_objects(dst)
    probe = h.pkg.BundlePlan.create(src, align=256)
    nbytes, inline = probe.payload_bytes, probe.launch_info()["inline_tables"]
    probe.close()
    payload = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    times = []
    for it in range(steps + 5):
        h.sync()
        t0 = time.perf_counter()
        p = C.c_void_p()
        capi.check(lib.axr_plan_create(sa.pointer(), sa.count, 256, 0, C.byref(p)))
        hp, hn = C.c_void_p(), C.c_size_t()
        capi.check(lib.axr_plan_header(p, C.byref(hp), C.byref(hn)))
        capi.check(lib.axr_pack(p, payload.data_ptr(), nbytes, h.stream))
        capi.check(lib.axr_stream_synchronize(h.stream))
        r = C.c_void_p()
        capi.check(lib.axr_plan_from_header(hp, hn.value, C.byref(r)))
        capi.check(lib.axr_plan_bind(r, da.pointer(), da.count))
        capi.check(lib.axr_unpack(r, payload.data_ptr(), nbytes, h.stream))
        capi.check(lib.axr_stream_synchronize(h.stream))
        t1 = time.perf_counter()
        capi.check(lib.axr_plan_free(p))
        capi.check(lib.axr_plan_free(r))
        if it >= 5:
            times.append(t1 - t0)
    assert all(torch.equal(a, b) for a, b in zip(src, dst))
    times.sort()
    return {"tensors": tensors, "bytes_each": each, "round_trip_us": round(times[len(times) // 2] * 1e6, 2),
            "tables_in_kernel_arguments": bool(inline)}


def stream_c5(h, chunks=32):
    """8 GiB as 32 chunks of 64 pitched views through the transfer object (axr_transfer_*):
    one sender plan and one receiver plan, moved over the chunks by their address deltas;
    only C ABI calls in the timed loop.  Three arrangements (one slot: the host waits for
    every chunk; two slots on two streams; two slots on one stream), each with the receiver
    borrowing the sender's slot and with a wire copy into a receive slot."""
    from execution_ucx_amd import workloads
    torch, lib, capi = h.torch, h.lib, h.capi
    spec = workloads.pitched_chunk()
    src = torch.empty(chunks, spec.views, spec.rows, spec.pitch, dtype=torch.bfloat16, device="cuda")
    src.view(torch.int16).random_(-32768, 32767)
    dst = torch.zeros_like(src)
    per_chunk = spec.views * spec.parent_elems * 2
    send = h.pkg.BundlePlan.create(workloads.pitched_views(src.data_ptr(), spec), align=256)
    recv = h.pkg.BundlePlan.from_header(send.header).bind(workloads.pitched_views(dst.data_ptr(), spec))
    out = {}
    for name, lanes, streams, zero_copy in (("one_lane", 1, 1, 1), ("two_streams", 2, 2, 1), ("one_stream_two_lanes", 2, 1, 1),
                                            ("copy_one_lane", 1, 1, 0), ("copy_two_streams", 2, 2, 0),
                                            ("copy_one_stream_two_lanes", 2, 1, 0)):
        t = C.c_void_p()
        capi.check(lib.axr_transfer_create(None, spec.payload_bytes, lanes, streams, C.byref(t)))
        capi.check(lib.axr_transfer_set_zero_copy(t, zero_copy))
        for k in range(2):              # warm the slots and the plans' tables
            capi.check(lib.axr_transfer_submit(t, send._h, k * per_chunk, recv._h, k * per_chunk))
        capi.check(lib.axr_transfer_finish(t))
        dst.zero_()
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            for k in range(chunks):
                rc = lib.axr_transfer_submit(t, send._h, k * per_chunk, recv._h, k * per_chunk)
                if rc:
                    capi.check(rc)
            capi.check(lib.axr_transfer_finish(t))
            times.append(time.perf_counter() - t0)
        capi.check(lib.axr_transfer_destroy(t))
        out[name] = sorted(times)[len(times) // 2]
    ok = bool(torch.equal(src.view(torch.int16)[..., :spec.cols], dst.view(torch.int16)[..., :spec.cols]))
    send.close()
    recv.close()
    if not ok:
        raise SystemExit("bench.py: streamed pipeline did not reproduce the source views")
    P = chunks * spec.payload_bytes
    best = min(out["two_streams"], out["one_stream_two_lanes"])
    best_copy = min(out["copy_two_streams"], out["copy_one_stream_two_lanes"])
    return {"payload_bytes_P": P, "chunks": chunks,
            "wire": "the receiver borrows the sender's slot (zero-copy rendezvous on one device): 4P bytes per chunk",
            "GBps_pack_unpack_4P": round(4.0 * P / best / 1e9, 1),
            "arrangement": ("two slots on one stream" if best == out["one_stream_two_lanes"]
                            else "two slots on two streams"),
            "two_streams": {"seconds": round(out["two_streams"], 5),
                            "GBps_4P": round(4.0 * P / out["two_streams"] / 1e9, 1),
                            "overlap_speedup": round(out["one_lane"] / out["two_streams"], 3)},
            "one_stream_two_lanes": {"seconds": round(out["one_stream_two_lanes"], 5),
                                     "GBps_4P": round(4.0 * P / out["one_stream_two_lanes"] / 1e9, 1),
                                     "overlap_speedup": round(out["one_lane"] / out["one_stream_two_lanes"], 3)},
            "seconds_one_lane": round(out["one_lane"], 5),
            "with_wire_copy": {
                "wire": "every chunk copied from the send slot to a receive slot: 6P bytes per chunk",
                "GBps_pack_unpack_4P": round(4.0 * P / best_copy / 1e9, 1),
                "GBps_with_wire_copy_6P": round(6.0 * P / best_copy / 1e9, 1),
                "seconds_two_streams": round(out["copy_two_streams"], 5),
                "seconds_one_stream_two_lanes": round(out["copy_one_stream_two_lanes"], 5),
                "seconds_one_lane": round(out["copy_one_lane"], 5)}}


def host_bundle_c1(h, reps=30):
    """64 fp32 host tensors (4 MiB) -> device payload -> host tensors: every byte
    crosses PCIe twice, so this is a transfer figure, not an HBM one."""
    import numpy as np
    from execution_ucx_amd import workloads
    srcs = workloads.host_bundle_c1(seed=0)
    outs = [np.zeros_like(s) for s in srcs]
    plan = h.pkg.BundlePlan.create(srcs, align=1)
    nbytes = plan.payload_bytes
    payload = h.torch.empty(nbytes, dtype=h.torch.uint8, device="cuda")
    rplan = h.pkg.BundlePlan.from_header(plan.header).bind(outs)
    times = []
    for _ in range(reps + 3):
        h.sync()
        t0 = time.perf_counter()
        plan.pack(payload.data_ptr(), nbytes, h.stream)
        rplan.unpack(payload.data_ptr(), nbytes, h.stream)
        h.capi.check(h.lib.axr_stream_synchronize(h.stream))
        times.append(time.perf_counter() - t0)
    if any(a.tobytes() != b.tobytes() for a, b in zip(srcs, outs)):
        raise SystemExit("bench.py: host bundle round trip differs")
    t = sorted(times[3:])[reps // 2]
    return {"payload_bytes_P": nbytes, "round_trip_us": round(t * 1e6, 1),
            "GBps_pcie_inclusive_4P": round(4.0 * nbytes / t / 1e9, 2)}


def iov_against_bundle(h, spec, reps=7):
    """The C2 tensors from sender memory to receiver memory on one device, two ways
    through the loopback context: the reference's way (one iov entry per tensor on
    both sides, ucx_connection.cpp:401-426: the transport copies entry by entry)
    and as a packed bundle (pack, ONE contiguous payload, unpack).  Microseconds
    per transfer, descriptors prepared beforehand."""
    from execution_ucx_amd import workloads
    from execution_ucx_amd.loopback import LoopbackAmContext
    torch = h.torch
    arena, _ = workloads.materialize_mixed(spec, "cuda", seed=17)
    dst = torch.zeros_like(arena)
    src_iov = [(arena.data_ptr() + s.arena_offset, s.nbytes) for s in spec.segments]
    dst_iov = [(dst.data_ptr() + s.arena_offset, s.nbytes) for s in spec.segments]
    client, server = LoopbackAmContext("client"), LoopbackAmContext("server")
    conn = client.connect(server)
    t_iov, t_bundle = [], []
    capi, lib = h.capi, h.lib
    nseg = len(src_iov)
    svec, dvec = (capi.Buffer * nseg)(), (capi.Buffer * nseg)()
    for i in range(nseg):
        svec[i] = capi.Buffer(src_iov[i][0], src_iov[i][1])
        dvec[i] = capi.Buffer(dst_iov[i][0], dst_iov[i][1])
    hdr = C.create_string_buffer(b"iov", 3)
    d = capi.AmIovec()
    d.header = capi.Buffer(C.addressof(hdr), 3)
    d.buffer_vec = C.cast(svec, C.POINTER(capi.Buffer))
    d.buffer_count = nseg
    d.buffer_type = capi.MEM_ROCM
    for _ in range(reps):
        h.sync()
        t0 = time.perf_counter()
        req, m = C.c_uint64(), capi.AmMessage()
        capi.check(lib.axr_am_send_iov(client._h, conn, C.byref(d), h.stream, C.byref(req)))
        capi.check(lib.axr_am_recv_header(server._h, C.byref(m)))
        capi.check(lib.axr_am_recv_buffer_iov(server._h, m.key, capi.MEM_ROCM, dvec, nseg, h.stream))
        h.sync()
        t_iov.append(time.perf_counter() - t0)
        done = C.c_int()
        capi.check(lib.axr_am_request_test(client._h, req.value, C.byref(done)))
    mask = torch.zeros(spec.arena_bytes, dtype=torch.bool, device="cuda")
    for s in spec.segments:
        mask[s.arena_offset:s.arena_offset + s.nbytes] = True
    ok_iov = bool(torch.equal(arena[mask], dst[mask])) and bool((dst[~mask] == 0).all())
    dst.zero_()
    from execution_ucx_amd.dlpack import TensorArray
    plan = h.pkg.BundlePlan.create(TensorArray(workloads.mixed_views(spec, arena.data_ptr())), align=256)
    rplan = h.pkg.BundlePlan.from_header(plan.header).bind(
        TensorArray(workloads.mixed_views(spec, dst.data_ptr())))
    n = plan.payload_bytes
    sendbuf = torch.empty(n, dtype=torch.uint8, device="cuda")
    recvbuf = torch.empty(n, dtype=torch.uint8, device="cuda")
    for _ in range(reps):
        h.sync()
        t0 = time.perf_counter()
        plan.pack(sendbuf.data_ptr(), n, h.stream)
        h.sync()                                  # the transport reads a finished buffer
        req = client.send(conn, plan.header, sendbuf.data_ptr(), n, stream=h.stream)
        msg = server.recv_header()
        server.recv_into(msg, recvbuf.data_ptr(), n, stream=h.stream, wait=False)
        rplan.unpack(recvbuf.data_ptr(), n, h.stream)
        h.sync()
        t_bundle.append(time.perf_counter() - t0)
        client.test(req)
    ok_bundle = bool(torch.equal(arena[mask], dst[mask])) and bool((dst[~mask] == 0).all())
    if not (ok_iov and ok_bundle):
        raise SystemExit("bench.py: loopback transfer differs")
    client.close()
    server.close()
    a, b = sorted(t_iov)[reps // 2] * 1e6, sorted(t_bundle)[reps // 2] * 1e6
    return {"tensors": len(spec.segments), "payload_bytes_P": plan.data_bytes,
            "iov_per_tensor_copies_us": round(a, 1), "packed_bundle_us": round(b, 1),
            "speedup": round(a / b, 1)}


def python_boundary(h, spec, reps=5):
    """Planning a 4096-tensor bundle from torch tensors through the Python layer
    (one DLPack export per tensor from C, descriptors read in C): us per 1k tensors."""
    from execution_ucx_amd import workloads
    arena, tensors = workloads.materialize_mixed(spec, "cuda", seed=5)
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        plan = h.pkg.BundlePlan.create(tensors, align=256)
        times.append(time.perf_counter() - t0)
        plan.close()
    return round(sorted(times)[reps // 2] * 1e6 / (len(tensors) / 1000.0), 1)


def checkpoint_staging(h, tensors=4096, each=64 * 1024, reps=5):
    """A packed device bundle to per-tensor host buffers (pageable, already
    touched): the staged path (8 MiB pinned blocks, one device copy each, pieces
    cut out on the host) against one pageable device-to-host copy per tensor, which
    is how the reference's checkpoint writer fetches a payload
    (axon/src/storage/avro_serialization.cpp:478-523).  C ABI calls only in the
    timed regions."""
    import numpy as np
    from execution_ucx_amd.dlpack import TensorArray, TensorView
    torch = h.torch
    src = torch.randint(0, 256, (tensors, each), dtype=torch.uint8, device="cuda")
    bundle = h.pkg.pack_bundle([src[i] for i in range(tensors)], align=256)
    torch.cuda.synchronize()
    nbytes = tensors * each
    outs = [np.zeros(each, dtype=np.uint8) for _ in range(tensors)]
    for o in outs:
        o.fill(1)
    views = TensorArray([TensorView(data=o.ctypes.data, device_type=h.capi.kDLCPU, device_id=0,
                                    dtype=(1, 8, 1), shape=(each,), strides=None) for o in outs])
    rplan = h.pkg.BundlePlan.from_header(bundle.header).bind(views)
    staged, naive = [], []
    host = src.cpu().numpy()
    for _ in range(reps):
        h.sync()
        t0 = time.perf_counter()
        rplan.unpack(bundle.payload.data, bundle.payload_bytes, h.stream)
        staged.append(time.perf_counter() - t0)
        if any(not np.array_equal(o, host[i]) for i, o in enumerate(outs)):
            raise SystemExit("bench.py: staged host copy differs")
        for o in outs:
            o.fill(1)
        t0 = time.perf_counter()
        for i, o in enumerate(outs):
            h.lib.axr_memcpy(h.capi.MEM_HOST, o.ctypes.data, h.capi.MEM_ROCM,
                             bundle.payload.data + i * each, each)
        naive.append(time.perf_counter() - t0)
        if any(not np.array_equal(o, host[i]) for i, o in enumerate(outs)):
            raise SystemExit("bench.py: per-tensor host copy differs")
    rplan.close()
    bundle.plan.close()
    bundle.payload.release()
    return {"tensors": tensors, "payload_bytes_P": nbytes,
            "staged_GBps": round(nbytes / sorted(staged)[reps // 2] / 1e9, 2),
            "copy_per_tensor_GBps": round(nbytes / sorted(naive)[reps // 2] / 1e9, 2)}


def cpu_baseline(spec, seed=0):
    """Reference host path on this box's cores: memcpy concat + split of the same bundle."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(seed)
    chunks = [rng.integers(0, 256, size=s.nbytes, dtype=np.uint8) for s in spec.segments]
    one = oracle.time_pack_unpack(chunks, align=1, threads=1, warmup=3, reps=30)
    cores = os.cpu_count() or 1
    cores = min(cores, 16)   # the GPU box grants 16 CPUs per GPU
    many = oracle.time_pack_unpack(chunks, align=1, threads=cores, warmup=3, reps=30,
                                   use_reference=False)
    P = one["data_bytes"]
    base = {"value": round(4.0 * P / one["seconds"] / 1e9, 3), "unit": "GB/s", "cores": 1,
            "kind": one["kind"],
            "sample": "same 4096-tensor bundle in pageable host memory, tight layout, "
                      "3 warm-ups + median of 30 pack+unpack repetitions"}
    allc = {"value": round(4.0 * P / many["seconds"] / 1e9, 3), "unit": "GB/s", "cores": cores,
            "kind": "port", "sample": "same bundle, tensor list cut into byte-balanced ranges, "
                                      "one thread per range, median of 30"}
    return base, allc


def cpu_baseline_other_configs():
    """The same reference host path on the host-memory bundle (64 x 64 KiB fp32) and on the
    Llama-7B layer bundle (0.4 GB), one thread, tight layout."""
    import numpy as np
    import oracle
    from execution_ucx_amd import workloads
    out = {}
    c1 = [a.view(np.uint8) for a in workloads.host_bundle_c1(seed=0)]
    r = oracle.time_pack_unpack(c1, align=1, threads=1, warmup=3, reps=200)
    out["cpu_baseline_c1"] = {"value": round(4.0 * r["data_bytes"] / r["seconds"] / 1e9, 3), "unit": "GB/s",
                              "cores": 1, "kind": r["kind"],
                              "sample": "64 fp32 tensors of 64 KiB (4 MiB), median of 200 pack+unpack repetitions"}
    rng = np.random.default_rng(0)
    c3 = [rng.integers(0, 256, size=int(np.prod(shape)) * 2, dtype=np.uint8)
          for _, shape in workloads.LLAMA7B_LAYER]
    r = oracle.time_pack_unpack(c3, align=1, threads=1, warmup=1, reps=7)
    out["cpu_baseline_c3"] = {"value": round(4.0 * r["data_bytes"] / r["seconds"] / 1e9, 3), "unit": "GB/s",
                              "cores": 1, "kind": r["kind"],
                              "sample": "the 9 bf16 tensors of one Llama-7B layer (404,766,720 B), "
                                        "median of 7 pack+unpack repetitions"}
    return out


def tune_get(pkg, key):
    v = C.c_int64()
    pkg._capi.check(pkg._capi.load().axr_tune_get(key.encode(), C.byref(v)))
    return v.value


def graph_replay(h, sets, P, steps_in_graph=20):
    """The pipelined steps recorded once into a HIP graph and replayed: GB/s, or a
    string saying why it could not be measured."""
    torch = h.torch
    lib, capi = h.lib, h.capi
    n = len(sets)
    try:
        for s in sets:
            capi.check(lib.axr_plan_prepare(s.pp, h.stream))
            capi.check(lib.axr_plan_prepare(s.up, h.stream))
        h.sync()
        side = torch.cuda.Stream()
        jobs = []
        for i in range(n):
            a, b = sets[(i + 1) % n], sets[i]
            arr = (capi.Job * 2)()
            arr[0] = capi.Job(a.pp, 0, a.ptr, a.nbytes, 0)
            arr[1] = capi.Job(b.up, 1, b.ptr, b.nbytes, 0)
            jobs.append(arr)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(steps_in_graph):
                capi.check(lib.axr_submit(jobs[i % n], 2, side.cuda_stream))
        clear_sets(h, sets)
        capi.check(lib.axr_pack(sets[0].pp, sets[0].ptr, sets[0].nbytes, h.stream))
        h.sync()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        times = []
        with torch.cuda.stream(side):
            for _ in range(3):
                graph.replay()
            side.synchronize()
            total = 0.0
            while total < h.MIN_TIMED_MS and len(times) < h.MAX_BATCHES:
                e0.record(side)
                graph.replay()
                e1.record(side)
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
                total += times[-1]
        check_sets(h, sets, "the graph replay")
        del graph
        times.sort()
        return round(rate(P, times[len(times) // 2], steps_in_graph), 1)
    except Exception as e:   # reported, never fatal for the benchmark line
        return f"not measured: {type(e).__name__}: {e}"


def ceilings(h):
    """What plain kernels of the library reach on this device: the copy kernel, the fill kernel
    and the row gather / scatter kernel (no tables, one 16-byte access per lane) on the row
    geometries of the strided workloads.  GB/s of bytes read plus bytes written."""
    torch, lib, check = h.torch, h.lib, h.capi.check
    out = {"copy_kernel": {}, "fill_kernel": {}, "row_kernel": {}}
    for label, n in (("48 MB", 47869056), ("405 MB", 404766720), ("1 GiB", 1 << 30)):
        copies = max(2, int((600 << 20) // (2 * n)) + 1)    # rotating buffers: more than the last-level cache holds
        a = [torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda") for _ in range(copies)]
        b = [torch.empty_like(x) for x in a]
        h.sync()
        k = max(10, int(4e9 // n))
        ms = h.time_steps(lambda i: check(lib.axr_copy_reference(b[i % copies].data_ptr(), a[i % copies].data_ptr(),
                                                                 n, h.stream)), k, 3)
        out["copy_kernel"][label] = {"GBps": round(2.0 * n * k / (ms * 1e-3) / 1e9, 1), "us_per_launch": round(ms * 1e3 / k, 2),
                                     "rotating_buffer_pairs": copies}
        ms = h.time_steps(lambda i: check(lib.axr_memset_async(b[i % copies].data_ptr(), 7, n, h.stream)), k, 3)
        out["fill_kernel"][label] = {"GBps": round(1.0 * n * k / (ms * 1e-3) / 1e9, 1)}
        # the same copy in the shapes of the bundle kernels' wavefronts (threads per workgroup,
        # KiB per wavefront, streaming hint): what a shape allows with no table in front of it
        whole = n // 4096 * 4096
        shaped = {}
        for threads, kib, nt in ((64, 1, 1), (64, 1, 0), (256, 1, 1), (128, 2, 1), (256, 2, 1), (256, 2, 0), (256, 4, 1)):
            ms = h.time_steps(lambda i: check(lib.axr_copy_reference_shaped(
                b[i % copies].data_ptr(), a[i % copies].data_ptr(), whole, threads, kib, nt, h.stream)), k, 3)
            shaped[f"{threads} threads, {kib} KiB per wavefront, {'streaming' if nt else 'cacheable'}"] = {
                "GBps": round(2.0 * whole * k / (ms * 1e-3) / 1e9, 1), "us_per_launch": round(ms * 1e3 / k, 2)}
        if not bool(torch.equal(a[0][:whole], b[0][:whole])):
            raise SystemExit("bench.py: the shaped copy kernel did not copy")
        out.setdefault("copy_kernel_shaped", {})[label] = shaped
        del a, b
        torch.cuda.empty_cache()
    for label, run, pitch, rows in (("100 B rows at a 256 B pitch", 100, 256, 1 << 21),
                                    ("250 B rows at a 1 KiB pitch", 250, 1024, 1 << 20),
                                    ("512 B rows at a 1 KiB pitch", 512, 1024, 1 << 19),
                                    ("128 B rows at a 256 B pitch", 128, 256, 1 << 21)):
        strided = [torch.randint(0, 256, (rows * pitch,), dtype=torch.uint8, device="cuda") for _ in range(2)]
        packed = [torch.empty(rows * run, dtype=torch.uint8, device="cuda") for _ in range(2)]
        h.sync()
        k = 20
        res = {}
        for scatter, name in ((0, "gather"), (1, "scatter")):
            best, every = None, {}
            for nt in (0, 1, 2, 3):
                def step(i, scatter=scatter, nt=nt):
                    check(lib.axr_rows_reference(strided[i % 2].data_ptr(), pitch, packed[i % 2].data_ptr(), run, rows,
                                                 scatter, nt, h.stream))
                ms = h.time_steps(step, k, 2)
                rate_ = 2.0 * rows * run * k / (ms * 1e-3) / 1e9
                every[str(nt)] = round(rate_, 1)
                if best is None or rate_ > best[0]:
                    best = (rate_, nt)
            res[name] = {"GBps": round(best[0], 1), "nontemporal_bits": best[1], "by_nontemporal_bits": every}
        g, sc = res["gather"]["GBps"], res["scatter"]["GBps"]
        res["pair_GBps"] = round(2.0 / (1.0 / g + 1.0 / sc), 1)
        res["payload_bytes_P"] = rows * run
        out["row_kernel"][label] = res
        del strided, packed
        torch.cuda.empty_cache()
    return out


def small_bundles_batched(h, bundles=16, tensors=4, each=16 * 1024, steps=200):
    """Sixteen small bundles (4 tensors of 16 KiB: the size of an RPC argument list) packed and
    unpacked with kept plans: one axr_pack / axr_unpack launch per bundle against ONE
    axr_submit launch for all sixteen packs and one for all unpacks.  us per bundle round trip."""
    torch, lib, capi = h.torch, h.lib, h.capi
    src = [[torch.randint(0, 255, (each,), dtype=torch.uint8, device="cuda") for _ in range(tensors)]
           for _ in range(bundles)]
    dst = [[torch.zeros_like(t) for t in b] for b in src]
    plans = [h.pkg.BundlePlan.create(b, align=256) for b in src]
    rplans = [h.pkg.BundlePlan.from_header(p.header).bind(d) for p, d in zip(plans, dst)]
    nbytes = plans[0].payload_bytes
    payloads = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(bundles)]
    for p in plans + rplans:
        p.prepare(h.stream)
    packs = (capi.Job * bundles)(*[capi.Job(p._h, 0, b.data_ptr(), nbytes, 0) for p, b in zip(plans, payloads)])
    unpacks = (capi.Job * bundles)(*[capi.Job(r._h, 1, b.data_ptr(), nbytes, 0) for r, b in zip(rplans, payloads)])
    calls = [(p._h, r._h, b.data_ptr()) for p, r, b in zip(plans, rplans, payloads)]

    def separate(i):
        rc = 0
        for pp, up, ptr in calls:
            rc |= lib.axr_pack(pp, ptr, nbytes, h.stream)
        for pp, up, ptr in calls:
            rc |= lib.axr_unpack(up, ptr, nbytes, h.stream)
        if rc:
            capi.check(rc)

    def batched(i):
        rc = lib.axr_submit(packs, bundles, h.stream) | lib.axr_submit(unpacks, bundles, h.stream)
        if rc:
            capi.check(rc)

    ms_sep = h.time_steps(separate, steps, 5)
    for d in dst:
        for t in d:
            t.zero_()
    h.sync()
    ms_bat = h.time_steps(batched, steps, 5)
    h.sync()
    if not all(bool(torch.equal(a, b)) for s_, d_ in zip(src, dst) for a, b in zip(s_, d_)):
        raise SystemExit("bench.py: batched small bundles did not reproduce the tensors")
    for p in plans + rplans:
        p.close()
    return {"bundles": bundles, "tensors_per_bundle": tensors, "bytes_per_tensor": each,
            "one_launch_per_bundle_us": round(ms_sep * 1e3 / (steps * bundles), 2),
            "sixteen_bundles_per_launch_us": round(ms_bat * 1e3 / (steps * bundles), 2)}


def small_segments(h, tensors=65536, lo=8, hi=512, copies=4, steps=400):
    """Bundles of many short tensors (RPC argument lists, norm scales, biases, optimizer
    scalars): `tensors` contiguous 1-D tensors of lo..hi bytes, log-uniform, five dtypes, at
    the benchmark's 256-byte alignment and in the reference's tight layout.  Pack-only,
    unpack-only and pack + unpack rates next to a plain device copy of the same byte count
    under the same rotation; launch geometry (wavefronts launched, device table bytes)."""
    from execution_ucx_amd import workloads
    torch, lib, check = h.torch, h.lib, h.capi.check
    spec = workloads.mixed_bundle(n=tensors, lo=lo, hi=hi, seed=3)
    out = {"tensors": tensors, "size_range_bytes": [lo, hi], "rotating_copies": copies}
    for align in (256, 1):
        _, sets = make_c2_sets(h, copies, seed=3, align=align, spec=spec)
        for s_ in sets:
            verify_set(h, s_)
        P = sets[0].data_bytes
        clear_sets(h, sets)
        pair = run_sets(h, sets, steps, 20)
        check_sets(h, sets, "the small-segment steps")
        one = run_sets_one_launch(h, sets, steps, 20)
        res = half_rates(h, sets, steps, 20)
        info = sets[0].pack_plan.launch_info()
        packed = sets[0].nbytes
        # what the kernels really move: the pack reads P and writes the packed buffer, gaps included
        # (zero bytes); the unpack reads P out of it and writes P
        res["pack_only"]["GBps_bytes_moved"] = round((P + packed) / (res["pack_only"]["avg_launch_us"] * 1e-6) / 1e9, 1)
        res["unpack_only"]["GBps_bytes_moved"] = res["unpack_only"]["GBps_2P"]
        res.update({"payload_bytes_P": P, "packed_bytes": sets[0].nbytes,
                    "pack_unpack_GBps_4P": round(rate(P, pair, steps), 1),
                    "one_launch_GBps_4P": round(rate(P, one, steps), 1),
                    "wavefronts": info["tiles"], "segments": info["segments"],
                    "table_bytes": info["table_bytes"]})
        out[f"align{align}"] = res
        del sets
        torch.cuda.empty_cache()
    n = (out["align1"]["payload_bytes_P"] + 15) // 16 * 16
    a = [torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda") for _ in range(copies)]
    b = [torch.empty_like(x) for x in a]
    h.sync()
    ms = h.time_steps(lambda i: check(lib.axr_copy_reference(b[i % copies].data_ptr(), a[i % copies].data_ptr(),
                                                             n, h.stream)), steps, 20)
    us = ms * 1e3 / steps
    out["plain_copy_same_bytes"] = {"bytes": n, "GBps_2n": round(2.0 * n / (us * 1e-6) / 1e9, 1),
                                    "avg_launch_us": round(us, 3)}
    for align in (256, 1):
        r = out[f"align{align}"]
        r["pack_vs_plain_copy"] = round(r["pack_only"]["GBps_2P"] / out["plain_copy_same_bytes"]["GBps_2n"], 3)
        r["pack_bytes_moved_vs_plain_copy"] = round(r["pack_only"]["GBps_bytes_moved"] /
                                                    out["plain_copy_same_bytes"]["GBps_2n"], 3)
        r["unpack_vs_plain_copy"] = round(r["unpack_only"]["GBps_2P"] / out["plain_copy_same_bytes"]["GBps_2n"], 3)
    # a bundle seen for the first time: plan -> pack -> sync -> header decode + bind -> unpack -> sync
    # (the group tables are built on the host; nothing is reused between repetitions)
    fresh = end_to_end_us(h, spec, steps=10)
    out["fresh_bundle"] = {k: round(v, 2) for k, v in fresh.items()}
    return out


def plain_copy_of(h, nbytes):
    """A plain device copy that reads and writes as many bytes as one step of the headline does
    (`nbytes` read, `nbytes` written), with rotating buffers, in the library's grid-stride copy
    kernel and in the best of its wavefront-shaped ones: the yardstick without tables, segments,
    gaps or partly filled tiles."""
    torch, lib, check = h.torch, h.lib, h.capi.check
    n = nbytes // 4096 * 4096
    copies = max(2, int((600 << 20) // (2 * n)) + 1)
    a = [torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda") for _ in range(copies)]
    b = [torch.empty_like(x) for x in a]
    h.sync()
    k = max(50, int(2e10 // n) // 10)
    out = {"bytes_read": n, "bytes_written": n, "rotating_buffer_pairs": copies}
    ms = h.time_steps(lambda i: check(lib.axr_copy_reference(b[i % copies].data_ptr(), a[i % copies].data_ptr(),
                                                             n, h.stream)), k, 5)
    out["grid_stride_256_threads"] = {"GBps": round(2.0 * n * k / (ms * 1e-3) / 1e9, 1), "us_per_launch": round(ms * 1e3 / k, 2)}
    best = None
    for threads, kib, nt in ((64, 1, 1), (256, 1, 1), (128, 2, 1), (256, 2, 1), (256, 2, 0)):
        ms = h.time_steps(lambda i: check(lib.axr_copy_reference_shaped(
            b[i % copies].data_ptr(), a[i % copies].data_ptr(), n, threads, kib, nt, h.stream)), k, 5)
        res = {"GBps": round(2.0 * n * k / (ms * 1e-3) / 1e9, 1), "us_per_launch": round(ms * 1e3 / k, 2),
               "shape": f"{threads} threads, {kib} KiB per wavefront, {'streaming' if nt else 'ordinary'} accesses"}
        if best is None or res["GBps"] > best["GBps"]:
            best = res
    if not bool(torch.equal(a[0], b[0])):
        raise SystemExit("bench.py: the plain copy did not copy")
    out["best_shape"] = best
    return out


def load_traffic(kernel_key):
    path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel_key)
    except (OSError, ValueError):
        return None


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the bundle path has no cross-GPU "
                 "step); run with --gpus 1")
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg._capi.load()          # no HIP library -> ImportError, there is no fallback
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    for kv in filter(None, args.tune.split(",")):
        k, v = kv.split("=")
        pkg.tune(**{k: int(v)})
    h = Harness(pkg)
    from execution_ucx_amd import workloads

    if args.ceilings:
        print(json.dumps({"ceilings": ceilings(h)}))
        return
    if args.small_segments:
        print(json.dumps({"small_segments": small_segments(h)}))
        return
    spec = workloads.mixed_bundle()
    extras = {}
    if args.workload == "c2":
        _, sets = make_c2_sets(h, max(1, args.rotate), align=args.align)
        name = ("C2 mixed small-tensor bundle: 4096 contiguous 1-D tensors, log-uniform "
                f"256 B-64 KiB, fp16/bf16/fp32/int32/int8, {args.align} B aligned offsets")
    elif args.workload == "small":
        small_spec = workloads.mixed_bundle(n=65536, lo=8, hi=512, seed=3)
        _, sets = make_c2_sets(h, max(1, args.rotate), seed=3, align=args.align, spec=small_spec)
        name = ("65,536 contiguous 1-D tensors, log-uniform 8 B-512 B, five dtypes, "
                f"{args.align} B aligned offsets")
    elif args.workload == "c3":
        sets = make_c3_sets(h, max(1, args.rotate))
        name = "C3 Llama-7B single-layer weight bundle, bf16, 9 tensors"
    elif args.workload == "c4":
        sets = [make_c4_set(h)]
        name = "C4 strided KV-cache block gather/scatter, 512 blocks x 32 layers"
    elif args.workload == "transposed":
        sets = make_transposed_sets(h, max(1, min(args.rotate, 2)))
        name = "8 transposed 4096 x 4096 bf16 matrices (x.t() views), 256 MiB"
    elif args.workload in VIEW_WORKLOADS:
        sets = make_view_sets(h, max(1, min(args.rotate, 2)), args.workload)
        name = VIEW_WORKLOADS[args.workload][0]
    else:
        sets = make_c5_sets(h, max(1, min(args.rotate, 2)))
        name = "C5 chunk: 64 pitched 2-D views, 256 MiB"
    for s in sets:
        verify_set(h, s)
    P = sets[0].data_bytes
    pipelined = len(sets) >= 2 and not args.separate_launches
    clear_sets(h, sets)
    if pipelined:
        ms = run_sets_one_launch(h, sets, args.steps, args.warmup)
        launches_per_step, bytes_per_launch = 1, 4 * P
        kernel = "axr::bundle_jobs_kernel (one launch: pack of bundle i+1 and unpack of bundle i)"
    elif args.direction != "both":
        ms = run_sets_one_direction(h, sets, args.steps, args.warmup, args.direction == "unpack")
        launches_per_step, bytes_per_launch = 1, 2 * P
        kernel = f"axr::bundle_kernel ({args.direction} instantiation only)"
    else:
        ms = run_sets(h, sets, args.steps, args.warmup)
        launches_per_step, bytes_per_launch = 2, 2 * P
        kernel = "axr::bundle_kernel (pack and unpack instantiations)"
    batches = h.batches
    if all(s.clear is not None for s in sets) and (pipelined or args.direction == "both"):
        check_sets(h, sets, "the timed steps")
    value = rate(P, ms, args.steps) * (0.5 if (not pipelined and args.direction != "both") else 1.0)
    info = sets[0].pack_plan.launch_info()
    launch_us = ms * 1e3 / (launches_per_step * args.steps)
    achieved = bytes_per_launch / (launch_us * 1e-6) / 1e9
    traffic = load_traffic(args.workload if not pipelined else args.workload + "_one_launch")

    result = {
        "metric": "bundle pack+unpack GB/s (read+write)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms / args.steps, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {
            "workload": name,
            "tensors": sets[0].pack_plan.num_tensors,
            "payload_bytes_P": P,
            "packed_bytes": sets[0].nbytes,
            "rotating_copies": len(sets),
            "working_set_bytes": len(sets) * 3 * sets[0].nbytes,
            "step": ("pack of bundle i+1 and unpack of bundle i in one launch (axr_submit), one stream"
                     if pipelined else "axr_pack then axr_unpack of one bundle, two launches, one stream"),
            "timing": f"median of {batches} batches of {args.steps} steps, HIP events on the launch stream",
            "launch": info,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "value_note": ("bytes the step moves (4P, read + written) per second against the 8 TB/s HBM peak.  With "
                       f"{len(sets)} rotating copies the payloads ({len(sets)} x {sets[0].nbytes} B) still fit the "
                       "256 MB last-level cache, so the unpack half reads a payload that was written one step "
                       "earlier out of that cache: extras.c2_payload_streaming is the same step with the payload "
                       "bypassing the cache on both sides, and --rotate 8 the step with everything coming from HBM"
                       if args.workload == "c2" else "bytes moved (read + written) per second against the 8 TB/s HBM peak"),
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": ("profiles/pmc_traffic.json: FETCH_SIZE and WRITE_SIZE of earlier rocprofv3 --pmc "
                               "runs of this command, scaled by a plain copy; not measured in this run"
                               if traffic is not None else None),
            "kernel": kernel,
            "bytes_per_launch": bytes_per_launch,
            "avg_launch_us": round(launch_us, 3),
        },
    }

    if not args.no_extras and args.workload == "c2":
        def c2_variant(align=256, **tune):
            """The headline steps on fresh plans under other tunables / another layout."""
            defaults = {k: tune_get(pkg, k) for k in tune}
            pkg.tune(**tune)
            try:
                _, vs = make_c2_sets(h, len(sets), align=align)
                for v in vs:
                    verify_set(h, v)
                clear_sets(h, vs)
                one = run_sets_one_launch(h, vs, args.steps, args.warmup)
                check_sets(h, vs, "a C2 variant")
                two = run_sets(h, vs, args.steps, args.warmup)
                res = {"one_launch_GBps": round(rate(P, one, args.steps), 1),
                       "separate_launches_GBps": round(rate(P, two, args.steps), 1)}
                res.update(half_rates(h, vs, args.steps, args.warmup))
                return res
            finally:
                pkg.tune(**defaults)

        ms_sep = run_sets(h, sets, args.steps, args.warmup)
        extras["c2_separate_launches_GBps"] = round(rate(P, ms_sep, args.steps), 1)
        # a deployed sender and receiver are different processes: each half on its own
        halves = half_rates(h, sets, args.steps, args.warmup)
        extras["c2_pack_only"], extras["c2_unpack_only"] = halves["pack_only"], halves["unpack_only"]
        # cache-resident rate of the same bundle (one copy only: pack then unpack)
        ms1 = run_sets(h, sets[:1], args.steps, args.warmup)
        extras["c2_cache_resident_GBps"] = round(rate(P, ms1, args.steps), 1)
        # not `value`: bundles in flight on two streams hide the gap between dependent launches
        ms2 = run_sets_two_streams(h, sets, args.steps, args.warmup)
        extras["c2_two_streams_GBps"] = round(rate(P, ms2, args.steps), 1)
        # a sender or a receiver alone, its independent bundles alternating between two streams (2P per launch)
        both = {}
        for name, unpack in (("pack", False), ("unpack", True)):
            ms = run_sets_one_direction_two_streams(h, sets, args.steps, args.warmup, unpack)
            gbps = 2.0 * P * args.steps / (ms * 1e-3) / 1e9
            both[name + "_only"] = {"GBps_2P": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
        extras["c2_one_direction_two_streams"] = both
        check_sets(h, sets, "the two-stream one-direction steps")
        extras["c2_graph_replay_GBps"] = graph_replay(h, sets, P)
        if len(sets) >= 4 and len(sets) % 2 == 0:
            # not `value`: two bundles each way per launch (four jobs), the fixed cost of a launch paid once
            clear_sets(h, sets)
            ms4 = run_sets_one_launch(h, sets, max(1, args.steps // 2), args.warmup, width=2)
            check_sets(h, sets, "the four-job steps")
            extras["c2_two_bundles_per_launch_GBps"] = round(rate(P, ms4, 2 * max(1, args.steps // 2)), 1)
        # the reference's own layout (tight concatenation) and a payload that bypasses the
        # last-level cache on both sides
        extras["c2_tight"] = c2_variant(align=1)
        # same geometry, both sides non-temporal (lowering payload_cache_bytes instead would also
        # switch the bundle to the tile geometry of payloads that stream)
        extras["c2_payload_streaming"] = c2_variant(nontemporal=3)
        extras["plain_copy_of_the_step_bytes"] = plain_copy_of(h, 2 * P)
        extras.update({k: round(v, 2) for k, v in end_to_end_us(h, spec).items()})
        extras["fresh_bundle_from_cpp"] = end_to_end_from_cpp()
        del sets
        torch.cuda.empty_cache()
        c3 = make_c3_sets(h, 2)
        verify_set(h, c3[0])
        k3 = max(20, args.steps // 20)
        ms3 = run_sets(h, c3, k3, 5)
        ms3b = run_sets_one_launch(h, c3, k3, 5)
        check_sets(h, c3, "C3")
        halves = half_rates(h, c3, k3, 5)
        extras["c3_pack_only"], extras["c3_unpack_only"] = halves["pack_only"], halves["unpack_only"]
        extras["c3_llama_layer"] = {"GBps": round(rate(c3[0].data_bytes, ms3, k3), 1),
                                    "pct_of_hbm_peak": round(100 * rate(c3[0].data_bytes, ms3, k3) / HBM_PEAK_GBPS, 2),
                                    "one_launch_GBps": round(rate(c3[0].data_bytes, ms3b, k3), 1),
                                    "payload_bytes_P": c3[0].data_bytes, "steps": k3,
                                    "ms_per_step": round(ms3 / k3, 5)}
        del c3
        torch.cuda.empty_cache()
        c5 = make_c5_sets(h, 2)
        verify_set(h, c5[0])
        k5 = max(20, args.steps // 20)
        ms5 = run_sets(h, c5, k5, 5)
        extras["c5_pitched_chunk"] = {"GBps": round(rate(c5[0].data_bytes, ms5, k5), 1),
                                      "payload_bytes_P": c5[0].data_bytes, "steps": k5}
        del c5
        torch.cuda.empty_cache()
        tr = make_transposed_sets(h, 2)
        verify_set(h, tr[0])
        mst = run_sets(h, tr, k5, 5)
        extras["transposed_views"] = {"GBps": round(rate(tr[0].data_bytes, mst, k5), 1),
                                      "payload_bytes_P": tr[0].data_bytes, "steps": k5}
        del tr
        torch.cuda.empty_cache()
        strided = {}
        for wl in VIEW_WORKLOADS:
            vs = make_view_sets(h, 2, wl)
            verify_set(h, vs[0])
            msv = run_sets(h, vs, k5, 5)
            check_sets(h, vs, wl)
            strided[wl] = {"GBps": round(rate(vs[0].data_bytes, msv, k5), 1), "payload_bytes_P": vs[0].data_bytes}
            del vs
            torch.cuda.empty_cache()
        extras["strided_views"] = strided
        extras["fresh_small_bundle"] = fresh_small_round_trip(h)
        # the same with axr_stream_synchronize polling a word of pinned memory first (opt-in)
        pkg.tune(spin_wait_us=200)
        try:
            extras["fresh_small_bundle"]["round_trip_us_with_polled_wait"] = fresh_small_round_trip(h)["round_trip_us"]
        finally:
            pkg.tune(spin_wait_us=0)
        extras["small_bundles_batched"] = small_bundles_batched(h)
        extras["small_segments"] = small_segments(h)
        extras["c1_host_bundle"] = host_bundle_c1(h)
        extras["loopback_iov_vs_bundle"] = iov_against_bundle(h, spec)
        extras["python_plan_us_per_1k_tensors"] = python_boundary(h, spec)
        extras["checkpoint_to_host"] = checkpoint_staging(h)
        extras["c5_streamed_8GiB"] = stream_c5(h)
        torch.cuda.empty_cache()
        c4 = make_c4_set(h)
        verify_set(h, c4)
        k4 = max(10, args.steps // 100)
        ms4 = run_sets(h, [c4], k4, 3)
        extras["c4_kv_gather"] = {"GBps": round(rate(c4.data_bytes, ms4, k4), 1),
                                  "payload_bytes_P": c4.data_bytes, "steps": k4}
        halves = half_rates(h, [c4], k4, 3)
        extras["c4_pack_only"], extras["c4_unpack_only"] = halves["pack_only"], halves["unpack_only"]
        del c4
        torch.cuda.empty_cache()
    if args.calibrate_copy:
        n = 256 << 20
        a = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        for _ in range(args.calibrate_copy):
            pkg._capi.check(h.lib.axr_copy_reference(b.data_ptr(), a.data_ptr(), n, h.stream))
        h.sync()
        extras["calibration_copy_bytes"] = n
    result["extras"] = extras

    if not args.no_cpu:
        base, allc = cpu_baseline(spec)
        result["cpu_baseline"] = base
        result["cpu_baseline_all_cores"] = allc
        if not args.no_extras:
            extras.update(cpu_baseline_other_configs())
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
