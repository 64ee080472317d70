"""The loopback AM context against the behaviour the reference's tests pin
(ucx_am_connection_test.cpp, ucx_am_context_test.cpp).  Host-memory cases run
without a GPU; the device cases are marked gpu."""
import numpy as np
import pytest

HOST, ROCM = 0, 3


def pattern(n, start=0):
    return ((np.arange(n, dtype=np.uint64) + start) % 256).astype(np.uint8)


@pytest.fixture
def pair(pkg):
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    yield client, server, conn
    client.close()
    server.close()


def test_header_is_required_and_payload_may_be_empty(pkg, pair):
    client, server, conn = pair
    with pytest.raises(pkg.AxonRocmError):
        client.send(conn, b"", 0, 0, memory_type=HOST)
    with pytest.raises(pkg.AxonRocmError):
        client.send(conn + 12345, b"h", 0, 0, memory_type=HOST)      # unknown connection
    req = client.send(conn, b"only header", 0, 0, memory_type=HOST)
    assert client.test(req)
    m = server.recv_header()
    assert m.header == b"only header" and m.data_length == 0 and not m.is_rndv and m.eager_data == b""
    assert m.conn_id == conn
    assert server.recv_header() is None


def test_eager_below_threshold_rendezvous_above(pkg):
    # UCX_ZCOPY_THRESH default 4096 (ucx_connection.cpp:45); tests force 8192 (ucx_am_context_test.cpp:131)
    client, server = pkg.LoopbackAmContext("c", zcopy_thresh=8192), pkg.LoopbackAmContext("s")
    conn = client.connect(server)
    src = pattern(8192)
    r_small = client.send(conn, b"\x01", src.ctypes.data, 8191, memory_type=HOST)
    r_big = client.send(conn, b"\x02", src.ctypes.data, 8192, memory_type=HOST)
    assert client.test(r_small) and not client.test(r_big)
    small = server.recv_header(release_eager=False)
    assert not small.is_rndv and small.eager_data == src[:8191].tobytes()
    dst = np.zeros(8192, np.uint8)
    with pytest.raises(pkg.NotImplementedForEager):          # UCS_ERR_NOT_IMPLEMENTED
        server.recv_into(small, dst.ctypes.data, 8192, memory_type=HOST)
    server.release(small)
    big = server.recv_header()
    assert big.is_rndv and big.data_length == 8192 and big.eager_data is None
    with pytest.raises(pkg.LengthError):
        server.recv_into(big, dst.ctypes.data, 100, memory_type=HOST)
    server.recv_into(big, dst.ctypes.data, 8192, memory_type=HOST)
    assert np.array_equal(dst, src) and client.test(r_big)
    with pytest.raises(pkg.NoMessageError):                  # UCS_ERR_NO_MESSAGE
        server.recv_into(big, dst.ctypes.data, 8192, memory_type=HOST)


@pytest.mark.parametrize("lens", [(256, 512, 300), (512 * 1024, 256 * 1024, 800 * 1024)])
def test_iov_send_contiguous_and_iov_receive_kat(pkg, pair, lens):
    """ucx_am_connection_test.cpp:933-1108: iov -> contiguous equals the flat
    pattern; iov -> iov of the same lengths equals the segments; header echoed."""
    client, server, conn = pair
    segs, cursor = [], 0
    for n in lens:
        segs.append(pattern(n, cursor))
        cursor += n
    bufs = [(s.ctypes.data, s.size) for s in segs]
    r1 = client.send_iov(conn, bytes([1, 2, 3, 4]), bufs, memory_type=HOST)
    r2 = client.send_iov(conn, bytes([1, 2, 3, 4]), bufs, memory_type=HOST)
    assert not client.test(r1)                               # iov is always rendezvous
    m = server.recv_header()
    assert m.header == bytes([1, 2, 3, 4]) and m.is_rndv and m.data_length == sum(lens)
    flat = np.zeros(sum(lens), np.uint8)
    server.recv_into(m, flat.ctypes.data, flat.size, memory_type=HOST)
    assert np.array_equal(flat, pattern(sum(lens)))
    m2 = server.recv_header()
    outs = [np.zeros(n, np.uint8) for n in lens]
    server.recv_buffer_iov(m2, [(o.ctypes.data, o.size) for o in outs], memory_type=HOST)
    for o, s in zip(outs, segs):
        assert np.array_equal(o, s)
    assert client.test(r1) and client.test(r2)


def test_iov_receive_needs_allocated_entries(pkg, pair):
    client, server, conn = pair
    src = pattern(100)
    client.send_iov(conn, b"h", [(src.ctypes.data, 100)], memory_type=HOST)
    m = server.recv_header()
    dst = np.zeros(100, np.uint8)
    with pytest.raises(pkg.AxonRocmError):
        server.recv_buffer_iov(m, [(dst.ctypes.data, 50), (0, 50)], memory_type=HOST)
    with pytest.raises(pkg.AxonRocmError):
        server.recv_buffer_iov(m, [(dst.ctypes.data, 100), (dst.ctypes.data, 0)], memory_type=HOST)
    server.recv_buffer_iov(m, [(dst.ctypes.data, 40), (dst.ctypes.data + 40, 60)], memory_type=HOST)
    assert np.array_equal(dst, src)


def test_fifo_order_and_cancel(pkg, pair):
    client, server, conn = pair
    src = pattern(10000)
    reqs = [client.send(conn, bytes([i]), src.ctypes.data + i, 5000, memory_type=HOST) for i in range(5)]
    assert server.pending() == 5
    for i in range(5):
        m = server.recv_header()
        assert m.header == bytes([i])
        if i == 2:
            server.release(m)                                # receiver drops the descriptor
            with pytest.raises(pkg.AxonRocmError):
                client.test(reqs[i])
            continue
        dst = np.zeros(5000, np.uint8)
        server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
        assert np.array_equal(dst, src[i:i + 5000]) and client.test(reqs[i])


def test_at_most_256_sends_in_flight_the_rest_wait_in_order(pkg, pair):
    """kCompletionQueueEntryCount (ucx_am_context.hpp:94,836-839): 256 operations may be
    under way; further ones are queued and submitted, first in first out, as completions
    make room (ucx_am_context.cpp:271-274).  An eager send behind waiting ones keeps its
    place in the order."""
    client, server, conn = pair
    src = pattern(300 * 8 + 5000)
    total = 300
    reqs = [client.send(conn, i.to_bytes(2, "little"), src.ctypes.data + 8 * i, 5000, memory_type=HOST)
            for i in range(total)]
    assert client.progress() == (256, total - 256)
    assert server.pending() == 256                           # the others have not been sent yet
    small = client.send(conn, b"eager", src.ctypes.data, 16, memory_type=HOST)   # below the threshold
    assert client.progress() == (256, total - 256 + 1) and server.pending() == 256
    dst = np.zeros(5000, np.uint8)
    for i in range(10):                                      # ten fetches make room for ten sends
        m = server.recv_header()
        assert int.from_bytes(m.header, "little") == i
        server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
        assert np.array_equal(dst, src[8 * i:8 * i + 5000])
    assert server.pending() == 246                           # nothing moves before the sender progresses
    assert client.test(reqs[0])                              # ... which a test of a request does
    assert client.progress() == (256, total - 256 + 1 - 10) and server.pending() == 256
    seen = []
    while True:
        m = server.recv_header()
        if m is None:
            if client.progress() == (0, 0):
                break
            continue
        if m.is_rndv:
            seen.append(int.from_bytes(m.header, "little"))
            server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
            assert np.array_equal(dst, src[8 * seen[-1]:8 * seen[-1] + 5000])
        else:
            seen.append(m.header)
            assert m.eager_data == bytes(src[:16])
    assert seen == list(range(10, total)) + [b"eager"]       # the order of the calls
    assert all(client.test(r) for r in reqs[1:]) and client.test(small)


def test_sender_cancels_waiting_and_unfetched_sends(pkg, pair):
    client, server, conn = pair
    src = pattern(9000)
    reqs = [client.send(conn, bytes([i % 251]), src.ctypes.data, 5000, memory_type=HOST) for i in range(260)]
    assert client.progress() == (256, 4)
    # a send that still waits for room: dropped before it reaches the peer
    client.cancel(reqs[258])
    assert client.progress() == (256, 3)
    with pytest.raises(pkg.AxonRocmError):
        client.test(reqs[258])
    # a rendezvous the receiver has not looked at: it never shows up, and its slot is free again
    client.cancel(reqs[0])
    assert client.progress() == (256, 2)                     # 255 + one waiting send started
    m = server.recv_header()
    assert m.header == bytes([1])
    # one the receiver holds the header of: its fetch fails, nothing is copied
    client.cancel(reqs[1])
    dst = np.full(5000, 7, np.uint8)
    with pytest.raises(pkg.AxonRocmError) as e:
        server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
    assert e.value.status == pkg._capi.AXR_ERR_CANCELED and (dst == 7).all()
    # a completed send cannot be cancelled any more
    m = server.recv_header()
    assert m.header == bytes([2])
    server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
    client.cancel(reqs[2])
    assert client.test(reqs[2]) and np.array_equal(dst, src[:5000])
    # the rest arrives in order, without the cancelled ones
    seen = []
    while True:
        m = server.recv_header()
        if m is None:
            if client.progress() == (0, 0):
                break
            continue
        seen.append(m.header[0])
        server.recv_into(m, dst.ctypes.data, 5000, memory_type=HOST)
    assert seen == [i % 251 for i in range(3, 260) if i != 258]
    with pytest.raises(pkg.AxonRocmError):
        client.cancel(10 ** 9)                               # unknown request


def test_send_to_a_destroyed_peer_is_an_error(pkg):
    """An endpoint outlives its peer context; sending on it fails cleanly (a closed
    connection is an error_code in the reference, ucx_am_context.hpp:2318-2392) and
    the request reads as failed."""
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    src = pattern(10000)
    ok = client.send(conn, b"first", src.ctypes.data, 10000, memory_type=HOST)
    server.close()                                           # the queued rendezvous send is cancelled
    with pytest.raises(pkg.AxonRocmError):
        client.test(ok)
    with pytest.raises(pkg.AxonRocmError, match="destroyed"):
        client.send(conn, b"second", src.ctypes.data, 10000, memory_type=HOST)
    other = pkg.LoopbackAmContext("other")                   # the client itself still works
    conn2 = client.connect(other)
    client.send(conn2, b"third", src.ctypes.data, 16, memory_type=HOST)
    assert other.recv_header().header == b"third"
    client.close()
    other.close()


def test_unsupported_memory_type(pkg, pair):
    client, server, conn = pair
    src = pattern(10)
    with pytest.raises(pkg.UnsupportedMemoryError):
        client.send(conn, b"h", src.ctypes.data, 10, memory_type=1)      # ucx_memory_type::CUDA


# ------------------------------------------------------------------ device cases

@pytest.mark.gpu
def test_c1_host_bundle_end_to_end(pkg, orc, gpu):
    """The host-memory bundle: 64 fp32 host tensors -> one packed buffer + header ->
    loopback AM -> unpack -> byte-for-byte."""
    import torch
    from execution_ucx_amd import workloads
    srcs = workloads.host_bundle_c1(seed=0)
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    stream = torch.cuda.current_stream().cuda_stream
    packed = pkg.pack_bundle(srcs, align=1, stream=stream)
    req = client.send_bundle(conn, packed, stream=stream)
    msg = server.recv_header()
    assert msg.is_rndv and msg.data_length == 4 << 20 and msg.buffer_type == ROCM
    assert msg.header == packed.header
    recv = server.recv_buffer(msg, stream=stream)            # allocates from the pool
    assert client.test(req)
    host = np.zeros(4 << 20, np.uint8)
    pkg.RocmMemoryResourceManager().memcpy(HOST, host.ctypes.data, ROCM, recv.data, host.size)
    assert np.array_equal(host, orc.pack([s.view(np.uint8) for s in srcs], 1))
    outs = [np.zeros_like(s) for s in srcs]
    plan = pkg.unpack_bundle(msg.header, recv, out=outs, stream=stream)
    torch.cuda.synchronize()
    plan.close()
    for a, b in zip(srcs, outs):
        assert a.tobytes() == b.tobytes()
    recv.release()
    packed.payload.release()


@pytest.mark.gpu
def test_device_iov_equals_packed_bundle(pkg, orc, gpu):
    """The reference's way (one iov entry per tensor, gathered by the transport)
    and this build's way (one pack kernel, one contiguous send) deliver the same
    bytes for the tight layout."""
    import torch
    rng = np.random.default_rng(3)
    tensors = [torch.from_numpy(rng.integers(0, 256, size=int(n), dtype=np.uint8)).to(gpu)
               for n in rng.integers(1, 300000, size=40)]
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    stream = torch.cuda.current_stream().cuda_stream
    packed = pkg.pack_bundle(tensors, align=1, stream=stream)
    r_iov = client.send_iov(conn, packed.header, [(t.data_ptr(), t.numel()) for t in tensors], ROCM,
                            stream=stream, keep=tensors)
    r_one = client.send_bundle(conn, packed, stream=stream)
    m_iov, m_one = server.recv_header(), server.recv_header()
    assert m_iov.data_length == m_one.data_length == packed.payload_bytes
    b_iov = server.recv_buffer(m_iov, stream=stream)
    b_one = server.recv_buffer(m_one, stream=stream)
    assert client.test(r_iov) and client.test(r_one)
    n = packed.payload_bytes
    got_iov = torch.empty(n, dtype=torch.uint8, device=gpu)
    got_one = torch.empty(n, dtype=torch.uint8, device=gpu)
    mr = pkg.RocmMemoryResourceManager()
    mr.memcpy(ROCM, got_iov.data_ptr(), ROCM, b_iov.data, n)
    mr.memcpy(ROCM, got_one.data_ptr(), ROCM, b_one.data, n)
    assert torch.equal(got_iov, got_one)
    want = orc.pack([t.cpu().numpy() for t in tensors], 1)
    assert np.array_equal(got_one.cpu().numpy(), want)
    # zero-copy receive: views over the received buffer, typed from the header
    outs = pkg.unpack_bundle(m_one.header, b_one, from_dlpack_fn=torch.from_dlpack)
    for t, o in zip(tensors, outs):
        assert torch.equal(t, o)


@pytest.mark.gpu
def test_device_eager_and_process_reply(pkg, gpu):
    """Small device payload goes eager through host memory; the send -> process ->
    reply round trip of ucx_am_context_test.cpp:1893-1944 with the halving kernel."""
    import torch
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    c2s, s2c = client.connect(server), server.connect(client)
    lib = pkg._capi.load()
    for n in (32, 1 << 20):
        x = torch.from_numpy((np.arange(n) % 256).astype(np.float32)).to(gpu)
        torch.cuda.synchronize()
        req = client.send(c2s, b"req", x.data_ptr(), 4 * n, ROCM, keep=x)
        m = server.recv_header()
        if 4 * n < 4096:
            assert not m.is_rndv
            y = torch.from_numpy(np.frombuffer(m.eager_data, dtype=np.float32).copy()).to(gpu)
        else:
            buf = server.recv_buffer(m)
            y = torch.empty(n, dtype=torch.float32, device=gpu)
            pkg.RocmMemoryResourceManager().memcpy(ROCM, y.data_ptr(), ROCM, buf.data, 4 * n)
            buf.release()
        assert client.test(req)
        pkg._capi.check(lib.axr_divide_by_two(y.data_ptr(), n, None))
        torch.cuda.synchronize()
        rep = server.send(s2c, b"rep", y.data_ptr(), 4 * n, ROCM, keep=y)
        r = client.recv_header()
        if r.is_rndv:
            z = torch.empty(n, dtype=torch.float32, device=gpu)
            client.recv_into(r, z.data_ptr(), 4 * n, ROCM)
            got = z.cpu().numpy()
        else:
            got = np.frombuffer(r.eager_data, dtype=np.float32)
        assert server.test(rep)
        assert np.array_equal(got, (np.arange(n) % 256).astype(np.float32) / 2)


@pytest.mark.gpu
def test_send_recv_tensors_with_memory_policy(pkg, gpu):
    """Receive side of the memory-policy contract: the policy sees the metas, its
    own tensors come back filled; without a policy the result is zero-copy views;
    a tiny bundle goes the eager way through host memory."""
    import torch
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    stream = torch.cuda.current_stream().cuda_stream
    big = [torch.randn(5000, device=gpu), torch.randn(33, 77, device=gpu).to(torch.bfloat16),
           torch.arange(1000, device=gpu, dtype=torch.int32)]
    tiny = [torch.arange(10, device=gpu, dtype=torch.int32), torch.ones(3, device=gpu)]
    for tensors, rndv in ((big, True), (tiny, False)):
        seen = {}

        def policy(metas):
            seen["metas"] = metas
            seen["outs"] = [torch.zeros(m.shape, dtype=t.dtype, device=gpu) for m, t in zip(metas, tensors)]
            return seen["outs"]

        req, bundle = pkg.send_tensors(client, conn, tensors, stream=stream)
        assert server.pending() == 1
        got = pkg.recv_tensors(server, memory_policy=policy, stream=stream)
        assert client.test(req)
        assert [m.shape for m in seen["metas"]] == [tuple(t.shape) for t in tensors]
        assert all(g is o for g, o in zip(got, seen["outs"]))         # the policy's own objects
        for a, b in zip(tensors, got):
            assert torch.equal(a, b)
        req, bundle2 = pkg.send_tensors(client, conn, tensors, stream=stream)
        views = pkg.recv_tensors(server, from_dlpack_fn=torch.from_dlpack, stream=stream)
        assert client.test(req)
        for a, b in zip(tensors, views):
            assert torch.equal(a, b) and b.device.type == "cuda"
        with pytest.raises(RuntimeError):
            pkg.send_tensors(client, conn, tensors, stream=stream)
            pkg.recv_tensors(server, memory_policy=lambda metas: [torch.zeros(1, device=gpu)], stream=stream)
        assert (bundle.payload_bytes >= 4096) == rndv
    assert pkg.recv_tensors(server) is None


# ------------------------------------------------------------------ argument structure

def test_arguments_are_classified_and_flattened_like_the_reference(pkg):
    """ClassifyArg / add_tensor / add_nested_tensor_list
    (bindings_runtime_helpers.hpp:262-330, 351-414): tensors in argument order, nested
    lists flattened with their group sizes kept, empty inner lists allowed."""
    t = [np.full(i + 1, i, np.float32) for i in range(8)]
    args = [t[0], [t[1], t[2]], [[t[3]], [], [t[4], t[5]]], (t[6],), [], t[7]]
    assert [pkg.classify_argument(a) for a in args] == [1, 2, 3, 2, 2, 1]
    flat, structure = pkg.flatten_arguments(args)
    assert [id(x) for x in flat] == [id(x) for x in t]                # argument order, depth first
    assert structure == [(1, []), (2, [2]), (3, [1, 0, 2]), (2, [1]), (2, [0]), (1, [])]
    from execution_ucx_amd import transfer
    blob = transfer.encode_structure(structure)
    assert blob[:4] == b"AXAG" and len(blob) == 8 + 6 * 5 + 4 * (1 + 3 + 1 + 1)
    back, rest = transfer.decode_structure(blob + b"AXTBrest")
    assert back == structure and rest == b"AXTBrest"
    assert transfer.decode_structure(b"AXTBplain") == ([], b"AXTBplain")
    again = pkg.regroup(structure, flat)
    assert again[0] is t[0] and again[2] == [[t[3]], [], [t[4], t[5]]] and again[4] == [] and again[5] is t[7]
    assert isinstance(again[3], list) and again[3][0] is t[6]
    with pytest.raises(RuntimeError, match="Not enough tensors"):
        pkg.regroup(structure, flat[:-2])
    with pytest.raises(RuntimeError):
        pkg.regroup(structure, flat + [t[0]])
    with pytest.raises(ValueError):
        transfer.decode_structure(blob[:-3])
    with pytest.raises(ValueError):
        transfer.decode_structure(b"AXAG" + (1).to_bytes(4, "little") + bytes([7]) + (0).to_bytes(4, "little"))

    # what the reference refuses (or sends as plain parameters) is refused here
    with pytest.raises(TypeError, match="Heterogeneous"):
        pkg.classify_argument([[], t[1], [t[0]]])                    # met while scanning for a tensor
    assert pkg.classify_argument([[t[0]], t[1]]) == 3                # the scan stops at the first tensor ...
    with pytest.raises(TypeError, match="Heterogeneous"):
        pkg.flatten_arguments([[[t[0]], t[1]]])                      # ... and flattening meets the stray one
    with pytest.raises(TypeError, match="nested sequence"):
        pkg.classify_argument([[1, 2], [3]])
    with pytest.raises(TypeError):
        pkg.classify_argument([[], []])                              # only empty inner lists: no tensors
    with pytest.raises(TypeError):
        pkg.classify_argument(3.5)
    with pytest.raises(TypeError, match="DLManagedTensor"):
        pkg.flatten_arguments([[t[0], "not a tensor"]])


def test_argument_structure_matches_the_oracle_and_the_fixture(pkg, orc):
    """The package's flattening, framing and regrouping against the oracle's restatement
    of the reference on random nestings, and against the committed fixture."""
    import json
    import os
    from execution_ucx_amd import transfer
    kinds = {1: "single", 2: "flat", 3: "nested"}
    rng = np.random.default_rng(4)
    mk = lambda: np.zeros(int(rng.integers(1, 5)), np.float32)
    for _ in range(200):
        args = []
        for _ in range(int(rng.integers(0, 6))):
            k = int(rng.integers(0, 3))
            if k == 0:
                args.append(mk())
            elif k == 1:
                args.append([mk() for _ in range(int(rng.integers(0, 4)))])
            else:
                inner = [[mk() for _ in range(int(rng.integers(0, 4)))] for _ in range(int(rng.integers(1, 4)))]
                if not any(inner):
                    inner.append([mk()])            # only empty inner lists hold no tensor at all
                args.append(inner)
        flat, structure = pkg.flatten_arguments(args)
        oflat, ostructure = orc.flatten_arguments(args, lambda x: isinstance(x, np.ndarray))
        assert [id(x) for x in flat] == [id(x) for x in oflat]
        assert [(kinds[k], c) for k, c in structure] == ostructure
        blob = transfer.encode_structure(structure)
        assert blob == orc.encode_argument_structure(ostructure)
        assert transfer.decode_structure(blob + b"AXTB")[0] == structure
        back, oback = pkg.regroup(structure, flat), orc.regroup_arguments(ostructure, oflat)
        same = lambda a, b: (a is b) if isinstance(a, np.ndarray) else (len(a) == len(b) and all(map(same, a, b)))
        assert same(back, oback) and same(back, [list(a) if isinstance(a, tuple) else a for a in args])
    here = os.path.dirname(os.path.abspath(__file__))
    for c in json.load(open(os.path.join(here, "golden", "argument_structure_v1.json"))):
        class Named(str):
            __dlpack__ = None                        # stands in for a tensor
        def named(x):
            return Named(x) if isinstance(x, str) else [named(y) for y in x]
        flat, structure = pkg.flatten_arguments(named(c["args"]))
        assert [str(x) for x in flat] == c["flat"]
        assert transfer.encode_structure(structure).hex() == c["blob_hex"]


@pytest.mark.gpu
def test_send_and_receive_nested_arguments(pkg, gpu):
    """invoke(a, [b, c], [[d], [], [e, f]]) travels as ONE packed payload and comes back
    with the same nesting, with and without a memory policy."""
    import torch
    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    g = torch.Generator(device="cpu").manual_seed(5)
    t = [torch.randn(n, generator=g).to(gpu) for n in (3000, 17, 4096, 1, 999, 70000)]
    t[2] = t[2].reshape(64, 64).t()                                   # a strided one in the middle
    args = [t[0], [t[1], t[2]], [[t[3]], [], [t[4], t[5]]]]
    for use_policy in (False, True):
        outs = {}

        def policy(metas):
            outs["tensors"] = [torch.zeros(m.shape, dtype=torch.float32, device=gpu) for m in metas]
            return outs["tensors"]

        req, bundle = pkg.send_arguments(client, conn, args)
        got = pkg.recv_arguments(server, memory_policy=policy if use_policy else None,
                                 from_dlpack_fn=None if use_policy else torch.from_dlpack)
        assert client.test(req)
        torch.cuda.synchronize()
        assert len(got) == 3 and len(got[1]) == 2 and [len(x) for x in got[2]] == [1, 0, 2]
        flat = [got[0], *got[1], *[x for inner in got[2] for x in inner]]
        for a, b in zip(flat, t):
            assert tuple(a.shape) == tuple(b.shape)
            assert torch.equal(a.reshape(-1).view(torch.uint8).cpu(), b.contiguous().reshape(-1).view(torch.uint8).cpu())
        if use_policy:
            assert all(x is y for x, y in zip(flat, outs["tensors"]))     # the policy's own objects
        del got, flat
        bundle.plan.close()
        bundle.payload.release()
    assert pkg.recv_arguments(server) is None
    # a plain send_tensors message reads as one list argument
    req, bundle = pkg.send_tensors(client, conn, t[:2])
    got = pkg.recv_arguments(server, from_dlpack_fn=torch.from_dlpack)
    assert len(got) == 1 and len(got[0]) == 2 and torch.equal(got[0][1], t[1])
    client.close()
    server.close()


@pytest.mark.gpu
def test_memory_policy_with_tracked_numpy_arrays(pkg, gpu):
    """The reference's memory-policy test (axon/python/tests/test_server_memory_policy.py:
    9-66, test_invoke_memory_policy.py:9-40): the policy gets a list of metas, allocates an
    ndarray subclass per meta from `tuple(meta.shape)`, returns the object itself for one
    meta and a list otherwise; the handler must see those very objects, filled."""
    import torch

    class TrackedArray(np.ndarray):
        pass
    created = {}

    def custom_policy(meta_list):
        assert isinstance(meta_list, list) and len(meta_list) > 0
        results = []
        for meta in meta_list:
            assert meta.dtype.bits == 32 and meta.dtype.code == 2 and meta.device.device_type == 10
            arr = np.zeros(tuple(meta.shape), dtype=np.float32).view(TrackedArray)
            created[id(arr)] = True
            results.append(arr)
        return results[0] if len(results) == 1 else results

    client, server = pkg.LoopbackAmContext("client"), pkg.LoopbackAmContext("server")
    conn = client.connect(server)
    for tensors in ([torch.ones(1024, 1024, device=gpu)],                      # 4 MiB: rendezvous
                    [torch.ones(300, device=gpu), torch.full((7, 9), 1.0, device=gpu)]):
        created.clear()
        req, bundle = pkg.send_tensors(client, conn, tensors)
        got = pkg.recv_tensors(server, memory_policy=custom_policy)
        assert client.test(req)
        assert len(got) == len(tensors)
        for arr, t in zip(got, tensors):
            assert isinstance(arr, TrackedArray) and id(arr) in created
            assert arr.shape == tuple(t.shape) and np.allclose(arr, 1.0)
        bundle.plan.close()
        bundle.payload.release()
    client.close()
    server.close()


@pytest.mark.gpu
def test_the_pytorch_rocm_example_runs(gpu):
    """examples/pytorch_rocm_example.py: the reference's torch example (custom memory policy,
    a + b) and its divide-by-two round trip known answer, on the GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "examples", "pytorch_rocm_example.py")],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "pytorch_rocm_example ok" in out.stdout and "all elements == 3.0" in out.stdout


@pytest.mark.gpu
def test_the_pytorch_host_example_runs(gpu):
    """examples/pytorch_host_example.py: the reference's host torch example (handler without a
    policy, rendezvous reply into the caller's policy, eager reply past it)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "examples", "pytorch_host_example.py")],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "pytorch_host_example ok" in out.stdout and "FAILED" not in out.stdout
