"""The AxonRuntime-shaped entry over the tensor-bundle path, written after the reference's own
Python tests: axon/python/tests/test_invoke_memory_policy.py:49-107 (a reply lands in the
objects the caller's memory policy created), test_server_memory_policy.py (the same on the
serving side), test_numpy_rpc.py:255-298 (argument classification: a tuple of tensors,
``[[], [t]]``, ``[]``), and axon/python/examples/pytorch_cuda_example.py:36-99.
"""
import asyncio

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

created_objects = {}


class TrackedArray(np.ndarray):
    pass


def tracked_policy(meta_list):
    assert isinstance(meta_list, list) and len(meta_list) > 0
    created_objects.clear()
    results = []
    for meta in meta_list:
        arr = np.zeros(tuple(meta.shape), dtype=np.float32).view(TrackedArray)
        created_objects[id(arr)] = True
        results.append(arr)
    return results[0] if len(results) == 1 else results


def run(coro):
    return asyncio.run(coro)


def pair(pkg, server_name, client_name, **kw):
    server = pkg.AxonRuntime(server_name, **kw)
    server.start()
    client = pkg.AxonRuntime(client_name, **kw)
    client.start_client()
    return server, client


def test_invoke_memory_policy_rndv(pkg, gpu):
    async def return_large_tensor() -> np.ndarray:
        return np.ones((1024, 1024), dtype=np.float32)

    async def body():
        server, client = pair(pkg, "test_server_invoke_mem", "test_client_invoke_mem")
        try:
            server.register_function(return_large_tensor, 0, function_name="return_large_tensor")
            await client.connect_endpoint_async(server.get_local_address(), "test_server_invoke_mem")
            result = await client.invoke(worker_name="test_server_invoke_mem", session_id=0, function=0,
                                         memory_policy=tracked_policy, from_dlpack_fn=np.from_dlpack)
            assert isinstance(result, TrackedArray)
            assert id(result) in created_objects
            assert np.array_equal(result, np.ones((1024, 1024), dtype=np.float32))
            # by name as well
            again = await client.invoke(worker_name="test_server_invoke_mem", session_id=0,
                                        function="return_large_tensor", memory_policy=tracked_policy)
            assert isinstance(again, TrackedArray) and float(again.sum()) == 1024 * 1024
        finally:
            client.stop()
            server.stop()
    run(body())
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_torch_tensors_through_policies_on_both_sides(pkg, gpu):
    import torch
    made = {}

    def torch_policy(meta_list):
        out = []
        for meta in meta_list:
            assert meta.device.device_type == 10            # kDLROCM
            t = torch.zeros(tuple(meta.shape), dtype=torch.float32, device=gpu)
            made[id(t)] = t
            out.append(t)
        return out[0] if len(out) == 1 else out

    seen = []

    async def tensor_op_func(a, b):
        seen.append((id(a) in made, id(b) in made, a.device.type))
        return a + b

    def halve(x):                                            # a plain function, in place on the device
        lib = pkg._capi.load()
        pkg._capi.check(lib.axr_divide_by_two(x.data_ptr(), x.numel(), torch.cuda.current_stream().cuda_stream))
        return x

    async def body():
        server, client = pair(pkg, "torch_worker", "client_worker", device=pkg.rocm(0), timeout=3000)
        try:
            server.register_function(tensor_op_func, from_dlpack_fn=torch.from_dlpack, memory_policy=torch_policy)
            server.register_function(halve, memory_policy=torch_policy)
            await client.connect_endpoint_async(server.get_local_address(), "torch_worker")
            a = torch.ones((1024, 1024), dtype=torch.float32, device=gpu)
            b = torch.ones((1024, 1024), dtype=torch.float32, device=gpu) * 2
            result = await client.invoke(a, b, worker_name="torch_worker", session_id=0, function="tensor_op_func",
                                         memory_policy=torch_policy, from_dlpack_fn=torch.from_dlpack)
            assert seen == [(True, True, "cuda")]
            assert id(result) in made and result.is_cuda
            assert torch.equal(result, torch.full((1024, 1024), 3.0, device=gpu))
            # the reference's device round trip: float(i % 256) -> divide by two -> (i % 256) / 2
            # (ucx_context/ucx_am_context/ucx_am_context_test.cpp:321-333)
            x = (torch.arange(1 << 20, device=gpu) % 256).to(torch.float32)
            got = await client.invoke(x, worker_name="torch_worker", session_id=0, function="halve",
                                      memory_policy=torch_policy)
            assert torch.equal(got, (torch.arange(1 << 20, device=gpu) % 256).to(torch.float32) / 2)
        finally:
            client.stop()
            server.stop()
    run(body())
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_argument_classification_cases(pkg, gpu):
    import torch
    shapes = []

    async def dummy_rpc(tensors):
        shapes.append([len(g) if isinstance(g, list) else -1 for g in tensors] if tensors and
                      isinstance(tensors[0], list) else len(tensors))
        return True

    def mixed(scale, xs, name, flag=None):
        assert name == "w" and flag is None and isinstance(scale, float)
        return [x * scale for x in xs], len(xs)

    async def body():
        server, client = pair(pkg, "test_classify_server", "test_classify_client")
        try:
            server.register_function(dummy_rpc, 99, from_dlpack_fn=torch.from_dlpack)
            server.register_function(mixed, from_dlpack_fn=torch.from_dlpack)
            await client.connect_endpoint_async(server.get_local_address(), "test_classify_server")
            tensor = torch.ones((10,), dtype=torch.float32, device=gpu)
            kw = dict(worker_name="test_classify_server", session_id=0, function=99)
            assert await client.invoke((tensor, tensor), **kw) is True
            assert await client.invoke([[], [tensor]], **kw) is True
            assert await client.invoke([], **kw) is True
            assert shapes == [2, [0, 1], 0]
            # plain values next to tensors, a tuple result with a list of tensors in it; the small
            # payload travels eagerly and is converted by from_dlpack_fn
            xs = [torch.arange(8, dtype=torch.float32, device=gpu), torch.ones(3, dtype=torch.float32, device=gpu)]
            out, n = await client.invoke(0.5, xs, "w", None, worker_name="test_classify_server", session_id=1,
                                         function="mixed", workflow_id=7, from_dlpack_fn=torch.from_dlpack)
            assert n == 2 and torch.equal(out[0], xs[0] * 0.5) and torch.equal(out[1], xs[1] * 0.5)
        finally:
            client.stop()
            server.stop()
    run(body())
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_failures_reach_the_caller_as_runtime_errors(pkg, gpu):
    import torch

    def broken(x):
        raise ValueError("handler said no")

    def bad_policy(metas):
        return []                                            # wrong count for one tensor

    async def body():
        server, client = pair(pkg, "err_server", "err_client")
        try:
            server.register_function(broken, 5)
            server.register_function(lambda x: x, 6, function_name="echo", memory_policy=bad_policy)
            with pytest.raises(RuntimeError, match="already registered"):
                server.register_function(broken, 5, function_name="other")
            with pytest.raises(RuntimeError, match="already registered"):
                server.register_function(broken, 8)
            with pytest.raises(RuntimeError, match="not connected"):
                await client.invoke(worker_name="err_server", session_id=0, function=5)
            with pytest.raises(RuntimeError, match="no worker at this address"):
                await client.connect_endpoint_async(b"somewhere else", "err_server")
            await client.connect_endpoint_async(server.get_local_address(), "err_server")
            big = torch.ones(1 << 20, dtype=torch.float32, device=gpu)      # rendezvous
            with pytest.raises(RuntimeError, match="ValueError: handler said no"):
                await client.invoke(big, worker_name="err_server", session_id=0, function=5)
            with pytest.raises(RuntimeError, match="not registered"):
                await client.invoke(big, worker_name="err_server", session_id=0, function="nobody")
            with pytest.raises(RuntimeError, match="incompatible buffer type"):
                await client.invoke(big, worker_name="err_server", session_id=0, function="echo")
            with pytest.raises(TypeError):
                await client.invoke({"a": 1}, worker_name="err_server", session_id=0, function=5)
            # and the pair still works afterwards
            server.register_function(lambda x: x, 7, function_name="echo2")
            back = await client.invoke(big, worker_name="err_server", session_id=0, function=7,
                                       from_dlpack_fn=torch.from_dlpack)
            assert torch.equal(back, big)
            del back
        finally:
            client.stop()
            server.stop()
    run(body())
    import gc
    gc.collect()
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_a_call_cancelled_inside_its_handler_gives_its_memory_back(pkg, gpu):
    """The caller gives up (asyncio.wait_for) while the handler is suspended: the request's
    payload block returns to the pool and the pair serves the next call."""
    import torch

    async def never(x):
        await asyncio.sleep(3600)
        return x

    async def body():
        server, client = pair(pkg, "cancel_server", "cancel_client")
        try:
            server.register_function(never, 1)
            server.register_function(lambda x: x * 2, 2, function_name="twice",
                                     from_dlpack_fn=torch.from_dlpack)
            await client.connect_endpoint_async(server.get_local_address(), "cancel_server")
            big = torch.arange(1 << 20, dtype=torch.float32, device=gpu)     # rendezvous
            with pytest.raises(asyncio.TimeoutError):
                await asyncio.wait_for(
                    client.invoke(big, worker_name="cancel_server", session_id=0, function=1), 0.05)
            out = await client.invoke(big, worker_name="cancel_server", session_id=0, function="twice",
                                      from_dlpack_fn=torch.from_dlpack)
            assert torch.equal(out, big * 2)
            del out
        finally:
            client.stop()
            server.stop()
    run(body())
    import gc
    gc.collect()
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0
