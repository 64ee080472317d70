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
            with pytest.raises(RuntimeError, match="Unsupported type for inference"):
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


def test_numpy_arguments_and_results_like_the_reference_suite(pkg, gpu):
    """axon/python/tests/test_numpy_rpc.py:94-247 with the same functions and values: tensors in,
    an int out; a tensor out; a list of tensors out; a tuple of an int and tensors out; a tensor,
    an int and a str in; the eight-argument receive_shards call with nested tensor lists next to
    lists of str, int and bool."""
    async def sum_int_func(a, b):
        return int(np.sum(a + b))

    async def sum_arr_func(a, b, c):
        return np.array([np.sum(a + b) + np.sum(c)], dtype=np.int64)

    async def list_func(a, b):
        return [a + b, a * b]

    async def tuple_func(x, y):
        return (int(np.sum(x) + np.sum(y)), x.copy(), y.copy())

    async def mixed_args_func(a, b, c):
        return f"{np.sum(a)}_{b}_{c}"

    seen = {}

    async def receive_shards_func(op_name, names, step, sender_rank, payload_groups, counts_groups,
                                  is_ragged_flags, has_indices_flags):
        assert isinstance(op_name, str) and isinstance(names, list) and isinstance(payload_groups, list)
        seen.update(names=names, step=step, rank=sender_rank, counts=counts_groups, ragged=is_ragged_flags,
                    indices=has_indices_flags, groups=[[np.array(t) for t in g] for g in payload_groups])
        return 0

    async def body():
        server, client = pair(pkg, "test_worker", "client_worker")
        try:
            for i, fn in enumerate([sum_int_func, sum_arr_func, list_func, tuple_func, mixed_args_func,
                                    receive_shards_func]):
                server.register_function(fn, i, from_dlpack_fn=np.from_dlpack)
            await client.connect_endpoint_async(server.get_local_address(), "test_worker")
            kw = dict(worker_name="test_worker", session_id=0)
            a = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.int64)
            b = np.array([9, 10, 11, 12, 13, 14, 15, 16], dtype=np.int64)
            c = np.array([17, 18, 19, 20], dtype=np.int64)
            result = await client.invoke(a, b, function=0, **kw)
            assert isinstance(result, int) and result == 136
            result = await client.invoke(a, b, c, function=1, from_dlpack_fn=np.from_dlpack, **kw)
            assert isinstance(result, np.ndarray) and result[0] == 210
            result = await client.invoke(a, b, function=2, from_dlpack_fn=np.from_dlpack, **kw)
            assert isinstance(result, list) and len(result) == 2
            assert isinstance(result[0], np.ndarray) and isinstance(result[1], np.ndarray)
            np.testing.assert_array_equal(result[0], a + b)
            np.testing.assert_array_equal(result[1], a * b)
            x, y = np.array([1, 2, 3], dtype=np.int64), np.array([4, 5, 6], dtype=np.int64)
            result = await client.invoke(x, y, function=3, from_dlpack_fn=np.from_dlpack, **kw)
            assert isinstance(result, tuple) and len(result) == 3 and result[0] == 21
            np.testing.assert_array_equal(result[1], x)
            np.testing.assert_array_equal(result[2], y)
            result = await client.invoke(x, 100, "hello", function=4, from_dlpack_fn=np.from_dlpack, **kw)
            assert isinstance(result, str) and result == "6_100_hello"
            rng = np.random.default_rng(0)
            groups = [[rng.random((2, 2)), rng.random((3, 3))], [rng.random((4, 4))]]
            result = await client.invoke("test_op", ["tensor_1", "tensor_2"], 10, 0, groups, [[2, 2], [1]],
                                         [False, True], [True, False], function=5,
                                         from_dlpack_fn=np.from_dlpack, **kw)
            assert result == 0
            assert seen["names"] == ["tensor_1", "tensor_2"] and seen["step"] == 10 and seen["rank"] == 0
            assert seen["counts"] == [[2, 2], [1]] and seen["ragged"] == [False, True]
            assert seen["indices"] == [True, False]
            assert [len(g) for g in seen["groups"]] == [2, 1]
            for got_group, want_group in zip(seen["groups"], groups):
                for got, want in zip(got_group, want_group):
                    np.testing.assert_array_equal(got, want)
        finally:
            client.stop()
            server.stop()
    run(body())
    seen.clear()
    import gc
    gc.collect()
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_a_tensor_the_handler_keeps_outlives_the_call(pkg, gpu):
    """axon/python/tests/test_numpy_rpc.py:472-583: an input tensor stored beyond the handler
    stays valid after the call has finished, and is released once the last reference goes."""
    import gc
    import weakref
    kept = {}

    async def store_input_func(a, b):
        kept["a"] = a
        return a + b

    async def store_then_release_input_func(a):
        kept["tmp"] = a
        kept["ref"] = weakref.ref(a)
        del a
        await asyncio.sleep(0)
        total = int(np.sum(kept["tmp"]))
        kept["tmp"] = None
        return total

    def add_one_in_place(a):
        a += 1
        return a

    async def body():
        server, client = pair(pkg, "test_lifetime_server", "test_lifetime_client")
        try:
            server.register_function(store_input_func, 200, from_dlpack_fn=np.from_dlpack)
            server.register_function(store_then_release_input_func, 201, from_dlpack_fn=np.from_dlpack)
            await client.connect_endpoint_async(server.get_local_address(), "test_lifetime_server")
            kw = dict(worker_name="test_lifetime_server", session_id=0, from_dlpack_fn=np.from_dlpack)
            a = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float64)
            b = np.array([10.0, 20.0, 30.0, 40.0], dtype=np.float64)
            result = await client.invoke(a, b, function=200, **kw)
            await asyncio.sleep(0)
            gc.collect()
            np.testing.assert_array_equal(kept["a"], a)
            np.testing.assert_array_equal(result, a + b)
            # the same with a rendezvous-sized tensor (its memory is a pool block)
            big = np.arange(1 << 18, dtype=np.float64)
            result = await client.invoke(big, big, function=200, **kw)
            await asyncio.sleep(0)
            gc.collect()
            np.testing.assert_array_equal(kept["a"], big)
            np.testing.assert_array_equal(result, big + big)
            del result
            kept["a"] = None
            # a handler may change what it received in place and hand the same array back
            server.register_function(add_one_in_place, 202, from_dlpack_fn=np.from_dlpack)
            for values in (np.arange(6, dtype=np.float64), np.arange(1 << 18, dtype=np.float64)):
                echoed = await client.invoke(values, function=202, **kw)
                np.testing.assert_array_equal(echoed, values + 1)
                assert echoed.flags.writeable
                del echoed
            c = np.array([3.0, 4.0, 5.0, 6.0], dtype=np.float64)
            assert await client.invoke(c, function=201, **kw) == int(np.sum(c))
            for _ in range(10):
                if kept["ref"]() is None:
                    break
                gc.collect()
                await asyncio.sleep(0)
            assert kept["tmp"] is None and kept["ref"]() is None
        finally:
            client.stop()
            server.stop()
    run(body())
    kept.clear()
    gc.collect()
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0


def test_server_memory_policy_objects_reach_the_handler_twice(pkg, gpu):
    """axon/python/tests/test_server_memory_policy.py:14-125: the handler receives the very object
    the registered policy created, with the data in it, on a first call and on a second one."""
    async def rpc_handler(arr):
        return bool(isinstance(arr, TrackedArray) and id(arr) in created_objects and np.allclose(arr, 1.0))

    async def body():
        server, client = pair(pkg, "test_memory_policy_worker", "client_worker_memfail")
        try:
            server.register_function(rpc_handler, 0, memory_policy=tracked_policy, from_dlpack_fn=np.from_dlpack)
            await client.connect_endpoint_async(server.get_local_address(), "test_memory_policy_worker")
            large_arr = np.ones((1024, 1024), dtype=np.float32)        # 4 MB: rendezvous
            kw = dict(worker_name="test_memory_policy_worker", session_id=0, function=0)
            assert await client.invoke(large_arr, **kw) is True
            assert await client.invoke(large_arr, **kw) is True
            # a payload small enough to travel eagerly bypasses the policy (axon_worker.cpp:1150-1172)
            assert await client.invoke(np.ones(4, dtype=np.float32), **kw) is False
        finally:
            client.stop()
            server.stop()
    run(body())
    assert pkg.DevicePool.default().stats()["live_blocks"] == 0
