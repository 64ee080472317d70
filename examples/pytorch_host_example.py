#!/usr/bin/env python3
"""Host PyTorch tensors through the tensor-bundle path: the counterpart of the reference's
``axon/python/examples/pytorch_example.py`` (:10-35 the memory policy, :46-148 the two calls),
with the same calls and the same two cases:

1. two large host tensors (rendezvous): the handler, registered WITHOUT a memory policy, gets
   host tensors converted by ``torch.from_dlpack``; the reply lands in the tensor the caller's
   memory policy created, and that very object is what ``invoke`` returns;
2. two small host tensors (eager): the reply bypasses the memory policy and is converted by
   ``from_dlpack_fn``.

The tensors still travel as ONE packed payload in device memory (gathered from and scattered to
host memory by the library's staging copies), so a GPU is needed.

Run:  python examples/pytorch_host_example.py
"""
import asyncio
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402

import __graft_entry__ as entry  # noqa: E402

axon_rocm = entry.load_package()     # the package directory's name is no Python identifier

created_objects = {}


def custom_torch_policy(meta_list):
    assert isinstance(meta_list, list) and len(meta_list) > 0
    created_objects.clear()
    results = []
    for meta in meta_list:
        tensor = torch.zeros(tuple(meta.shape), dtype=torch.float32)     # host memory
        created_objects[id(tensor)] = tensor
        results.append(tensor)
    return results[0] if len(results) == 1 else results


seen_by_the_server = []


async def tensor_op_func(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    seen_by_the_server.append((type(a).__name__, a.device.type, b.device.type))
    return a + b


async def main() -> int:
    server = axon_rocm.AxonRuntime("torch_worker")
    server.start()
    server.register_function(tensor_op_func, function_name="tensor_op", from_dlpack_fn=torch.from_dlpack)
    client = axon_rocm.AxonRuntime("client_worker")
    client.start_client()
    failures = 0
    try:
        await client.connect_endpoint_async(server.get_local_address(), "torch_worker")
        call = dict(worker_name="torch_worker", session_id=0, function="tensor_op",
                    memory_policy=custom_torch_policy, from_dlpack_fn=torch.from_dlpack)
        a = torch.ones((1024, 1024), dtype=torch.float32)
        b = torch.ones((1024, 1024), dtype=torch.float32) * 2
        result_rndv = await client.invoke(a, b, **call)
        checks = [
            ("the handler got host torch tensors", seen_by_the_server == [("Tensor", "cpu", "cpu")]),
            ("rendezvous reply is the policy's own tensor", isinstance(result_rndv, torch.Tensor)
             and id(result_rndv) in created_objects),
            ("rendezvous data", torch.equal(result_rndv, a + b)),
        ]
        small_a = torch.ones((10, 10), dtype=torch.float32)
        small_b = torch.ones((10, 10), dtype=torch.float32) * 2
        created_objects.clear()
        result_eager = await client.invoke(small_a, small_b, **call)
        checks += [
            ("eager reply was not created by the policy", isinstance(result_eager, torch.Tensor)
             and id(result_eager) not in created_objects and not created_objects),
            ("eager reply is a host tensor", result_eager.device.type == "cpu"),
            ("eager data", torch.equal(result_eager, small_a + small_b)),
        ]
        for what, ok in checks:
            print(("SUCCESS: " if ok else "FAILED: ") + what)
            failures += 0 if ok else 1
    finally:
        client.stop()
        server.stop()
    if failures == 0:
        print("pytorch_host_example ok")
    return failures


if __name__ == "__main__":
    sys.exit(asyncio.run(main()))
