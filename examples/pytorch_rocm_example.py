#!/usr/bin/env python3
"""PyTorch tensors on an AMD GPU through the tensor-bundle path: the ROCm counterpart of the
reference's ``axon/python/examples/pytorch_cuda_example.py`` (:9-34 the custom memory policy,
:36-99 the round trip), with the same calls: two ``AxonRuntime`` objects on ``rocm()``, a
registered handler, ``connect_endpoint_async`` and ``invoke`` with a custom memory policy.

The runtime here is the in-process one of this package (no RPC control plane, no network: the
two runtimes are loopback peers inside this process); everything the tensors pass through is
the real path: the packing of the argument list into one contiguous payload, the
active-message send and receive, the receiver's memory policy, the scatter into the policy's
own tensors, and the reply.  Two calls:

1. ``tensor_op_func(a, b) -> a + b`` with a custom memory policy, as in the reference
   example; the handler must be given the very tensor objects the policy created.
2. the reference's device round trip known answer: send float(i % 256), the server divides
   by two on the device, the client expects (i % 256) / 2 exactly
   (ucx_context/ucx_am_context/ucx_am_context_test.cpp:321-333, 1893-1944).

Run:  python examples/pytorch_rocm_example.py
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

# objects created by the policy, to verify that the handler gets these and no copies
created_objects = {}


def custom_torch_policy(meta_list):
    """A list of TensorMeta in, one torch tensor on the GPU per meta out (a single tensor for a
    single meta), as in the reference example."""
    assert isinstance(meta_list, list) and len(meta_list) > 0
    created_objects.clear()
    results = []
    for meta in meta_list:
        assert meta.device.device_type == 10          # kDLROCM: the sender's tensors were on the GPU
        tensor = torch.zeros(tuple(meta.shape), dtype=torch.float32, device="cuda")
        created_objects[id(tensor)] = tensor
        results.append(tensor)
    return results[0] if len(results) == 1 else results


async def tensor_op_func(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    print(f"Server received tensors: type(a)={type(a).__name__}, device(a)={a.device}")
    for tensor in (a, b):
        assert id(tensor) in created_objects, "the handler must get the policy's own tensors"
    return a + b


def divide_by_two_func(x: torch.Tensor) -> torch.Tensor:
    lib = axon_rocm._capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    axon_rocm._capi.check(lib.axr_divide_by_two(x.data_ptr(), x.numel(), stream))   # in place, on the device
    return x


async def main():
    if not torch.cuda.is_available():
        print("No GPU is visible. Skipping example.")
        return 0
    _ = torch.zeros(1, device="cuda")            # the framework's GPU context
    device = axon_rocm.rocm(0)
    print(f"Using {device!r} ({torch.cuda.get_device_name(0)}), type {device.get_type_string()}")

    # 1. server on the ROCm device, handlers registered with the custom memory policy
    server = axon_rocm.AxonRuntime("torch_worker", device=axon_rocm.rocm(), timeout=3000)
    server.start()
    server.register_function(tensor_op_func, from_dlpack_fn=torch.from_dlpack, memory_policy=custom_torch_policy)
    server.register_function(divide_by_two_func, from_dlpack_fn=torch.from_dlpack, memory_policy=custom_torch_policy)
    server_addr = server.get_local_address()

    # 2. client, connected to the server's address
    client = axon_rocm.AxonRuntime("client_worker", device=axon_rocm.rocm(), timeout=3000)
    client.start_client()
    await client.connect_endpoint_async(server_addr, "torch_worker")

    # 3. two 4 MiB tensors: the rendezvous path, so the memory policy is used on both sides
    a = torch.ones((1024, 1024), dtype=torch.float32, device="cuda")
    b = torch.ones((1024, 1024), dtype=torch.float32, device="cuda") * 2
    print("Invoking tensor_op_func with two 4 MiB tensors (rendezvous path, custom memory policy)...")
    result = await client.invoke(a, b, worker_name="torch_worker", session_id=0, function="tensor_op_func",
                                 memory_policy=custom_torch_policy, from_dlpack_fn=torch.from_dlpack)
    assert isinstance(result, torch.Tensor) and result.is_cuda
    assert id(result) in created_objects, "the client's result is the policy's own tensor"
    assert torch.equal(result, torch.full((1024, 1024), 3.0, device="cuda"))
    print(f"Result received: device={result.device}, all elements == 3.0")

    # 4. the device round trip of the reference's context test; 32 floats travel eagerly (the
    #    policy is bypassed, from_dlpack_fn converts), 2^20 floats by rendezvous
    for count in (32, 1 << 20):
        x = (torch.arange(count, device="cuda") % 256).to(torch.float32)
        halved = await client.invoke(x, worker_name="torch_worker", session_id=0, function="divide_by_two_func",
                                     memory_policy=custom_torch_policy, from_dlpack_fn=torch.from_dlpack)
        expect = (torch.arange(count, device="cuda") % 256).to(torch.float32) / 2
        assert torch.equal(halved, expect), "the device round trip must be bit-exact"
        print(f"Round trip of {count} floats through divide_by_two: exact")
        del halved
    client.stop()
    server.stop()
    pool = axon_rocm.DevicePool.default().stats()
    assert pool["live_blocks"] == 0, "every payload block went back to the pool"
    print("pytorch_rocm_example ok")
    return 0


if __name__ == "__main__":
    sys.exit(asyncio.run(main()))
