#!/usr/bin/env python3
"""PyTorch tensors on an AMD GPU through the tensor-bundle path: the ROCm counterpart of the
reference's ``axon/python/examples/pytorch_cuda_example.py`` (:9-34 the custom memory policy,
:58-99 the round trip).

The reference example starts an ``AxonRuntime`` on ``axon.cuda()``, registers a handler and
invokes it with two device tensors and a custom memory policy.  The RPC runtime is not part
of this package; what is, is everything the tensors pass through on the way: the ``rocm()``
device, the packing of the argument list into one contiguous payload, the active-message
send and receive (an in-process loopback pair stands in for two workers), the receiver's
memory policy, the scatter into the policy's own tensors, and the reply.  Two calls:

1. ``tensor_op_func(a, b) -> a + b`` with a custom memory policy, as in the reference
   example; the handler must be given the very tensor objects the policy created.
2. the reference's device round trip known answer: send float(i % 256), the server divides
   by two on the device, the client expects (i % 256) / 2 exactly
   (ucx_context/ucx_am_context/ucx_am_context_test.cpp:321-333, 1893-1944).

Run:  python examples/pytorch_rocm_example.py
"""
import ctypes as C
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


def tensor_op_func(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    print(f"Server received tensors: type(a)={type(a).__name__}, device(a)={a.device}")
    return a + b


def divide_by_two_func(x: torch.Tensor) -> torch.Tensor:
    lib = axon_rocm._capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    axon_rocm._capi.check(lib.axr_divide_by_two(x.data_ptr(), x.numel(), stream))   # in place, on the device
    return x


def serve_one(server, to_client, handler):
    """What the server loop does with one request: receive the arguments through the memory
    policy, run the handler, send the result back."""
    args = axon_rocm.recv_arguments(server, memory_policy=custom_torch_policy)
    assert args is not None, "no request queued"
    for tensor in args:
        assert id(tensor) in created_objects, "the handler must get the policy's own tensors"
    result = handler(*args)
    request, bundle = axon_rocm.send_arguments(server, to_client, [result])
    return request, bundle


def invoke(client, server, to_server, to_client, handler, *tensors):
    request, sent = axon_rocm.send_arguments(client, to_server, list(tensors))
    reply_request, reply = serve_one(server, to_client, handler)
    assert client.test(request), "the request's payload has been fetched"
    sent.close()
    results = axon_rocm.recv_arguments(client, memory_policy=custom_torch_policy)
    assert server.test(reply_request)
    reply.close()
    return results[0]


def main():
    if not torch.cuda.is_available():
        print("No GPU is visible. Skipping example.")
        return 0
    device = axon_rocm.rocm(0)
    print(f"Using {device!r} ({torch.cuda.get_device_name(0)}), type {device.get_type_string()}")
    with device.activate():
        _ = torch.zeros(1, device="cuda")        # the framework's GPU context
        server = axon_rocm.LoopbackAmContext("torch_worker")
        client = axon_rocm.LoopbackAmContext("client_worker")
        to_server, to_client = client.connect(server), server.connect(client)

        a = torch.ones((1024, 1024), dtype=torch.float32, device="cuda")
        b = torch.ones((1024, 1024), dtype=torch.float32, device="cuda") * 2
        print("Invoking tensor_op_func with two 4 MiB tensors (rendezvous path, custom memory policy)...")
        result = invoke(client, server, to_server, to_client, tensor_op_func, a, b)
        assert isinstance(result, torch.Tensor) and result.is_cuda
        assert id(result) in created_objects, "the client's result is the policy's own tensor"
        assert torch.equal(result, torch.full((1024, 1024), 3.0, device="cuda"))
        print(f"Result received: device={result.device}, all elements == 3.0")

        for count in (32, 1 << 20):
            x = (torch.arange(count, device="cuda") % 256).to(torch.float32)
            halved = invoke(client, server, to_server, to_client, divide_by_two_func, x)
            expect = (torch.arange(count, device="cuda") % 256).to(torch.float32) / 2
            assert torch.equal(halved, expect), "the device round trip must be bit-exact"
            print(f"Round trip of {count} floats through divide_by_two: exact")
        pool = axon_rocm.DevicePool.default().stats()
        assert pool["live_blocks"] == 0, "every payload block went back to the pool"
        client.close()
        server.close()
    print("pytorch_rocm_example ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
