// Self-test of the C++ host layer (memory manager, device context, bundle
// helpers) over the C ABI.  Needs a GPU; `--no-device` checks the failure
// behaviour on a machine without one.  Prints "host_selftest ok" and exits 0.
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <numeric>
#include <thread>
#include <vector>

#include "axon_tensor_bundle.hpp"
#include "ucx_rocm_context.hpp"
#include "ucx_rocm_memory_manager.hpp"

using eux::ucxx::UcxAutoRocmDeviceContext;
using eux::ucxx::UcxRocmMemoryResourceManager;
namespace bundle = eux::axon::rocm;

#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                         \
    }                                                                       \
  } while (0)

static axr_tensor_t Tensor1D(void* data, int64_t* shape, int32_t device_type, uint8_t code, uint8_t bits) {
  axr_tensor_t t;
  std::memset(&t, 0, sizeof(t));
  t.data = data;
  t.device_type = device_type;
  t.ndim = 1;
  t.dtype_code = code;
  t.dtype_bits = bits;
  t.dtype_lanes = 1;
  t.shape = shape;
  return t;
}

static int RunNoDevice() {
  bool threw = false;
  try {
    UcxRocmMemoryResourceManager mr(0);
  } catch (const std::runtime_error& e) {
    threw = true;
    std::printf("expected failure without a device: %s\n", e.what());
  }
  EXPECT(threw);
  std::printf("host_selftest ok (no device)\n");
  return 0;
}

int main(int argc, char** argv) {
  if (argc > 1 && std::strcmp(argv[1], "--no-device") == 0) return RunNoDevice();
  int count = 0;
  EXPECT(axr_device_count(&count) == AXR_OK);
  if (count == 0) {
    std::fprintf(stderr, "no ROCm device\n");
    return 2;
  }

  // device context: RAII activation, nested, cloned, from another thread
  UcxAutoRocmDeviceContext ctx(0);
  {
    auto op = ctx(nullptr, nullptr);
    int cur = -1;
    EXPECT(axr_device_get(&cur) == AXR_OK && cur == 0);
    auto cloned = ctx.clone();
    std::thread t([&] {
      auto op2 = (*cloned)(nullptr, nullptr);
      int c2 = -1;
      EXPECT(axr_device_get(&c2) == AXR_OK && c2 == 0);
    });
    t.join();
    op->deactivate();
    op->deactivate();   // idempotent
  }

  // memory manager with a registrar: one registration per slab, handle travels
  int registrations = 0, unregistrations = 0;
  {
    UcxRocmMemoryResourceManager mr(0, 8u << 20);
    mr.set_registrar(
        [&](void*, size_t) { return reinterpret_cast<void*>(static_cast<uintptr_t>(0x1000 + ++registrations)); },
        [&](void*) { ++unregistrations; });

    // send -> process -> reply KAT (ucx_am_context_test.cpp:321-333, 1893-1944):
    // float(i % 256) to the device, halve there, expect float(i % 256) / 2 back
    const size_t n = 1u << 20;
    std::vector<float> host(n), back(n);
    for (size_t i = 0; i < n; ++i) host[i] = static_cast<float>(i % 256);
    void* dev = mr.allocate(ucx_memory_type::ROCM, n * sizeof(float));
    mr.memcpy(ucx_memory_type::ROCM, dev, ucx_memory_type::HOST, host.data(), n * sizeof(float));
    EXPECT(axr_divide_by_two(static_cast<float*>(dev), n, nullptr) == AXR_OK);
    EXPECT(axr_device_synchronize() == AXR_OK);
    mr.memcpy(ucx_memory_type::HOST, back.data(), ucx_memory_type::ROCM, dev, n * sizeof(float));
    for (size_t i = 0; i < n; ++i) EXPECT(back[i] == static_cast<float>(i % 256) / 2);
    mr.deallocate(ucx_memory_type::ROCM, dev, n * sizeof(float));
    EXPECT(registrations == 1);

    // iov -> contiguous KAT (ucx_am_connection_test.cpp:1051-1108): three device
    // segments filled with the running pattern, packed tight, equal the flat pattern
    const size_t lens[3] = {512 * 1024, 256 * 1024, 800 * 1024};
    std::vector<void*> segs(3);
    std::vector<int64_t> shapes(3);
    std::vector<axr_tensor_t> tensors(3);
    size_t cursor = 0;
    for (int s = 0; s < 3; ++s) {
      std::vector<uint8_t> fill(lens[s]);
      for (size_t i = 0; i < lens[s]; ++i, ++cursor) fill[i] = static_cast<uint8_t>(cursor % 256);
      segs[s] = mr.allocate(ucx_memory_type::ROCM, lens[s]);
      mr.memcpy(ucx_memory_type::ROCM, segs[s], ucx_memory_type::HOST, fill.data(), lens[s]);
      shapes[s] = static_cast<int64_t>(lens[s]);
      tensors[s] = Tensor1D(segs[s], &shapes[s], 10, 1, 8);
    }
    bundle::TensorBundle packed = bundle::PackTensors(mr, tensors.data(), 3, 1, nullptr);
    EXPECT(axr_device_synchronize() == AXR_OK);
    ucx_am_data_t am = packed.as_am_data();
    EXPECT(am.buffer.size == cursor && am.buffer_type == ucx_memory_type::ROCM);
    EXPECT(am.mem_h == reinterpret_cast<void*>(static_cast<uintptr_t>(0x1001)) || registrations == 2);
    std::vector<uint8_t> flat(cursor);
    mr.memcpy(ucx_memory_type::HOST, flat.data(), ucx_memory_type::ROCM, am.buffer.data, cursor);
    for (size_t i = 0; i < cursor; ++i) EXPECT(flat[i] == static_cast<uint8_t>(i % 256));

    // receiver: size from the header, zero-copy split, then scatter into fresh buffers
    EXPECT(bundle::PayloadBytes(am.header.data, am.header.size) == cursor);
    auto views = bundle::SplitPayload(am.header.data, am.header.size, am.buffer.data, am.buffer.size);
    EXPECT(views.size() == 3 && views[0].data == am.buffer.data && views[1].size == lens[1]);
    EXPECT(views[2].data == static_cast<char*>(am.buffer.data) + lens[0] + lens[1]);
    bool length_error = false;
    try {
      bundle::SplitPayload(am.header.data, am.header.size, am.buffer.data, am.buffer.size - 1);
    } catch (const std::length_error&) {
      length_error = true;
    }
    EXPECT(length_error);
    std::vector<void*> outs(3);
    std::vector<axr_tensor_t> dst(3);
    for (int s = 0; s < 3; ++s) {
      outs[s] = mr.allocate(ucx_memory_type::ROCM, lens[s]);
      dst[s] = Tensor1D(outs[s], &shapes[s], 10, 1, 8);
    }
    {
      bundle::BundlePlan rplan = bundle::UnpackTensors(am.header.data, am.header.size, am.buffer.data,
                                                       am.buffer.size, dst.data(), 3, nullptr);
    }   // plan destructor drains the stream
    size_t at = 0;
    for (int s = 0; s < 3; ++s) {
      std::vector<uint8_t> got(lens[s]);
      mr.memcpy(ucx_memory_type::HOST, got.data(), ucx_memory_type::ROCM, outs[s], lens[s]);
      for (size_t i = 0; i < lens[s]; ++i, ++at) EXPECT(got[i] == static_cast<uint8_t>(at % 256));
      mr.deallocate(ucx_memory_type::ROCM, outs[s], lens[s]);
      mr.deallocate(ucx_memory_type::ROCM, segs[s], lens[s]);
    }
    // checkpoint path: the payload as one host vector per tensor
    {
      auto vecs = bundle::PayloadToHost(am.header.data, am.header.size, am.buffer.data, am.buffer.size,
                                        nullptr);
      EXPECT(vecs.size() == 3);
      size_t k = 0;
      for (int s = 0; s < 3; ++s) {
        EXPECT(vecs[s].size() == lens[s]);
        for (size_t i = 0; i < lens[s]; ++i, ++k) EXPECT(vecs[s][i] == static_cast<uint8_t>(k % 256));
      }
    }
    packed.release();
    packed.release();   // idempotent, like a moved-from UcxBuffer
    EXPECT(mr.stats().live_blocks == 0);

    // ownership (the release-function rules of ucx_context_data_test.cpp:85-128):
    // a detached block is no longer released by the bundle, an owned one exactly once
    {
      std::vector<uint8_t> fill(4096, 7);
      void* seg = mr.allocate(ucx_memory_type::ROCM, fill.size());
      mr.memcpy(ucx_memory_type::ROCM, seg, ucx_memory_type::HOST, fill.data(), fill.size());
      int64_t shape = static_cast<int64_t>(fill.size());
      axr_tensor_t one = Tensor1D(seg, &shape, 10, 1, 8);
      void* kept = nullptr;
      size_t kept_bytes = 0;
      {
        bundle::TensorBundle b = bundle::PackTensors(mr, &one, 1, 256, nullptr);
        EXPECT(axr_device_synchronize() == AXR_OK);
        kept_bytes = b.payload_bytes();
        kept = b.detach();
      }   // destructor runs: nothing to release
      EXPECT(mr.stats().live_blocks == 2);
      {
        bundle::TensorBundle b = bundle::PackTensors(mr, &one, 1, 256, nullptr);
        bundle::TensorBundle moved = std::move(b);
        EXPECT(b.payload() == nullptr && moved.payload() != nullptr);
      }   // released once, by the moved-to object
      EXPECT(mr.stats().live_blocks == 2);
      mr.deallocate(ucx_memory_type::ROCM, kept, kept_bytes);
      mr.deallocate(ucx_memory_type::ROCM, seg, fill.size());
      EXPECT(mr.stats().live_blocks == 0);
    }

    // a payload streamed in chunks of one geometry: one pair of plans, moved over the
    // chunks by address deltas; then two independent bundles in one launch
    {
      const size_t chunk = 1u << 20, chunks = 6, parts = 4, part = chunk / parts;
      std::vector<uint8_t> pattern(chunk * chunks);
      for (size_t i = 0; i < pattern.size(); ++i) pattern[i] = static_cast<uint8_t>((i * 7 + i / 4099) % 251);
      void* src = mr.allocate(ucx_memory_type::ROCM, pattern.size());
      void* dst = mr.allocate(ucx_memory_type::ROCM, pattern.size());
      mr.memcpy(ucx_memory_type::ROCM, src, ucx_memory_type::HOST, pattern.data(), pattern.size());
      std::vector<uint8_t> zeros(pattern.size(), 0);
      mr.memcpy(ucx_memory_type::ROCM, dst, ucx_memory_type::HOST, zeros.data(), zeros.size());
      int64_t shape = static_cast<int64_t>(part);
      std::vector<axr_tensor_t> from(parts), to(parts);
      for (size_t k = 0; k < parts; ++k) {
        from[k] = Tensor1D(static_cast<uint8_t*>(src) + k * part, &shape, 10, 1, 8);
        to[k] = Tensor1D(static_cast<uint8_t*>(dst) + k * part, &shape, 10, 1, 8);
      }
      {
        bundle::BundlePlan send = bundle::BundlePlan::Create(from.data(), parts, 256);
        const std::vector<uint8_t> header = send.header();
        bundle::BundlePlan recv = bundle::BundlePlan::FromHeaderBind(header.data(), header.size(), to.data(), parts);
        bundle::StreamedTransfer transfer(mr, send.payload_bytes(), /*lanes=*/2, /*streams=*/1);
        for (size_t c = 0; c < chunks; ++c)
          transfer.Submit(send, static_cast<int64_t>(c * chunk), recv, static_cast<int64_t>(c * chunk));
        transfer.Finish();
      }
      std::vector<uint8_t> got(pattern.size());
      mr.memcpy(ucx_memory_type::HOST, got.data(), ucx_memory_type::ROCM, dst, got.size());
      EXPECT(got == pattern);

      // pack of chunk 1 and unpack of chunk 0's payload in ONE launch
      mr.memcpy(ucx_memory_type::ROCM, dst, ucx_memory_type::HOST, zeros.data(), zeros.size());
      bundle::BundlePlan send = bundle::BundlePlan::Create(from.data(), parts, 256);
      const std::vector<uint8_t> header = send.header();
      bundle::BundlePlan recv = bundle::BundlePlan::FromHeaderBind(header.data(), header.size(), to.data(), parts);
      const size_t bytes = send.payload_bytes();
      void* pay0 = mr.allocate(ucx_memory_type::ROCM, bytes);
      void* pay1 = mr.allocate(ucx_memory_type::ROCM, bytes);
      send.pack(pay0, bytes, nullptr);
      EXPECT(axr_device_synchronize() == AXR_OK);
      bundle::SubmitBundles({bundle::PackJob(send, pay1, bytes, static_cast<int64_t>(chunk)),
                             bundle::UnpackJob(recv, pay0, bytes, 0)}, nullptr);
      bundle::SubmitBundles({bundle::UnpackJob(recv, pay1, bytes, static_cast<int64_t>(chunk))}, nullptr);
      EXPECT(axr_device_synchronize() == AXR_OK);
      mr.memcpy(ucx_memory_type::HOST, got.data(), ucx_memory_type::ROCM, dst, 2 * chunk);
      EXPECT(std::equal(got.begin(), got.begin() + 2 * chunk, pattern.begin()));
      send.reset();
      recv.reset();
      mr.deallocate(ucx_memory_type::ROCM, pay0, bytes);
      mr.deallocate(ucx_memory_type::ROCM, pay1, bytes);
      mr.deallocate(ucx_memory_type::ROCM, src, pattern.size());
      mr.deallocate(ucx_memory_type::ROCM, dst, pattern.size());
      EXPECT(mr.stats().live_blocks == 0);
    }

    // unsupported types throw std::runtime_error like the reference's manager
    bool threw = false;
    try {
      mr.allocate(ucx_memory_type::CUDA, 16);
    } catch (const std::runtime_error&) {
      threw = true;
    }
    EXPECT(threw);
    threw = false;
    try {
      uint8_t a[4], b[4];
      mr.memcpy(ucx_memory_type::CUDA, a, ucx_memory_type::HOST, b, 4);
    } catch (const std::runtime_error&) {
      threw = true;
    }
    EXPECT(threw);

    // pinned host memory and HOST memory through the same interface
    void* pinned = mr.allocate(ucx_memory_type::ROCM_MANAGED, 4096);
    void* plain = mr.allocate(ucx_memory_type::HOST, 4096, 64);
    std::memset(plain, 0x5a, 4096);
    mr.memcpy(ucx_memory_type::ROCM_MANAGED, pinned, ucx_memory_type::HOST, plain, 4096);
    EXPECT(static_cast<uint8_t*>(pinned)[4095] == 0x5a);
    mr.deallocate(ucx_memory_type::ROCM_MANAGED, pinned, 4096);
    mr.deallocate(ucx_memory_type::HOST, plain, 4096);
  }
  EXPECT(unregistrations == registrations && registrations >= 1);
  std::printf("host_selftest ok\n");
  return 0;
}
