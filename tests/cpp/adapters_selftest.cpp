// Runs the receive-side adapters of execution-ucx_amd/host/reference_adapters.hpp against
// the reference's REAL UcxBuffer / UcxBufferVec / UcxMemoryResourceManager
// (ucx_context/ucx_context_data.hpp:58-129,641-665, ucx_context/ucx_memory_resource.hpp:99-123),
// on a GPU.  TEST INFRASTRUCTURE: built by oracle/Makefile into oracle/_ref/ with the
// execution-ucx tree on the include path and its ucx_memory_resource.cpp compiled in
// place; links the C oracle (liborc.so) as the checker.
//
//   PackTensors -> ToUcxBuffer -> ReceiveBufferFor -> mr.memcpy -> ToUcxBufferVec
//   RocmBundleReceivePolicy (the CustomMemoryPolicy of axon/include/axon/memory_policy.hpp:72-73,
//   called like axon/src/axon_worker.cpp:1150-1172 calls it)
//
// Checks: the views equal the reference's own to_buffer_vec over the same memory, the
// payload equals the oracle's pack, sizes follow the header, every pool block is back
// (live_blocks == 0) once the owning buffers are gone, and no release function runs twice.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "reference_adapters.hpp"
#include "ucx_rocm_context.hpp"
#include "ucx_rocm_memory_manager.hpp"

#ifndef AXON_ROCM_HAVE_REFERENCE_MEMORY_RESOURCE
#error "build with -DAXON_ROCM_IN_REFERENCE_TREE and the execution-ucx tree on the include path"
#endif

extern "C" {
uint64_t orc_layout(const uint64_t* sizes, size_t n, uint64_t align, uint64_t* offsets);
int orc_pack(const void* const* srcs, const uint64_t* sizes, const uint64_t* offsets, size_t n, void* dst,
             uint64_t total);
uint64_t orc_tensor_nbytes(int32_t ndim, const int64_t* shape, uint8_t bits);
}

using eux::axon::rocm::BundleBytesFor;
using eux::axon::rocm::Check;
using eux::axon::rocm::PackTensors;
using eux::axon::rocm::ReceiveBufferFor;
using eux::axon::rocm::RocmBundleReceivePolicy;
using eux::axon::rocm::ToUcxBuffer;
using eux::axon::rocm::ToUcxBufferVec;
using eux::ucxx::UcxBuffer;
using eux::ucxx::UcxBufferVec;
using eux::ucxx::UcxRocmMemoryResourceManager;

namespace {

int g_failures = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);           \
      std::fflush(stdout);                                                    \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

// A record with the fields of rpc::utils::TensorMeta (rpc_core/utils/tensor_meta.hpp:77-82);
// the real one needs cista, which this image does not have.
struct MetaLike {
  struct { int32_t device_type, device_id; } device;
  int32_t ndim;
  struct { uint8_t code, bits; uint16_t lanes; } dtype;
  uint64_t byte_offset;
  std::vector<int64_t> shape, strides;
};

struct DeviceTensors {
  UcxRocmMemoryResourceManager& mr;
  std::vector<std::vector<uint8_t>> host;     // the bytes each tensor holds
  std::vector<std::vector<int64_t>> shapes;
  std::vector<void*> device;
  std::vector<axr_tensor_t> desc;
  std::vector<MetaLike> metas;

  explicit DeviceTensors(UcxRocmMemoryResourceManager& m) : mr(m) {}
  ~DeviceTensors() {
    for (size_t i = 0; i < device.size(); ++i)
      if (device[i]) mr.deallocate(ucx_memory_type::ROCM, device[i], host[i].size());
  }
  void add(std::mt19937_64& rng, std::vector<int64_t> shape, uint8_t code, uint8_t bits) {
    shapes.push_back(std::move(shape));
    const std::vector<int64_t>& s = shapes.back();
    const uint64_t nbytes = orc_tensor_nbytes(static_cast<int32_t>(s.size()), s.data(), bits);
    std::vector<uint8_t> bytes(nbytes);
    for (auto& b : bytes) b = static_cast<uint8_t>(rng());
    void* d = nullptr;
    if (nbytes) {
      d = mr.allocate(ucx_memory_type::ROCM, nbytes, 256);
      mr.memcpy(ucx_memory_type::ROCM, d, ucx_memory_type::HOST, bytes.data(), nbytes);
    }
    host.push_back(std::move(bytes));
    device.push_back(d);
  }
  void finish(const std::vector<std::pair<uint8_t, uint8_t>>& dtypes) {
    for (size_t i = 0; i < shapes.size(); ++i) {
      axr_tensor_t t;
      std::memset(&t, 0, sizeof(t));
      t.data = device[i];
      t.device_type = 10;   // kDLROCM
      t.device_id = mr.device();
      t.ndim = static_cast<int32_t>(shapes[i].size());
      t.dtype_code = dtypes[i].first;
      t.dtype_bits = dtypes[i].second;
      t.dtype_lanes = 1;
      t.shape = shapes[i].data();
      desc.push_back(t);
      MetaLike m;
      m.device.device_type = 10;
      m.device.device_id = mr.device();
      m.ndim = t.ndim;
      m.dtype.code = t.dtype_code;
      m.dtype.bits = t.dtype_bits;
      m.dtype.lanes = 1;
      m.byte_offset = 0;
      m.shape = shapes[i];
      metas.push_back(m);
    }
  }
  std::vector<uint8_t> oracle_pack(uint64_t align) const {
    std::vector<uint64_t> sizes, offsets(host.size());
    std::vector<const void*> srcs;
    for (const auto& h : host) {
      sizes.push_back(h.size());
      srcs.push_back(h.data());
    }
    const uint64_t total = orc_layout(sizes.data(), sizes.size(), align, offsets.data());
    std::vector<uint8_t> out(total);
    if (orc_pack(srcs.data(), sizes.data(), offsets.data(), sizes.size(), out.data(), total) != 0)
      std::abort();
    return out;
  }
};

// The whole receive path with the tight layout, which the reference's to_buffer_vec
// understands; returns with every owning object destroyed.
void round_trip(UcxRocmMemoryResourceManager& mr, DeviceTensors& t) {
  const size_t n = t.desc.size();
  const std::vector<uint8_t> want = t.oracle_pack(1);
  int releases = 0;
  {
    auto bundle = PackTensors(mr, n ? t.desc.data() : nullptr, n, 1, nullptr);
    EXPECT(bundle.payload_bytes() == want.size());
    auto sent = ToUcxBuffer(std::move(bundle), mr);          // header bytes + owning UcxBuffer
    std::vector<uint8_t>& header = sent.first;
    UcxBuffer& payload = sent.second;
    EXPECT(payload.type() == ucx_memory_type::ROCM);
    EXPECT(payload.size() == want.size());
    EXPECT(payload.own_buffer());
    // the sender's bytes are the oracle's
    std::vector<uint8_t> got(want.size());
    Check(axr_device_synchronize(), "axr_device_synchronize");
    if (!got.empty())
      mr.memcpy(ucx_memory_type::HOST, got.data(), ucx_memory_type::ROCM, payload.data(), got.size());
    EXPECT(got == want);

    // receiver: one pool block sized from the header, filled by the "transport"
    UcxBuffer recv = ReceiveBufferFor(header.data(), header.size(), mr);
    EXPECT(recv.size() == want.size() && recv.data() != nullptr && recv.own_buffer());
    EXPECT(recv.data() != payload.data());
    if (recv.size())
      mr.memcpy(ucx_memory_type::ROCM, recv.data(), ucx_memory_type::ROCM, payload.data(), recv.size());
    void* const base = recv.data();

    // what the reference's own split gives over the same memory (non-owning view of it)
    std::vector<size_t> sizes;
    for (const auto& h : t.host) sizes.push_back(h.size());
    UcxBuffer alias(mr, ucx_memory_type::ROCM, base, recv.size(), nullptr, /*own_buffer=*/false);
    UcxBufferVec expected = std::move(alias).to_buffer_vec(sizes);

    UcxBufferVec views = ToUcxBufferVec(std::move(recv), header.data(), header.size());
    EXPECT(views.has_backing_buffer());                       // the pool block lives on behind the views
    EXPECT(views.type() == ucx_memory_type::ROCM);
    EXPECT(views.buffers().size() == n && expected.buffers().size() == n);
    for (size_t i = 0; i < n && i < views.buffers().size(); ++i) {
      EXPECT(views.at(i).data == expected.at(i).data);
      EXPECT(views.at(i).size == expected.at(i).size);
      // and the bytes under every view are the tensor's
      std::vector<uint8_t> back(views.at(i).size);
      if (!back.empty())
        mr.memcpy(ucx_memory_type::HOST, back.data(), ucx_memory_type::ROCM, views.at(i).data, back.size());
      EXPECT(back == t.host[i]);
    }
    // moving the sender's buffer keeps one owner; an extra release function counts its calls
    UcxBuffer moved = std::move(payload);
    EXPECT(payload.data() == nullptr && !payload.own_buffer() && moved.own_buffer());
    void* probe = mr.allocate(ucx_memory_type::ROCM, 16, 256);
    {
      UcxRocmMemoryResourceManager* pmr = &mr;
      UcxBuffer counted(mr, ucx_memory_type::ROCM, probe, 16, nullptr, true, [pmr, &releases](void* p) {
        ++releases;
        pmr->deallocate(ucx_memory_type::ROCM, p, 16);
      });
      UcxBuffer second = std::move(counted);
    }
  }
  EXPECT(releases == 1);
}

void policy(UcxRocmMemoryResourceManager& mr, const DeviceTensors& t, uint32_t align) {
  const uint64_t before = mr.stats().live_blocks;
  {
    RocmBundleReceivePolicy provider(mr, align);
    RocmBundleReceivePolicy copy = provider;                  // the facade copies providers
    UcxBuffer block = copy(t.metas);
    // the size the sender's plan computes for the same tensors
    auto plan = eux::axon::rocm::BundlePlan::Create(t.desc.empty() ? nullptr : t.desc.data(), t.desc.size(), align);
    EXPECT(block.size() == plan.payload_bytes());
    EXPECT(block.size() == BundleBytesFor(t.metas, align));
    EXPECT(block.size() == t.oracle_pack(align).size());
    EXPECT(block.type() == ucx_memory_type::ROCM && block.own_buffer() && block.data() != nullptr);
    EXPECT(mr.stats().live_blocks == before + 1);
    // scatter out of the policy's block into fresh tensors: the bytes arrive
    const std::vector<uint8_t> packed = t.oracle_pack(align);
    if (!packed.empty())
      mr.memcpy(ucx_memory_type::ROCM, block.data(), ucx_memory_type::HOST, packed.data(), packed.size());
    std::vector<void*> outs;
    std::vector<axr_tensor_t> dst = t.desc;
    for (size_t i = 0; i < dst.size(); ++i) {
      void* d = t.host[i].empty() ? nullptr : mr.allocate(ucx_memory_type::ROCM, t.host[i].size(), 256);
      outs.push_back(d);
      dst[i].data = d;
    }
    const std::vector<uint8_t> header = plan.header();
    {
      auto rplan = eux::axon::rocm::UnpackTensors(header.data(), header.size(), block.data(), block.size(),
                                                  dst.empty() ? nullptr : dst.data(), dst.size(), nullptr);
    }   // destroying the plan waits for the kernel
    for (size_t i = 0; i < dst.size(); ++i) {
      std::vector<uint8_t> back(t.host[i].size());
      if (!back.empty()) mr.memcpy(ucx_memory_type::HOST, back.data(), ucx_memory_type::ROCM, outs[i], back.size());
      EXPECT(back == t.host[i]);
      if (outs[i]) mr.deallocate(ucx_memory_type::ROCM, outs[i], back.size());
    }
  }
  EXPECT(mr.stats().live_blocks == before);
}

}  // namespace

int main() {
  int count = 0;
  if (axr_device_count(&count) != AXR_OK || count == 0) {
    std::printf("adapters_selftest: no device\n");
    return 2;
  }
  std::mt19937_64 rng(20240607);
  try {
    eux::ucxx::UcxAutoRocmDeviceContext context(0);
    auto active = context(nullptr, nullptr);   // what AxonWorker's constructor does (axon_worker.cpp:80-83)
    UcxRocmMemoryResourceManager mr(0);
    // slabs carry a registration handle, as ucp_mem_map would give one
    int registered = 0, unregistered = 0;
    mr.set_registrar(
        [&registered](void* addr, size_t) { ++registered; return addr; },
        [&unregistered](void*) { ++unregistered; });
    {
      // the reference's own tensor-meta cases (axon_worker_test.cpp:1236-1545): fp32[1024],
      // int32[512] + int32[256], plus ragged sizes, a 0-d and an empty tensor in between
      DeviceTensors t(mr);
      std::vector<std::pair<uint8_t, uint8_t>> dtypes;
      const struct { std::vector<int64_t> shape; uint8_t code, bits; } cases[] = {
          {{1024}, 2, 32}, {{512}, 0, 32}, {{256}, 0, 32}, {{}, 2, 32}, {{3, 0, 5}, 2, 16},
          {{33, 7}, 4, 16}, {{1000003}, 1, 8}, {{5}, 2, 64}, {{300, 300}, 2, 32}, {{1}, 1, 8}};
      for (const auto& c : cases) {
        t.add(rng, c.shape, c.code, c.bits);
        dtypes.push_back({c.code, c.bits});
      }
      t.finish(dtypes);
      round_trip(mr, t);
      policy(mr, t, 1);
      policy(mr, t, 256);
    }
    {
      // a bundle without a single byte: one-byte blocks of size 0 travel and come back
      DeviceTensors t(mr);
      t.add(rng, {0}, 2, 32);
      t.add(rng, {}, 2, 32);
      t.finish({{2, 32}, {2, 32}});
      round_trip(mr, t);
      policy(mr, t, 256);
    }
    {
      DeviceTensors t(mr);   // no tensors at all
      t.finish({});
      round_trip(mr, t);
    }
    const axr_pool_stats_t s = mr.stats();
    EXPECT(s.live_blocks == 0);
    EXPECT(s.allocated_bytes == 0);
    EXPECT(registered >= 1 && unregistered == 0);   // slabs stay registered while the pool lives
    // an oversized split is the reference's std::length_error
    bool threw = false;
    try {
      DeviceTensors t(mr);
      t.add(rng, {64}, 1, 8);
      t.finish({{1, 8}});
      auto bundle = PackTensors(mr, t.desc.data(), 1, 1, nullptr);
      auto sent = ToUcxBuffer(std::move(bundle), mr);
      UcxBuffer small(mr, ucx_memory_type::ROCM, 32);
      (void)ToUcxBufferVec(std::move(small), sent.first.data(), sent.first.size());
    } catch (const std::length_error&) {
      threw = true;
    }
    EXPECT(threw);
    EXPECT(mr.stats().live_blocks == 0);
  } catch (const std::exception& e) {
    std::printf("adapters_selftest: exception: %s\n", e.what());
    return 1;
  }
  if (g_failures) {
    std::printf("adapters_selftest: %d check(s) failed\n", g_failures);
    return 1;
  }
  std::printf("adapters_selftest ok\n");
  return 0;
}
