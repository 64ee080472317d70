// Adapters that only make sense inside the execution-ucx source tree: they turn
// a packed bundle into the reference's owning buffer types.  Compiled when
// AXON_ROCM_IN_REFERENCE_TREE is defined and the reference headers are on the
// include path (ucx_context/ucx_context_data.hpp needs nothing but the standard
// library, so this part also builds where UCX itself is not installed).
#ifndef AXON_ROCM_REFERENCE_ADAPTERS_HPP_
#define AXON_ROCM_REFERENCE_ADAPTERS_HPP_

#if defined(AXON_ROCM_IN_REFERENCE_TREE) && __has_include("ucx_context/ucx_context_data.hpp")

#include <memory>
#include <utility>

#include "axon_tensor_bundle.hpp"
#include "ucx_context/ucx_context_data.hpp"

namespace eux {
namespace axon {
namespace rocm {

// The packed payload as an owning UcxBuffer (memory type ROCM, the slab's
// ucp_mem_h attached).  The block returns to the pool through the buffer's
// release function (ucx_context_data.hpp:121-129), the way the reference keeps
// DLPack owners alive in dlpack_helpers.cpp:739-742.  The header bytes are
// returned next to it; they become the AM header.
inline std::pair<std::vector<uint8_t>, ucxx::UcxBuffer> ToUcxBuffer(
    TensorBundle&& bundle, ucxx::UcxRocmMemoryResourceManager& mr) {
  std::vector<uint8_t> header = bundle.header();
  const size_t bytes = bundle.payload_bytes();
  void* mem_h = bundle.mem_h();
  // keep the plan (and with it the stream ordering) alive until the block is released
  auto keep = std::make_shared<TensorBundle>(std::move(bundle));
  void* data = keep->payload();
  ucxx::UcxBuffer buffer(mr, ucx_memory_type::ROCM, data, bytes, mem_h, /*own_buffer=*/true,
                         [keep](void*) mutable { keep->release(); });
  return {std::move(header), std::move(buffer)};
}

// Receive side of a custom memory policy (axon/include/axon/memory_policy.hpp:72-73):
// one ROCM pool block sized from the bundle header, as an owning UcxBuffer.
inline ucxx::UcxBuffer ReceiveBufferFor(const void* header, size_t header_length,
                                        ucxx::UcxRocmMemoryResourceManager& mr) {
  const size_t bytes = PayloadBytes(header, header_length);
  void* mem_h = nullptr;
  void* data = mr.allocate_registered(bytes ? bytes : 1, 256, &mem_h);
  ucxx::UcxRocmMemoryResourceManager* pmr = &mr;
  return ucxx::UcxBuffer(mr, ucx_memory_type::ROCM, data, bytes, mem_h, /*own_buffer=*/true,
                         [pmr, bytes](void* p) { pmr->deallocate(ucx_memory_type::ROCM, p, bytes); });
}

// Bytes of the packed payload for a list of tensor metas: the layout rule of the
// bundle (offset[i+1] = align_up(offset[i] + nbytes[i])) with the reference's size
// rule (rpc_core/utils/tensor_meta.hpp:91-104).  `Metas` is any range of records
// with the fields of rpc::utils::TensorMeta (`ndim`, `dtype.bits`, `shape[i]`),
// e.g. rpc::utils::TensorMetaSpan.
template <typename Metas>
inline size_t BundleBytesFor(const Metas& metas, uint32_t align) {
  uint64_t end = 0;
  for (const auto& m : metas) {
    uint64_t nbytes = 0;
    if (m.ndim != 0) {
      nbytes = (static_cast<uint64_t>(m.dtype.bits) + 7) / 8;
      for (int32_t d = 0; d < m.ndim; ++d) nbytes *= static_cast<uint64_t>(m.shape[d]);
    }
    end = (end + align - 1) / align * align + nbytes;
  }
  return static_cast<size_t>(end);
}

// A receive-side memory policy: callable with the tensor metas of an incoming
// rendezvous message, returns ONE ROCm pool block (with the slab's ucp_mem_h) that
// the whole bundle lands in.  Usable as eux::axon::CustomMemoryPolicy<ucxx::UcxBuffer>
// (axon/include/axon/memory_policy.hpp:28-36,72-73); the worker calls it from
// ProcessRndvBufferImpl_ (axon/src/axon_worker.cpp:1150-1172).  Copyable, as the
// facade requires; the manager must outlive it.
class RocmBundleReceivePolicy {
 public:
  RocmBundleReceivePolicy(ucxx::UcxRocmMemoryResourceManager& mr, uint32_t align)
      : mr_(&mr), align_(align) {}

  template <typename Metas>
  ucxx::UcxBuffer operator()(Metas metas) const {
    const size_t bytes = BundleBytesFor(metas, align_);
    void* mem_h = nullptr;
    void* data = mr_->allocate_registered(bytes ? bytes : 1, 256, &mem_h);
    ucxx::UcxRocmMemoryResourceManager* mr = mr_;
    return ucxx::UcxBuffer(*mr, ucx_memory_type::ROCM, data, bytes, mem_h, /*own_buffer=*/true,
                           [mr, bytes](void* p) { mr->deallocate(ucx_memory_type::ROCM, p, bytes); });
  }

 private:
  ucxx::UcxRocmMemoryResourceManager* mr_;
  uint32_t align_;
};

// Zero-copy split of a received payload: UcxBuffer::to_buffer_vec with the sizes
// the bundle header carries, valid for the tight layout (align == 1) the
// reference understands; aligned layouts use SplitPayload instead.
inline ucxx::UcxBufferVec ToUcxBufferVec(ucxx::UcxBuffer&& payload, const void* header,
                                         size_t header_length) {
  BundlePlan plan = BundlePlan::FromHeader(header, header_length);
  const size_t n = plan.size();
  std::vector<uint64_t> sizes(n);
  Check(axr_plan_layout(plan.get(), nullptr, sizes.data()), "axr_plan_layout");
  return std::move(payload).to_buffer_vec(std::vector<size_t>(sizes.begin(), sizes.end()));
}

}  // namespace rocm
}  // namespace axon
}  // namespace eux

#endif
#endif  // AXON_ROCM_REFERENCE_ADAPTERS_HPP_
