// Compiled (syntax only) by tests/test_host_cpp.py with -DAXON_ROCM_IN_REFERENCE_TREE
// and the execution-ucx tree on the include path: proves that the ROCm classes
// derive from the reference's real UcxMemoryResourceManager and that the
// adapters build against its real UcxBuffer / UcxBufferVec.
#include "reference_adapters.hpp"
#include "ucx_rocm_context.hpp"
#include "ucx_rocm_memory_manager.hpp"

#ifndef AXON_ROCM_HAVE_REFERENCE_MEMORY_RESOURCE
#error "the reference's ucx_memory_resource.hpp was not picked up"
#endif

static_assert(std::is_base_of<eux::ucxx::UcxMemoryResourceManager,
                              eux::ucxx::UcxRocmMemoryResourceManager>::value,
              "ROCm manager must plug into the reference interface");
static_assert(!std::is_abstract<eux::ucxx::UcxRocmMemoryResourceManager>::value,
              "every pure virtual of the reference interface is implemented");
static_assert(static_cast<int>(ucx_memory_type::ROCM) == AXR_MEM_ROCM &&
              static_cast<int>(ucx_memory_type::ROCM_MANAGED) == AXR_MEM_ROCM_MANAGED &&
              static_cast<int>(ucx_memory_type::HOST) == AXR_MEM_HOST,
              "memory type numbering is shared with the C ABI");
static_assert(sizeof(ucx_buffer_t) == sizeof(axr_buffer_t), "buffer views are interchangeable");

eux::ucxx::UcxBufferVec Exercise(eux::ucxx::UcxRocmMemoryResourceManager& mr, const axr_tensor_t* t,
                                 size_t n) {
  auto bundle = eux::axon::rocm::PackTensors(mr, t, n, 1, nullptr);
  auto sent = eux::axon::rocm::ToUcxBuffer(std::move(bundle), mr);
  eux::ucxx::UcxBuffer recv =
      eux::axon::rocm::ReceiveBufferFor(sent.first.data(), sent.first.size(), mr);
  mr.memcpy(ucx_memory_type::ROCM, recv.data(), ucx_memory_type::ROCM, sent.second.data(),
            sent.second.size());
  return eux::axon::rocm::ToUcxBufferVec(std::move(recv), sent.first.data(), sent.first.size());
}

// The receive policy is generic over the meta record; rpc::utils::TensorMeta itself
// needs cista, which is not installed here, so a record with the same fields stands in.
namespace {
struct MetaLike {
  struct { int32_t device_type, device_id; } device;
  int32_t ndim;
  struct { uint8_t code, bits; uint16_t lanes; } dtype;
  uint64_t byte_offset;
  std::vector<int64_t> shape, strides;
};
}  // namespace

eux::ucxx::UcxBuffer ExercisePolicy(eux::ucxx::UcxRocmMemoryResourceManager& mr,
                                    const std::vector<MetaLike>& metas) {
  eux::axon::rocm::RocmBundleReceivePolicy policy(mr, 256);
  eux::axon::rocm::RocmBundleReceivePolicy copy = policy;   // the facade copies providers
  return copy(metas);
}
