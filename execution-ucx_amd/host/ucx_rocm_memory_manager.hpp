// UcxRocmMemoryResourceManager: the ROCm memory backend of execution-ucx.
//
// Takes the place ucx_context/cuda/ucx_cuda_memory_manager.hpp:43-154 has for
// CUDA, written against the C ABI of libaxon_rocm (no HIP header is included):
//   HOST          std::malloc / std::free, as the CUDA manager does (:93, :124)
//   ROCM          blocks of a hipMalloc slab pool, 256-byte granules; each slab
//                 can be registered once with ucp_mem_map through set_registrar,
//                 and mem_h_of() returns that handle for ucx_am_data_t::mem_h
//   ROCM_MANAGED  pinned, device-visible host memory
// memcpy is blocking like the reference's cudaMemcpy table (:62-78) and covers
// H<->H, H<->D, D<->D plus the pinned type.  Unsupported types throw
// std::runtime_error("Unsupported memory type"), as the reference does; HIP
// failures throw std::runtime_error instead of aborting.  All methods are
// thread-safe: the UCX worker thread, thread-pool threads and Python threads
// all call into one manager (ucx_am_context.cpp:896-905, axon_worker.cpp:1204-1212).
#ifndef AXON_ROCM_UCX_ROCM_MEMORY_MANAGER_HPP_
#define AXON_ROCM_UCX_ROCM_MEMORY_MANAGER_HPP_

#include <functional>
#include <stdexcept>
#include <string>
#include <utility>

#include "axon_rocm.h"
#include "reference_interfaces.hpp"

namespace eux {
namespace ucxx {

class UcxRocmMemoryResourceManager : public UcxMemoryResourceManager {
 public:
  using RegisterFn = std::function<void*(void* addr, size_t length)>;   // returns ucp_mem_h
  using UnregisterFn = std::function<void(void* mem_h)>;

  explicit UcxRocmMemoryResourceManager(int device = 0, size_t slab_bytes = 0) : device_(device) {
    Check(axr_pool_create(device, slab_bytes, &pool_), "axr_pool_create");
  }
  ~UcxRocmMemoryResourceManager() override {
    if (pool_) (void)axr_pool_destroy(pool_);
  }
  UcxRocmMemoryResourceManager(const UcxRocmMemoryResourceManager&) = delete;
  UcxRocmMemoryResourceManager& operator=(const UcxRocmMemoryResourceManager&) = delete;

  // Wire slab registration to ucx_am_context::register_ucx_memory /
  // unregister_ucx_memory (ucx_am_context.cpp:1128-1147).  Call before the
  // first ROCM allocation.
  void set_registrar(RegisterFn reg, UnregisterFn unreg) {
    reg_ = std::move(reg);
    unreg_ = std::move(unreg);
    Check(axr_pool_set_registrar(pool_, &UcxRocmMemoryResourceManager::RegisterThunk,
                                 &UcxRocmMemoryResourceManager::UnregisterThunk, this),
          "axr_pool_set_registrar");
  }

  void* allocate(ucx_memory_type_t type, size_t bytes, size_t alignment = 8) override {
    void* p = nullptr;
    switch (type) {
      case ucx_memory_type::ROCM:
        Check(axr_pool_alloc(pool_, bytes, alignment, &p, nullptr), "axr_pool_alloc");
        return p;
      case ucx_memory_type::HOST:
      case ucx_memory_type::ROCM_MANAGED:
        Check(axr_mem_alloc(static_cast<int>(type), bytes, alignment, &p), "axr_mem_alloc");
        return p;
      default:
        throw std::runtime_error("Unsupported memory type");
    }
  }

  // Same as allocate(ROCM, ...) but also hands back the slab's registration
  // handle, the value for ucx_am_data_t::mem_h (ucx_context_def.h:80-93).
  void* allocate_registered(size_t bytes, size_t alignment, void** mem_h) {
    void* p = nullptr;
    Check(axr_pool_alloc(pool_, bytes, alignment, &p, mem_h), "axr_pool_alloc");
    return p;
  }

  void deallocate(ucx_memory_type_t type, void* p, size_t bytes, size_t /*alignment*/ = 8) override {
    switch (type) {
      case ucx_memory_type::ROCM:
        Check(axr_pool_free(pool_, p), "axr_pool_free");
        return;
      case ucx_memory_type::HOST:
      case ucx_memory_type::ROCM_MANAGED:
        Check(axr_mem_free(static_cast<int>(type), p, bytes), "axr_mem_free");
        return;
      default:
        throw std::runtime_error("Unsupported memory type");
    }
  }

  void* memcpy(ucx_memory_type_t dest_type, void* dest, ucx_memory_type_t src_type,
               const void* src, size_t count) override {
    const int rc = axr_memcpy(static_cast<int>(dest_type), dest, static_cast<int>(src_type), src, count);
    if (rc == AXR_ERR_UNSUPPORTED) throw std::runtime_error("Unsupported memory copy combination");
    Check(rc, "axr_memcpy");
    return dest;
  }

  axr_pool_t* pool() const { return pool_; }
  int device() const { return device_; }
  axr_pool_stats_t stats() const {
    axr_pool_stats_t s{};
    Check(axr_pool_get_stats(pool_, &s), "axr_pool_get_stats");
    return s;
  }

 private:
  static void Check(int rc, const char* what) {
    if (rc != AXR_OK)
      throw std::runtime_error(std::string(what) + ": " + axr_status_string(rc) + ": " + axr_last_error());
  }
  static int RegisterThunk(void* user, void* addr, size_t length, void** mem_h) {
    auto* self = static_cast<UcxRocmMemoryResourceManager*>(user);
    try {
      *mem_h = self->reg_ ? self->reg_(addr, length) : nullptr;
      return 0;
    } catch (...) {
      return -1;
    }
  }
  static void UnregisterThunk(void* user, void* mem_h) {
    auto* self = static_cast<UcxRocmMemoryResourceManager*>(user);
    if (self->unreg_) self->unreg_(mem_h);
  }

  int device_;
  axr_pool_t* pool_ = nullptr;
  RegisterFn reg_;
  UnregisterFn unreg_;
};

}  // namespace ucxx
}  // namespace eux

#endif  // AXON_ROCM_UCX_ROCM_MEMORY_MANAGER_HPP_
