// Where the ROCm backend plugs into execution-ucx.
//
// Inside the execution-ucx source tree the real headers are used:
//   ucx_context/ucx_context_def.h          ucx_memory_type_t, ucx_buffer_t, ucx_am_data_t
//   ucx_context/ucx_memory_resource.hpp    eux::ucxx::UcxMemoryResourceManager  (:99-123)
//   ucx_context/ucx_device_context.hpp     eux::ucxx::OperationRAII, UcxAutoDeviceContext (:38-80)
// Outside it (this repository's own build and tests) the same names are declared
// here with the same signatures, reduced to what the ROCm classes override, so
// that the backend compiles and can be exercised without UCX installed.
#ifndef AXON_ROCM_REFERENCE_INTERFACES_HPP_
#define AXON_ROCM_REFERENCE_INTERFACES_HPP_

#include <cstddef>
#include <memory>

#if defined(AXON_ROCM_IN_REFERENCE_TREE) && __has_include("ucx_context/ucx_memory_resource.hpp")
#include "ucx_context/ucx_context_def.h"
#include "ucx_context/ucx_memory_resource.hpp"
#define AXON_ROCM_HAVE_REFERENCE_MEMORY_RESOURCE 1
#if __has_include(<ucp/api/ucp.h>)
#include "ucx_context/ucx_device_context.hpp"
#define AXON_ROCM_HAVE_REFERENCE_DEVICE_CONTEXT 1
#endif
#endif

#ifndef AXON_ROCM_HAVE_REFERENCE_MEMORY_RESOURCE
extern "C" {
typedef enum ucx_memory_type {
  HOST, CUDA, CUDA_MANAGED, ROCM, ROCM_MANAGED, RDMA, ZE_HOST, ZE_DEVICE, ZE_MANAGED,
  LAST, UNKNOWN = LAST
} ucx_memory_type_t;
typedef struct ucx_buffer { void* data; size_t size; } ucx_buffer_t;
typedef ucx_buffer_t ucx_header_t;
typedef struct ucx_am_data {
  ucx_buffer_t header;
  ucx_buffer_t buffer;
  ucx_memory_type_t buffer_type;
  void* mem_h;
} ucx_am_data_t;
}
namespace eux {
namespace ucxx {
class UcxMemoryResourceManager {
 public:
  virtual ~UcxMemoryResourceManager() = default;
  virtual void* allocate(ucx_memory_type_t type, size_t bytes, size_t alignment = 8) = 0;
  virtual void deallocate(ucx_memory_type_t type, void* p, size_t bytes, size_t alignment = 8) = 0;
  virtual void* memcpy(ucx_memory_type_t dest_type, void* dest, ucx_memory_type_t src_type,
                       const void* src, size_t count) = 0;
};
}  // namespace ucxx
}  // namespace eux
#endif

#ifndef AXON_ROCM_HAVE_REFERENCE_DEVICE_CONTEXT
#if !__has_include(<ucp/api/ucp.h>)
typedef struct ucp_context* ucp_context_h;   // opaque UCX handles, never dereferenced here
typedef struct ucp_worker* ucp_worker_h;
#else
#include <ucp/api/ucp.h>
#endif
namespace eux {
namespace ucxx {
class UcxAutoDeviceContext;
class OperationRAII {
 public:
  OperationRAII(UcxAutoDeviceContext* context, const ucp_context_h ucp_context,
                const ucp_worker_h ucp_worker)
      : context_(context), ucp_context_(ucp_context), ucp_worker_(ucp_worker) {}
  virtual ~OperationRAII() = default;
  virtual void activate() = 0;
  virtual void deactivate() = 0;
  OperationRAII(const OperationRAII&) = delete;
  OperationRAII& operator=(const OperationRAII&) = delete;

 protected:
  UcxAutoDeviceContext* context_;
  const ucp_context_h ucp_context_;
  const ucp_worker_h ucp_worker_;
};
class UcxAutoDeviceContext {
 public:
  virtual ~UcxAutoDeviceContext() = default;
  virtual std::unique_ptr<OperationRAII> operator()(const ucp_context_h ucp_context,
                                                    const ucp_worker_h ucp_worker) = 0;
  virtual std::unique_ptr<UcxAutoDeviceContext> clone() const = 0;
};
}  // namespace ucxx
}  // namespace eux
#endif

#endif  // AXON_ROCM_REFERENCE_INTERFACES_HPP_
