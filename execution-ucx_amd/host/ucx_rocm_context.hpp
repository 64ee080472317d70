// UcxAutoRocmDeviceContext: thread-level device activation for execution-ucx.
//
// Same contract as UcxAutoCudaDeviceContext (ucx_context/cuda/ucx_cuda_context.hpp:31-88):
// operator() returns an RAII object that makes the device current on the calling
// thread and restores the previous one when destroyed; clone() gives every
// ucx_am_context its own copy.  It is activated for the whole AxonWorker
// constructor, for each ucx_am_context constructor and for the lifetime of the
// worker loop (axon_worker.cpp:80-83, ucx_am_context.cpp:140-144, 237-240), with
// null UCX handles in the first two cases, which this class never dereferences.
// HIP has one primary context per device, so the device ordinal plays the role
// the CUcontext plays there.  Failures throw instead of aborting.
#ifndef AXON_ROCM_UCX_ROCM_CONTEXT_HPP_
#define AXON_ROCM_UCX_ROCM_CONTEXT_HPP_

#include <memory>
#include <stdexcept>
#include <string>

#include "axon_rocm.h"
#include "reference_interfaces.hpp"

namespace eux {
namespace ucxx {

class UcxAutoRocmDeviceContext : public UcxAutoDeviceContext {
 public:
  explicit UcxAutoRocmDeviceContext(int device) : device_(device) {}
  ~UcxAutoRocmDeviceContext() override = default;

  class RocmOperation : public OperationRAII {
   public:
    using OperationRAII::OperationRAII;
    ~RocmOperation() override { deactivate(); }

    void activate() override {
      if (active_) return;
      auto* owner = static_cast<UcxAutoRocmDeviceContext*>(context_);
      const int rc = axr_device_push(owner->device_, &previous_);
      if (rc != AXR_OK)
        throw std::runtime_error(std::string("axr_device_push: ") + axr_last_error());
      active_ = true;
    }

    void deactivate() override {
      if (!active_) return;
      active_ = false;
      (void)axr_device_pop(previous_);   // runs from a destructor: never throws
    }

   private:
    int previous_ = 0;
    bool active_ = false;
  };

  std::unique_ptr<OperationRAII> operator()(const ucp_context_h ucp_context,
                                            const ucp_worker_h ucp_worker) override {
    auto op = std::make_unique<RocmOperation>(this, ucp_context, ucp_worker);
    op->activate();
    return op;
  }

  std::unique_ptr<UcxAutoDeviceContext> clone() const override {
    return std::make_unique<UcxAutoRocmDeviceContext>(device_);
  }

  int device() const { return device_; }

 private:
  int device_;
};

}  // namespace ucxx
}  // namespace eux

#endif  // AXON_ROCM_UCX_ROCM_CONTEXT_HPP_
