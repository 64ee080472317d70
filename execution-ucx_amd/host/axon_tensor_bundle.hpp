// C++ face of the tensor-bundle path, for the Axon send and receive call sites.
//
// Sender (replaces building one iov entry per tensor,
// axon/python/src/dlpack_helpers.cpp:745-787, and the forced-rendezvous iov send,
// ucx_context/ucx_connection.cpp:401-426):
//     auto bundle = PackTensors(mr, tensors, n, /*align=*/256, stream);
//     ucx_am_data_t am = bundle.as_am_data();      // one contiguous ROCM buffer + header
//     connection_send(scheduler, conn_id, am);     // ucx_connection.cpp:353-374
// Receiver (replaces the iov scatter of connection_recv_buffer(key, UcxBufferVec),
// ucx_am_context.hpp:1808-1818): receive into ONE pool buffer of
// PayloadBytes(header) bytes, then either SplitPayload (zero copy, the result of
// UcxBuffer::to_buffer_vec, ucx_context_data.hpp:641-665) or UnpackTensors.
#ifndef AXON_ROCM_AXON_TENSOR_BUNDLE_HPP_
#define AXON_ROCM_AXON_TENSOR_BUNDLE_HPP_

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "axon_rocm.h"
#include "ucx_rocm_memory_manager.hpp"

namespace eux {
namespace axon {
namespace rocm {

inline void Check(int rc, const char* what) {
  if (rc == AXR_OK) return;
  const std::string msg = std::string(what) + ": " + axr_status_string(rc) + ": " + axr_last_error();
  if (rc == AXR_ERR_LENGTH) throw std::length_error(msg);   // as to_buffer_vec does
  throw std::runtime_error(msg);
}

// RAII owner of an axr_plan_t.
class BundlePlan {
 public:
  BundlePlan() = default;
  static BundlePlan Create(const axr_tensor_t* tensors, size_t n, uint32_t align) {
    BundlePlan p;
    Check(axr_plan_create(tensors, n, align, 0, &p.plan_), "axr_plan_create");
    return p;
  }
  static BundlePlan FromHeader(const void* header, size_t length) {
    BundlePlan p;
    Check(axr_plan_from_header(header, length, &p.plan_), "axr_plan_from_header");
    return p;
  }
  // The receiver's plan in one pass over the header: decoded and bound to the destination
  // tensors (a memory policy that answers from buffers it already holds).
  static BundlePlan FromHeaderBind(const void* header, size_t length, const axr_tensor_t* tensors, size_t n) {
    BundlePlan p;
    Check(axr_plan_from_header_bind(header, length, tensors, n, &p.plan_), "axr_plan_from_header_bind");
    return p;
  }
  ~BundlePlan() { reset(); }
  BundlePlan(BundlePlan&& o) noexcept : plan_(o.plan_) { o.plan_ = nullptr; }
  BundlePlan& operator=(BundlePlan&& o) noexcept {
    if (this != &o) {
      reset();
      plan_ = o.plan_;
      o.plan_ = nullptr;
    }
    return *this;
  }
  BundlePlan(const BundlePlan&) = delete;
  BundlePlan& operator=(const BundlePlan&) = delete;

  void reset() {
    if (plan_) (void)axr_plan_free(plan_);
    plan_ = nullptr;
  }
  axr_plan_t* get() const { return plan_; }
  size_t size() const {
    size_t n = 0;
    Check(axr_plan_num_tensors(plan_, &n), "axr_plan_num_tensors");
    return n;
  }
  uint64_t payload_bytes() const {
    uint64_t n = 0;
    Check(axr_plan_payload_bytes(plan_, &n), "axr_plan_payload_bytes");
    return n;
  }
  std::vector<uint8_t> header() const {
    const void* p = nullptr;
    size_t n = 0;
    Check(axr_plan_header(plan_, &p, &n), "axr_plan_header");
    const uint8_t* b = static_cast<const uint8_t*>(p);
    return std::vector<uint8_t>(b, b + n);
  }
  void bind(const axr_tensor_t* tensors, size_t n) { Check(axr_plan_bind(plan_, tensors, n), "axr_plan_bind"); }
  // Upload the device tables now: pack/unpack are then single kernel launches
  // that stream capture can record into a HIP graph.
  void prepare(void* stream) { Check(axr_plan_prepare(plan_, stream), "axr_plan_prepare"); }
  void pack(void* payload, size_t bytes, void* stream) { Check(axr_pack(plan_, payload, bytes, stream), "axr_pack"); }
  void unpack(const void* payload, size_t bytes, void* stream) {
    Check(axr_unpack(plan_, payload, bytes, stream), "axr_unpack");
  }
  std::vector<ucx_buffer_t> split(void* payload, size_t bytes) const {
    std::vector<axr_buffer_t> views(size());
    Check(axr_plan_split(plan_, payload, bytes, views.data()), "axr_plan_split");
    std::vector<ucx_buffer_t> out(views.size());
    for (size_t i = 0; i < views.size(); ++i) out[i] = ucx_buffer_t{views[i].data, views[i].size};
    return out;
  }

 private:
  axr_plan_t* plan_ = nullptr;
};

// One packed bundle: header bytes + an owned ROCM pool block.
class TensorBundle {
 public:
  TensorBundle(ucxx::UcxRocmMemoryResourceManager& mr, BundlePlan plan, void* payload,
               size_t payload_bytes, void* mem_h)
      : mr_(&mr), plan_(std::move(plan)), header_(plan_.header()), payload_(payload),
        payload_bytes_(payload_bytes), mem_h_(mem_h) {}
  ~TensorBundle() { release(); }
  TensorBundle(TensorBundle&& o) noexcept
      : mr_(o.mr_), plan_(std::move(o.plan_)), header_(std::move(o.header_)), payload_(o.payload_),
        payload_bytes_(o.payload_bytes_), mem_h_(o.mem_h_) {
    o.payload_ = nullptr;
  }
  TensorBundle(const TensorBundle&) = delete;
  TensorBundle& operator=(const TensorBundle&) = delete;

  // The descriptor connection_send takes (ucx_context/ucx_context_def.h:80-93).
  // Valid while this object lives; the pack must have completed on its stream
  // before the transport reads the buffer.
  ucx_am_data_t as_am_data() {
    ucx_am_data_t d;
    std::memset(&d, 0, sizeof(d));
    d.header = ucx_buffer_t{header_.data(), header_.size()};
    d.buffer = ucx_buffer_t{payload_, payload_bytes_};
    d.buffer_type = ucx_memory_type::ROCM;
    d.mem_h = mem_h_;
    return d;
  }
  const std::vector<uint8_t>& header() const { return header_; }
  void* payload() const { return payload_; }
  size_t payload_bytes() const { return payload_bytes_; }
  void* mem_h() const { return mem_h_; }
  BundlePlan& plan() { return plan_; }
  // Give the block away (e.g. into a UcxBuffer with a release function).
  void* detach() {
    void* p = payload_;
    payload_ = nullptr;
    return p;
  }
  void release() {
    if (payload_) {
      plan_.reset();   // drains the stream the pack ran on
      mr_->deallocate(ucx_memory_type::ROCM, payload_, payload_bytes_);
      payload_ = nullptr;
    }
  }

 private:
  ucxx::UcxRocmMemoryResourceManager* mr_;
  BundlePlan plan_;
  std::vector<uint8_t> header_;
  void* payload_;
  size_t payload_bytes_;
  void* mem_h_;
};

// Gather n tensors (argument order, as InvokeContext::add_tensor establishes it,
// bindings_runtime_helpers.hpp:351-414) into one pool buffer on `stream`.
inline TensorBundle PackTensors(ucxx::UcxRocmMemoryResourceManager& mr, const axr_tensor_t* tensors,
                                size_t n, uint32_t align, void* stream) {
  BundlePlan plan = BundlePlan::Create(tensors, n, align);
  const size_t bytes = plan.payload_bytes();
  void* mem_h = nullptr;
  void* payload = mr.allocate_registered(bytes ? bytes : 1, 256, &mem_h);
  try {
    plan.pack(payload, bytes, stream);
  } catch (...) {
    mr.deallocate(ucx_memory_type::ROCM, payload, bytes);
    throw;
  }
  return TensorBundle(mr, std::move(plan), payload, bytes, mem_h);
}

// Bytes the receiver must provide for a header (the size for the custom memory
// policy's single UcxBuffer, axon/src/axon_worker.cpp:1151-1172).
inline uint64_t PayloadBytes(const void* header, size_t length) {
  return BundlePlan::FromHeader(header, length).payload_bytes();
}

// Scatter a received payload into destination tensors on `stream`.  The returned
// plan must outlive the kernel (destroying it waits for the stream).
inline BundlePlan UnpackTensors(const void* header, size_t header_length, const void* payload,
                                size_t payload_bytes, const axr_tensor_t* dst, size_t n, void* stream) {
  BundlePlan plan = BundlePlan::FromHeader(header, header_length);
  plan.bind(dst, n);
  plan.unpack(payload, payload_bytes, stream);
  return plan;
}

// A device payload as one host byte vector per tensor: what the reference's
// checkpoint writer builds buffer by buffer with mr.memcpy(HOST, ...) per tensor
// (axon/src/storage/avro_serialization.cpp:478-523).  Here the payload crosses the
// bus in 8 MiB pinned blocks, one device copy per block whatever the tensor count,
// and the pieces are cut out on the host.  Blocks until the vectors are filled.
inline std::vector<std::vector<uint8_t>> PayloadToHost(const void* header, size_t header_length,
                                                       const void* payload, size_t payload_bytes,
                                                       void* stream) {
  BundlePlan plan = BundlePlan::FromHeader(header, header_length);
  const size_t n = plan.size();
  std::vector<uint64_t> sizes(n);
  Check(axr_plan_layout(plan.get(), nullptr, sizes.data()), "axr_plan_layout");
  std::vector<std::vector<uint8_t>> out(n);
  std::vector<axr_tensor_t> dst(n);
  for (size_t i = 0; i < n; ++i) {
    out[i].resize(sizes[i]);
    Check(axr_plan_tensor_meta(plan.get(), i, &dst[i]), "axr_plan_tensor_meta");
    dst[i].data = out[i].empty() ? nullptr : out[i].data();
    dst[i].device_type = 1;   // kDLCPU
    dst[i].device_id = 0;
    dst[i].strides = nullptr;
  }
  plan.bind(dst.data(), n);
  plan.unpack(payload, payload_bytes, stream);
  return out;
}

// Several gathers and scatters handed over together (a worker with requests to send and
// responses to scatter at the same moment, axon/src/axon_worker.cpp:1424-1490 next to
// :1098-1219): neighbouring jobs share one kernel launch.  The jobs must not depend on each
// other.
inline void SubmitBundles(const std::vector<axr_job_t>& jobs, void* stream) {
  Check(axr_submit(jobs.data(), jobs.size(), stream), "axr_submit");
}
inline axr_job_t PackJob(const BundlePlan& plan, void* payload, size_t bytes, int64_t tensor_delta = 0) {
  return axr_job_t{plan.get(), 0, payload, bytes, tensor_delta, 0, 0};
}
inline axr_job_t UnpackJob(const BundlePlan& plan, const void* payload, size_t bytes, int64_t tensor_delta = 0) {
  return axr_job_t{plan.get(), 1, const_cast<void*>(payload), bytes, tensor_delta, 0, 0};
}

// A large payload moved in chunks of one geometry: pack -> connection_send ->
// connection_recv_buffer -> unpack per chunk, the chunks double-buffered over `lanes` pairs
// of slots from the manager's pool (ucx_am_context.hpp:2234-2642 and :1511-1844 are the two
// ends of the wire; here a loopback pair stands in for it).  ONE sender plan and ONE receiver
// plan serve every chunk: Submit says how far this chunk's tensors lie from the ones the
// plans are bound to, and never plans, uploads or allocates.
class StreamedTransfer {
 public:
  StreamedTransfer(ucxx::UcxRocmMemoryResourceManager& mr, size_t slot_bytes, int lanes = 2, int streams = 1) {
    Check(axr_transfer_create(mr.pool(), slot_bytes, lanes, streams, &transfer_), "axr_transfer_create");
  }
  ~StreamedTransfer() {
    if (transfer_) (void)axr_transfer_destroy(transfer_);
  }
  StreamedTransfer(const StreamedTransfer&) = delete;
  StreamedTransfer& operator=(const StreamedTransfer&) = delete;
  void Submit(const BundlePlan& send, int64_t send_delta, const BundlePlan& recv, int64_t recv_delta) {
    Check(axr_transfer_submit(transfer_, send.get(), send_delta, recv.get(), recv_delta), "axr_transfer_submit");
  }
  // Zero copy (the default): the receiver scatters straight out of the sender's slot, as after a
  // same-device zero-copy rendezvous; false: every chunk is copied into a receive slot first.
  void SetZeroCopy(bool enable) { Check(axr_transfer_set_zero_copy(transfer_, enable ? 1 : 0), "axr_transfer_set_zero_copy"); }
  // Returns when every submitted chunk has arrived in its destination tensors.
  void Finish() { Check(axr_transfer_finish(transfer_), "axr_transfer_finish"); }

 private:
  axr_transfer_t* transfer_ = nullptr;
};

// Zero-copy receive: views into the payload at the header's offsets.
inline std::vector<ucx_buffer_t> SplitPayload(const void* header, size_t header_length, void* payload,
                                              size_t payload_bytes) {
  return BundlePlan::FromHeader(header, header_length).split(payload, payload_bytes);
}

}  // namespace rocm
}  // namespace axon
}  // namespace eux

#endif  // AXON_ROCM_AXON_TENSOR_BUNDLE_HPP_
