// The active-message bundle surface of execution-ucx over the loopback context of
// libaxon_rocm: the C++ face the pack / unpack stage sits behind.
//
//   connection_send(sched, conn, ucx_am_data& | UcxAmData&& | ucx_am_iovec& | UcxAmIovec&&)
//   connection_recv(sched, ucx_am_data& | ucx_memory_type)          -> active_message_bundle
//   connection_recv_header(sched)                                   -> recv_header_result_type
//   connection_recv_buffer(sched, key, ucx_memory_type | UcxBuffer&& | UcxBufferVec&&)
//                                                                   -> active_message_buffer_bundle_t<...>
//
// Same names, argument types and result types as the customisation points of
// ucx_context/ucx_context_concept.hpp:247-470 and the bundle classes of
// ucx_context/ucx_am_context/ucx_am_context.hpp:128-315, with the reference's own
// UcxBuffer / UcxHeader / UcxAmData / UcxAmIovec / UcxBufferVec (ucx_context_data.hpp) as
// the owning types.  Each call returns a sender: `connect(sender, receiver)` gives an
// operation, `start()` runs it, and the receiver is completed exactly once with
//   set_value(result...)            success
//   set_error(std::error_code)      failure (category names the UCS status the reference reports)
//   set_done()                      cancelled (`request_stop()` on the operation)
// which is the completion contract of the reference's senders (ucx_am_context.hpp:1352-1400,
// 1734-1765, 2508-2560).  Lvalue arguments are borrowed and must outlive the operation;
// rvalue arguments are owned by the operation until it completes.
//
// What is different from the reference: there is no UCX and no unifex here, so the
// scheduler is this header's own small type and nothing hops to a context thread.  An
// operation does its work inside start() when it can; one that has to wait (a receive with
// no message queued, a rendezvous send whose payload has not been fetched) is parked in the
// context and completed by a later loopback_am_context::progress() call, the stand-in for
// the reference's run loop (ucx_am_context.cpp:218-296).  sync_wait(sender) drives
// progress() until the sender has completed.
//
// Needs the execution-ucx tree on the include path (-DAXON_ROCM_IN_REFERENCE_TREE): the
// owning types are the reference's.
#ifndef AXON_ROCM_LOOPBACK_AM_CONTEXT_HPP_
#define AXON_ROCM_LOOPBACK_AM_CONTEXT_HPP_

#if defined(AXON_ROCM_IN_REFERENCE_TREE) && __has_include("ucx_context/ucx_context_data.hpp")

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <system_error>
#include <type_traits>
#include <utility>
#include <variant>
#include <vector>

#include "axon_rocm.h"
#include "ucx_context/ucx_context_data.hpp"
#include "ucx_rocm_memory_manager.hpp"

namespace eux {
namespace ucxx {
namespace loopback {

// ---------------------------------------------------------------- error codes

// The statuses this surface reports, named after the ucs_status_t values the reference
// completes with (ucx_status.hpp:35-148 maps those into std::error_code the same way).
enum class am_errc : int {
  no_message = AXR_ERR_NO_MESSAGE,            // UCS_ERR_NO_MESSAGE       ucx_am_context.hpp:1570-1574
  not_implemented = AXR_ERR_NOT_IMPLEMENTED,  // UCS_ERR_NOT_IMPLEMENTED  :1643-1651
  canceled = AXR_ERR_CANCELED,                // UCS_ERR_CANCELED
  invalid_param = AXR_ERR_INVALID,            // UCS_ERR_INVALID_PARAM
  no_memory = AXR_ERR_NOMEM,                  // UCS_ERR_NO_MEMORY
  message_truncated = AXR_ERR_LENGTH,         // UCS_ERR_MESSAGE_TRUNCATED
  unsupported = AXR_ERR_UNSUPPORTED,          // UCS_ERR_UNSUPPORTED
  unreachable = AXR_ERR_NO_DEVICE,            // UCS_ERR_UNREACHABLE (peer gone)
  io_error = AXR_ERR_HIP                      // UCS_ERR_IO_ERROR
};

class am_error_category final : public std::error_category {
 public:
  const char* name() const noexcept override { return "ucx.loopback"; }
  std::string message(int value) const override {
    switch (static_cast<am_errc>(value)) {
      case am_errc::no_message: return "UCS_ERR_NO_MESSAGE";
      case am_errc::not_implemented: return "UCS_ERR_NOT_IMPLEMENTED";
      case am_errc::canceled: return "UCS_ERR_CANCELED";
      case am_errc::invalid_param: return "UCS_ERR_INVALID_PARAM";
      case am_errc::no_memory: return "UCS_ERR_NO_MEMORY";
      case am_errc::message_truncated: return "UCS_ERR_MESSAGE_TRUNCATED";
      case am_errc::unsupported: return "UCS_ERR_UNSUPPORTED";
      case am_errc::unreachable: return "UCS_ERR_UNREACHABLE";
      case am_errc::io_error: return "UCS_ERR_IO_ERROR";
    }
    return std::string("axon_rocm status ") + axr_status_string(value);
  }
};
inline const std::error_category& am_category() {
  static am_error_category category;
  return category;
}
inline std::error_code make_error_code(am_errc e) { return {static_cast<int>(e), am_category()}; }
// A status of the C ABI as the error the reference would complete with.
inline std::error_code status_to_error(int axr_status) {
  return axr_status == AXR_ERR_MISMATCH || axr_status == AXR_ERR_HEADER || axr_status == AXR_ERR_BUSY
             ? make_error_code(am_errc::invalid_param)
             : std::error_code(axr_status, am_category());
}

// ---------------------------------------------------------------- connection, bundles

// What the reference's UcxConnection is to its bundles: the endpoint a message came from
// or goes to.  id() is the value connection_send takes (ucx_connection.hpp:364).
class LoopbackConnection {
 public:
  LoopbackConnection() = default;
  explicit LoopbackConnection(std::uint64_t id) : id_(id) {}
  std::uint64_t id() const { return id_; }

 private:
  std::uint64_t id_ = 0;
};

// ucx_am_context.hpp:128-169
class active_message_bundle {
 public:
  active_message_bundle(UcxAmData&& data, const LoopbackConnection& conn) : data_(std::move(data)), conn_(conn) {}
  active_message_bundle(const active_message_bundle&) = delete;
  active_message_bundle& operator=(const active_message_bundle&) = delete;
  active_message_bundle(active_message_bundle&&) = default;
  active_message_bundle& operator=(active_message_bundle&&) = delete;
  const UcxAmData& data() const { return data_; }
  UcxAmData&& move_data() { return std::move(data_); }
  const ucx_am_data& get_raw_data() const { return *data_.get(); }
  const LoopbackConnection& connection() const { return conn_; }

 private:
  UcxAmData data_;
  LoopbackConnection conn_;
};

// ucx_am_context.hpp:210-253
template <typename BufferType>
class active_message_buffer_bundle_t {
  static_assert(std::is_same_v<BufferType, UcxBuffer> || std::is_same_v<BufferType, UcxBufferVec>,
                "UcxBuffer or UcxBufferVec");

 public:
  active_message_buffer_bundle_t(BufferType&& buffer, const LoopbackConnection& conn)
      : buffer_(std::move(buffer)), conn_(conn) {}
  active_message_buffer_bundle_t(const active_message_buffer_bundle_t&) = delete;
  active_message_buffer_bundle_t& operator=(const active_message_buffer_bundle_t&) = delete;
  active_message_buffer_bundle_t(active_message_buffer_bundle_t&&) = default;
  active_message_buffer_bundle_t& operator=(active_message_buffer_bundle_t&&) = default;
  const BufferType& buffer() const { return buffer_; }
  BufferType&& move_buffer() { return std::move(buffer_); }
  const LoopbackConnection& connection() const { return conn_; }

 private:
  BufferType buffer_;
  LoopbackConnection conn_;
};
using active_message_buffer_bundle = active_message_buffer_bundle_t<UcxBuffer>;
using active_message_iovec_buffer_bundle = active_message_buffer_bundle_t<UcxBufferVec>;

// ucx_am_context.hpp:255-315
template <typename BufferType>
class active_message_header_buffer_bundle_t {
 public:
  active_message_header_buffer_bundle_t(UcxHeader&& header, BufferType&& buffer, const LoopbackConnection& conn)
      : header_(std::move(header)), buffer_(std::move(buffer)), conn_(conn) {}
  active_message_header_buffer_bundle_t(const active_message_header_buffer_bundle_t&) = delete;
  active_message_header_buffer_bundle_t& operator=(const active_message_header_buffer_bundle_t&) = delete;
  active_message_header_buffer_bundle_t(active_message_header_buffer_bundle_t&&) = default;
  active_message_header_buffer_bundle_t& operator=(active_message_header_buffer_bundle_t&&) = default;
  const UcxHeader& header() const { return header_; }
  UcxHeader&& move_header() { return std::move(header_); }
  const BufferType& buffer() const { return buffer_; }
  BufferType&& move_buffer() { return std::move(buffer_); }
  const LoopbackConnection& connection() const { return conn_; }

 private:
  UcxHeader header_;
  BufferType buffer_;
  LoopbackConnection conn_;
};
using active_message_header_buffer_bundle = active_message_header_buffer_bundle_t<UcxBuffer>;

// ucx_am_context.hpp:313-315
using recv_header_result_type =
    std::variant<std::pair<size_t, UcxHeader>, active_message_header_buffer_bundle>;

// ---------------------------------------------------------------- the context

class loopback_am_context;

namespace detail {
// An operation that could not complete inside start(): poll() is called from
// loopback_am_context::progress() until it returns true (then it has completed its receiver).
struct parked_operation {
  virtual ~parked_operation() = default;
  virtual bool poll() = 0;
};
}  // namespace detail

// One endpoint of a loopback pair (test_code/test_cuda_connection.cpp:256-297 is the
// reference's own in-process topology).  Holds the memory resource that header and receive
// buffers come from, as ucx_am_context holds its `mr_`.
class loopback_am_context {
 public:
  class scheduler {
   public:
    explicit scheduler(loopback_am_context* ctx) : ctx_(ctx) {}
    loopback_am_context& context() const { return *ctx_; }

   private:
    loopback_am_context* ctx_;
  };

  explicit loopback_am_context(UcxMemoryResourceManager& mr, const char* name = "loopback",
                               size_t zcopy_thresh = 0, void* stream = nullptr)
      : mr_(mr), stream_(stream) {
    const int rc = axr_am_context_create(name, zcopy_thresh, &ctx_);
    if (rc) throw std::system_error(status_to_error(rc), axr_last_error());
    if (!stream_) {
      const int rs = axr_stream_create(&stream_);
      if (rs == AXR_OK) own_stream_ = true;
      else stream_ = nullptr;   // no device: host payloads still move
    }
  }
  ~loopback_am_context() {
    if (ctx_) (void)axr_am_context_destroy(ctx_);
    if (own_stream_) (void)axr_stream_destroy(stream_);
  }
  loopback_am_context(const loopback_am_context&) = delete;
  loopback_am_context& operator=(const loopback_am_context&) = delete;

  scheduler get_scheduler() { return scheduler(this); }
  UcxMemoryResourceManager& memory_resource() const { return mr_.get(); }
  std::reference_wrapper<UcxMemoryResourceManager> mr() const { return mr_; }
  axr_am_context_t* handle() const { return ctx_; }
  void* stream() const { return stream_; }

  // Endpoint from this context to `peer` (connect_endpoint of the reference, reduced to the
  // in-process case).
  LoopbackConnection connect(loopback_am_context& peer) {
    std::uint64_t id = 0;
    const int rc = axr_am_connect(ctx_, peer.ctx_, &id);
    if (rc) throw std::system_error(status_to_error(rc), axr_last_error());
    return LoopbackConnection(id);
  }

  // One turn of the run loop: lets waiting sends start, and completes parked operations
  // that can complete now.  Returns the number of operations still parked.
  size_t progress() {
    (void)axr_am_progress(ctx_, nullptr, nullptr);
    std::vector<detail::parked_operation*> turn;
    {
      std::lock_guard<std::mutex> lock(mu_);
      turn = parked_;
    }
    for (detail::parked_operation* op : turn) {
      {
        std::lock_guard<std::mutex> lock(mu_);
        if (std::find(parked_.begin(), parked_.end(), op) == parked_.end()) continue;   // stopped meanwhile
      }
      if (op->poll()) unpark(op);
    }
    std::lock_guard<std::mutex> lock(mu_);
    return parked_.size();
  }

  void park(detail::parked_operation* op) {
    std::lock_guard<std::mutex> lock(mu_);
    parked_.push_back(op);
  }
  // True when the operation was still parked (the caller then completes it).
  bool unpark(detail::parked_operation* op) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = std::find(parked_.begin(), parked_.end(), op);
    if (it == parked_.end()) return false;
    parked_.erase(it);
    return true;
  }

 private:
  std::reference_wrapper<UcxMemoryResourceManager> mr_;
  axr_am_context_t* ctx_ = nullptr;
  void* stream_ = nullptr;
  bool own_stream_ = false;
  std::mutex mu_;
  std::vector<detail::parked_operation*> parked_;
};

using scheduler = loopback_am_context::scheduler;

// connect(sender, receiver): the operation state.  The receiver is any type with
// set_value(...), set_error(std::error_code) and set_done().
template <typename Sender, typename Receiver>
auto connect(Sender&& sender, Receiver&& receiver) {
  return std::forward<Sender>(sender).connect(std::forward<Receiver>(receiver));
}

namespace detail {

inline std::uint64_t conn_id_of(std::uint64_t id) { return id; }
inline std::uint64_t conn_id_of(const LoopbackConnection& c) { return c.id(); }

static_assert(sizeof(axr_am_data_t) == sizeof(ucx_am_data_t) && sizeof(axr_am_iovec_t) == sizeof(ucx_am_iovec_t) &&
                  sizeof(axr_buffer_t) == sizeof(ucx_buffer_t),
              "the C ABI's descriptors are the reference's, field for field");

inline axr_am_data_t to_abi(const ucx_am_data& d) {
  axr_am_data_t out;
  out.header = axr_buffer_t{d.header.data, d.header.size};
  out.buffer = axr_buffer_t{d.buffer.data, d.buffer.size};
  out.buffer_type = static_cast<int>(d.buffer_type);
  out.mem_h = d.mem_h;
  return out;
}

// Host copy of a message header in memory of the context's resource manager, as
// am_recv_callback makes one (ucx_am_context.cpp:896-905).
inline UcxHeader copy_header(loopback_am_context& ctx, const axr_am_message_t& m) {
  UcxHeader header(ctx.mr(), m.header.size, /*own_header=*/true);
  if (m.header.size) std::memcpy(header.data(), m.header.data, m.header.size);
  return header;
}

// ------------------------------------------------------------ send

// ucx_am_context.hpp:2234-2642.  Payload is ucx_am_data or ucx_am_iovec (borrowed) or
// UcxAmData / UcxAmIovec (owned).
template <typename Owned, typename View>
class send_sender {
 public:
  send_sender(loopback_am_context& ctx, std::uint64_t conn, View& borrowed) : ctx_(ctx), conn_(conn), view_(&borrowed) {}
  send_sender(loopback_am_context& ctx, std::uint64_t conn, Owned&& owned)
      : ctx_(ctx), conn_(conn), owned_(std::move(owned)), view_(nullptr) {}

  template <typename Receiver>
  class operation final : private parked_operation {
   public:
    operation(send_sender&& s, Receiver&& r)
        : ctx_(s.ctx_), conn_(s.conn_), owned_(std::move(s.owned_)),
          view_(owned_ ? owned_->get() : s.view_), receiver_(std::move(r)) {}
    operation(const operation&) = delete;
    operation& operator=(const operation&) = delete;
    ~operation() override { (void)ctx_.unpark(this); }

    void start() noexcept {
      // a send needs a header (ucx_am_context.hpp:2275-2278)
      if (!view_->header.data || view_->header.size == 0) return fail(AXR_ERR_INVALID);
      int rc;
      if constexpr (std::is_same_v<View, ucx_am_data>) {
        const axr_am_data_t d = to_abi(*view_);
        rc = axr_am_send(ctx_.handle(), conn_, &d, ctx_.stream(), &request_);
      } else {
        axr_am_iovec_t d;
        d.header = axr_buffer_t{view_->header.data, view_->header.size};
        d.buffer_vec = reinterpret_cast<axr_buffer_t*>(view_->buffer_vec);
        d.buffer_count = view_->buffer_count;
        d.buffer_type = static_cast<int>(view_->buffer_type);
        d.mem_h = view_->mem_h;
        rc = axr_am_send_iov(ctx_.handle(), conn_, &d, ctx_.stream(), &request_);
      }
      if (rc) return fail(rc);
      started_ = true;
      if (!poll()) ctx_.park(this);
    }

    // The sender-side stop request: a send that the receiver has not begun to fetch is
    // withdrawn and the receiver is completed with set_done().
    void request_stop() noexcept {
      if (!started_ || completed_) return;
      (void)axr_am_request_cancel(ctx_.handle(), request_);
      if (poll()) (void)ctx_.unpark(this);
    }

   private:
    bool poll() override {
      if (completed_) return true;
      int done = 0;
      const int rc = axr_am_request_test(ctx_.handle(), request_, &done);
      if (rc) {
        complete_error(rc);
        return true;
      }
      if (done == 0) return false;
      completed_ = true;
      owned_.reset();   // an owned payload lives exactly until the send has completed
      if (done > 0) std::move(receiver_).set_value();
      else std::move(receiver_).set_done();
      return true;
    }
    void fail(int rc) noexcept { complete_error(rc); }
    void complete_error(int rc) {
      completed_ = true;
      owned_.reset();
      std::move(receiver_).set_error(status_to_error(rc));
    }

    loopback_am_context& ctx_;
    std::uint64_t conn_;
    std::optional<Owned> owned_;
    View* view_;
    Receiver receiver_;
    std::uint64_t request_ = 0;
    bool started_ = false, completed_ = false;
  };

  template <typename Receiver>
  operation<std::decay_t<Receiver>> connect(Receiver&& r) && {
    return operation<std::decay_t<Receiver>>(std::move(*this), std::decay_t<Receiver>(std::forward<Receiver>(r)));
  }

 private:
  loopback_am_context& ctx_;
  std::uint64_t conn_;
  std::optional<Owned> owned_;
  View* view_;
};

// ------------------------------------------------------------ receive pieces

// Fetch of a rendezvous payload into `buffer` the way recv_buffer_sender_t<UcxBuffer> does:
// a null or too small buffer is released and allocated again from the context's memory
// resource with the buffer's own memory type, and its size becomes the message's
// (ucx_am_context.hpp:1604-1621).
inline int fetch_into(loopback_am_context& ctx, std::uint64_t key, size_t data_length, ucx_memory_type_t type,
                      ucx_buffer_t* buffer) {
  const bool reallocate = !buffer->data || buffer->size < data_length;
  if (reallocate && buffer->data) ctx.memory_resource().deallocate(type, buffer->data, buffer->size);
  if (reallocate) {
    buffer->data = nullptr;   // nothing to release twice if the allocation throws
    buffer->size = 0;
    buffer->data = ctx.memory_resource().allocate(type, data_length);
  }
  buffer->size = data_length;
  return axr_am_recv_buffer(ctx.handle(), key, static_cast<int>(type), buffer->data, buffer->size, ctx.stream());
}

// ------------------------------------------------------------ connection_recv_header

// ucx_am_context.hpp:1846-2232: the next message in arrival order.  A rendezvous message
// with a payload yields its key and the header; anything else (an eager message, a message
// without payload) yields the complete bundle, its payload in host memory.
class recv_header_sender {
 public:
  explicit recv_header_sender(loopback_am_context& ctx) : ctx_(ctx) {}

  template <typename Receiver>
  class operation final : private parked_operation {
   public:
    operation(loopback_am_context& ctx, Receiver&& r) : ctx_(ctx), receiver_(std::move(r)) {}
    operation(const operation&) = delete;
    operation& operator=(const operation&) = delete;
    ~operation() override { (void)ctx_.unpark(this); }

    void start() noexcept {
      if (!poll()) ctx_.park(this);   // no message yet: wait for one (pendingRecvIoQueue_)
    }
    // Only a receive that is still waiting for a message can be stopped (:2021-2033).
    void request_stop() noexcept {
      if (completed_ || !ctx_.unpark(this)) return;
      completed_ = true;
      std::move(receiver_).set_done();
    }

   private:
    bool poll() override {
      if (completed_) return true;
      axr_am_message_t m;
      const int rc = axr_am_recv_header(ctx_.handle(), &m);
      if (rc == AXR_ERR_NO_MESSAGE) return false;
      completed_ = true;
      if (rc) {
        std::move(receiver_).set_error(status_to_error(rc));
        return true;
      }
      try {
        UcxHeader header = copy_header(ctx_, m);
        const LoopbackConnection conn(m.conn_id);
        if (m.is_rndv && m.data_length > 0) {
          std::move(receiver_).set_value(
              recv_header_result_type(std::in_place_index<0>, static_cast<size_t>(m.key), std::move(header)));
          return true;
        }
        // eager: the payload is host memory that the transport holds; the buffer hands it
        // back through its release function, as the reference does with ucp_am_data_release
        // (:1969-1986).  No payload: an empty buffer.
        axr_am_context_t* handle = ctx_.handle();
        const std::uint64_t key = m.key;
        UcxBuffer buffer =
            m.eager_data.size
                ? UcxBuffer(ctx_.mr(), ucx_memory_type::HOST, ucx_buffer_t{m.eager_data.data, m.eager_data.size},
                            nullptr, /*own_buffer=*/true,
                            [handle, key](void*) { (void)axr_am_message_release(handle, key); })
                : UcxBuffer(ctx_.mr(), ucx_memory_type::HOST, 0, nullptr, /*own_buffer=*/true);
        if (!m.eager_data.size) (void)axr_am_message_release(handle, key);
        std::move(receiver_).set_value(recv_header_result_type(
            std::in_place_index<1>, active_message_header_buffer_bundle(std::move(header), std::move(buffer), conn)));
      } catch (const std::bad_alloc&) {
        (void)axr_am_message_release(ctx_.handle(), m.key);
        std::move(receiver_).set_error(make_error_code(am_errc::no_memory));
      } catch (...) {
        (void)axr_am_message_release(ctx_.handle(), m.key);
        std::move(receiver_).set_error(make_error_code(am_errc::no_message));   // UNIFEX_CATCH(...) of :2012
      }
      return true;
    }

    loopback_am_context& ctx_;
    Receiver receiver_;
    bool completed_ = false;
  };

  template <typename Receiver>
  operation<std::decay_t<Receiver>> connect(Receiver&& r) && {
    return operation<std::decay_t<Receiver>>(ctx_, std::decay_t<Receiver>(std::forward<Receiver>(r)));
  }

 private:
  loopback_am_context& ctx_;
};

// ------------------------------------------------------------ connection_recv_buffer

// ucx_am_context.hpp:1511-1844.  Unknown key: UCS_ERR_NO_MESSAGE (:1570-1574).  Key of a
// message whose payload came with its header: UCS_ERR_NOT_IMPLEMENTED (:1643-1651).
template <typename BufferType>
class recv_buffer_sender {
 public:
  recv_buffer_sender(loopback_am_context& ctx, size_t key, BufferType&& buffer)
      : ctx_(ctx), key_(key), buffer_(std::move(buffer)) {}

  template <typename Receiver>
  class operation final {
   public:
    operation(loopback_am_context& ctx, size_t key, BufferType&& buffer, Receiver&& r)
        : ctx_(ctx), key_(key), buffer_(std::move(buffer)), receiver_(std::move(r)) {}
    operation(const operation&) = delete;
    operation& operator=(const operation&) = delete;

    void start() noexcept {
      if (stopped_) return std::move(receiver_).set_done();
      int rc = AXR_OK;
      try {
        if constexpr (std::is_same_v<BufferType, UcxBuffer>) {
          size_t length = 0;
          rc = probe(&length);
          if (rc == AXR_OK)
            rc = fetch_into(ctx_, key_, length, buffer_.type(), buffer_.get());
        } else {
          // every entry allocated and non-empty (:1808-1818); entries are filled in order
          if (buffer_.size() == 0) rc = AXR_ERR_INVALID;
          for (size_t i = 0; i < buffer_.size() && rc == AXR_OK; ++i)
            if (!buffer_[i].data || buffer_[i].size == 0) rc = AXR_ERR_INVALID;
          size_t length = 0;
          if (rc == AXR_OK) rc = probe(&length);
          if (rc == AXR_OK)
            rc = axr_am_recv_buffer_iov(ctx_.handle(), key_, static_cast<int>(buffer_.type()),
                                        reinterpret_cast<const axr_buffer_t*>(buffer_.data()), buffer_.size(),
                                        ctx_.stream());
        }
      } catch (const std::bad_alloc&) {
        rc = AXR_ERR_NOMEM;
      } catch (...) {
        rc = AXR_ERR_NO_MESSAGE;   // UNIFEX_CATCH(...) of :1654
      }
      if (rc == AXR_ERR_CANCELED) return std::move(receiver_).set_done();
      if (rc) return std::move(receiver_).set_error(status_to_error(rc));
      std::move(receiver_).set_value(
          active_message_buffer_bundle_t<BufferType>(std::move(buffer_), LoopbackConnection(conn_)));
    }
    // Before start(): the operation completes with set_done() and the message stays parked.
    void request_stop() noexcept { stopped_ = true; }

   private:
    // Length of the parked rendezvous message `key_`, from the parked descriptor.
    int probe(size_t* length) {
      uint64_t n = 0;
      int is_rndv = 0;
      const int rc = axr_am_message_info(ctx_.handle(), key_, &n, &conn_, &is_rndv);
      if (rc) return rc;                                // unknown key: UCS_ERR_NO_MESSAGE
      if (!is_rndv) return AXR_ERR_NOT_IMPLEMENTED;     // its payload came with the header
      *length = static_cast<size_t>(n);
      return AXR_OK;
    }

    loopback_am_context& ctx_;
    size_t key_;
    BufferType buffer_;
    Receiver receiver_;
    std::uint64_t conn_ = 0;
    bool stopped_ = false;
  };

  template <typename Receiver>
  operation<std::decay_t<Receiver>> connect(Receiver&& r) && {
    return operation<std::decay_t<Receiver>>(ctx_, key_, std::move(buffer_),
                                             std::decay_t<Receiver>(std::forward<Receiver>(r)));
  }

 private:
  loopback_am_context& ctx_;
  size_t key_;
  BufferType buffer_;
};

// ------------------------------------------------------------ connection_recv

// ucx_am_context.hpp:1075-1509: header and payload of the next message in one step.  The
// borrowed form fills the caller's ucx_am_data (its header must be {nullptr, 0}, :1092-1095;
// a null or too small buffer is replaced by one from the memory resource, :1204-1213); the
// owning form allocates everything.  Eager payloads arrive in host memory and are copied to
// the requested memory type with the resource's memcpy (:1258-1260).
class recv_sender {
 public:
  recv_sender(loopback_am_context& ctx, ucx_am_data& borrowed) : ctx_(ctx), borrowed_(&borrowed) {}
  recv_sender(loopback_am_context& ctx, ucx_memory_type type) : ctx_(ctx), borrowed_(nullptr), type_(type) {}

  template <typename Receiver>
  class operation final : private parked_operation {
   public:
    operation(loopback_am_context& ctx, ucx_am_data* borrowed, ucx_memory_type type, Receiver&& r)
        : ctx_(ctx), borrowed_(borrowed), type_(borrowed ? borrowed->buffer_type : type), receiver_(std::move(r)) {}
    operation(const operation&) = delete;
    operation& operator=(const operation&) = delete;
    ~operation() override { (void)ctx_.unpark(this); }

    void start() noexcept {
      if (borrowed_ && (borrowed_->header.data || borrowed_->header.size)) {
        completed_ = true;
        return std::move(receiver_).set_error(make_error_code(am_errc::invalid_param));
      }
      if (!poll()) ctx_.park(this);
    }
    void request_stop() noexcept {
      if (completed_ || !ctx_.unpark(this)) return;
      completed_ = true;
      std::move(receiver_).set_done();
    }

   private:
    bool poll() override {
      if (completed_) return true;
      axr_am_message_t m;
      int rc = axr_am_recv_header(ctx_.handle(), &m);
      if (rc == AXR_ERR_NO_MESSAGE) return false;
      completed_ = true;
      if (rc) {
        std::move(receiver_).set_error(status_to_error(rc));
        return true;
      }
      UcxMemoryResourceManager& mr = ctx_.memory_resource();
      ucx_am_data data;
      std::memset(&data, 0, sizeof(data));
      data.buffer_type = type_;
      if (borrowed_) data = *borrowed_;
      bool own_buffer = !borrowed_;
      try {
        data.header.data = m.header.size ? mr.allocate(ucx_memory_type::HOST, m.header.size) : nullptr;
        data.header.size = m.header.size;
        if (m.header.size) std::memcpy(data.header.data, m.header.data, m.header.size);
        if (m.is_rndv && m.data_length > 0) {
          rc = fetch_into(ctx_, m.key, m.data_length, type_, &data.buffer);
        } else if (m.data_length > 0) {
          const bool reallocate = !data.buffer.data || data.buffer.size < m.data_length;
          if (reallocate && data.buffer.data) mr.deallocate(type_, data.buffer.data, data.buffer.size);
          if (reallocate) data.buffer.data = mr.allocate(type_, m.data_length);
          data.buffer.size = m.data_length;
          mr.memcpy(type_, data.buffer.data, ucx_memory_type::HOST, m.eager_data.data, m.data_length);
          (void)axr_am_message_release(ctx_.handle(), m.key);
        } else {
          data.buffer.size = 0;
          (void)axr_am_message_release(ctx_.handle(), m.key);
        }
      } catch (const std::bad_alloc&) {
        rc = AXR_ERR_NOMEM;
      } catch (...) {
        rc = AXR_ERR_NO_MESSAGE;
      }
      if (borrowed_) *borrowed_ = data;   // the caller sees (and owns) what was allocated, also on failure
      if (rc) {
        if (!borrowed_) {
          if (data.header.data) mr.deallocate(ucx_memory_type::HOST, data.header.data, data.header.size);
          if (data.buffer.data) mr.deallocate(type_, data.buffer.data, data.buffer.size);
        }
        (void)axr_am_message_release(ctx_.handle(), m.key);
        if (rc == AXR_ERR_CANCELED) std::move(receiver_).set_done();
        else std::move(receiver_).set_error(status_to_error(rc));
        return true;
      }
      // borrowed: a view of the caller's descriptor; owning: header and buffer belong to the bundle
      UcxAmData wrapper = borrowed_ ? UcxAmData(ctx_.mr(), data, /*own_header=*/false, /*own_buffer=*/false)
                                    : UcxAmData(ctx_.mr(), std::move(data), /*own_header=*/true, own_buffer);
      std::move(receiver_).set_value(active_message_bundle(std::move(wrapper), LoopbackConnection(m.conn_id)));
      return true;
    }

    loopback_am_context& ctx_;
    ucx_am_data* borrowed_;
    ucx_memory_type type_;
    Receiver receiver_;
    bool completed_ = false;
  };

  template <typename Receiver>
  operation<std::decay_t<Receiver>> connect(Receiver&& r) && {
    return operation<std::decay_t<Receiver>>(ctx_, borrowed_, type_, std::decay_t<Receiver>(std::forward<Receiver>(r)));
  }

 private:
  loopback_am_context& ctx_;
  ucx_am_data* borrowed_;
  ucx_memory_type type_ = ucx_memory_type::HOST;
};

}  // namespace detail

// ---------------------------------------------------------------- the customisation points

// connection_send: ucx_context_concept.hpp:247-289.  `conn` is a connection id or a
// LoopbackConnection.  The sender completes with set_value() when the payload may be
// reused: at once for an eager message, after the receiver's fetch for a rendezvous.
template <typename Conn>
auto connection_send(scheduler sched, Conn&& conn, ucx_am_data& data) {
  return detail::send_sender<UcxAmData, ucx_am_data>(sched.context(), detail::conn_id_of(conn), data);
}
template <typename Conn>
auto connection_send(scheduler sched, Conn&& conn, UcxAmData&& data) {
  return detail::send_sender<UcxAmData, ucx_am_data>(sched.context(), detail::conn_id_of(conn), std::move(data));
}
template <typename Conn>
auto connection_send(scheduler sched, Conn&& conn, ucx_am_iovec& data) {
  return detail::send_sender<UcxAmIovec, ucx_am_iovec>(sched.context(), detail::conn_id_of(conn), data);
}
template <typename Conn>
auto connection_send(scheduler sched, Conn&& conn, UcxAmIovec&& data) {
  return detail::send_sender<UcxAmIovec, ucx_am_iovec>(sched.context(), detail::conn_id_of(conn), std::move(data));
}

// connection_recv: ucx_context_concept.hpp:291-327.
inline auto connection_recv(scheduler sched, ucx_am_data& data) { return detail::recv_sender(sched.context(), data); }
inline auto connection_recv(scheduler sched, ucx_memory_type type) { return detail::recv_sender(sched.context(), type); }

// connection_recv_header: ucx_context_concept.hpp:329-377.
inline auto connection_recv_header(scheduler sched) { return detail::recv_header_sender(sched.context()); }

// connection_recv_buffer: ucx_context_concept.hpp:379-470.
inline auto connection_recv_buffer(scheduler sched, size_t key, UcxBuffer&& buffer) {
  return detail::recv_buffer_sender<UcxBuffer>(sched.context(), key, std::move(buffer));
}
inline auto connection_recv_buffer(scheduler sched, size_t key, UcxBufferVec&& buffers) {
  return detail::recv_buffer_sender<UcxBufferVec>(sched.context(), key, std::move(buffers));
}
inline auto connection_recv_buffer(scheduler sched, size_t key, ucx_memory_type type) {
  // allocated from the memory resource once the length is known (:1822-1828)
  return detail::recv_buffer_sender<UcxBuffer>(sched.context(), key,
                                               UcxBuffer(sched.context().mr(), type, 0, nullptr, /*own_buffer=*/true));
}

// ---------------------------------------------------------------- sync_wait

// Starts `sender` and turns the context's progress loop until it has completed.  Returns the
// value (std::optional, empty after set_done()); set_error becomes std::system_error.
// `also` names other contexts whose progress the completion depends on (the peer of a
// rendezvous send).  An operation that has not completed after `limit` is stopped and the
// wait ends with std::errc::timed_out: a wait for something that nobody will ever send must
// not spin for ever.
namespace detail {
template <typename T>
struct wait_state {
  std::optional<T> value;
  std::error_code error;
  bool done = false, finished = false;
};
template <typename T>
struct wait_receiver {
  wait_state<T>* st;
  template <typename... A>
  void set_value(A&&... a) && {
    st->value.emplace(std::forward<A>(a)...);
    st->finished = true;
  }
  void set_error(std::error_code ec) && {
    st->error = ec;
    st->finished = true;
  }
  void set_done() && {
    st->done = true;
    st->finished = true;
  }
};
struct unit {};
}  // namespace detail

template <typename T, typename Sender>
std::optional<T> sync_wait(loopback_am_context& ctx, Sender&& sender,
                           std::initializer_list<loopback_am_context*> also = {},
                           std::chrono::milliseconds limit = std::chrono::seconds(30)) {
  detail::wait_state<T> st;
  auto op = connect(std::forward<Sender>(sender), detail::wait_receiver<T>{&st});
  op.start();
  const auto deadline = std::chrono::steady_clock::now() + limit;
  while (!st.finished) {
    ctx.progress();
    for (loopback_am_context* other : also) other->progress();
    if (!st.finished && std::chrono::steady_clock::now() > deadline) {
      op.request_stop();
      if (!st.finished || st.done) throw std::system_error(std::make_error_code(std::errc::timed_out));
    }
  }
  if (st.error) throw std::system_error(st.error);
  return std::move(st.value);
}
// For senders of no value (connection_send): true on set_value, false on set_done.
template <typename Sender>
bool sync_wait_void(loopback_am_context& ctx, Sender&& sender,
                    std::initializer_list<loopback_am_context*> also = {},
                    std::chrono::milliseconds limit = std::chrono::seconds(30)) {
  return sync_wait<detail::unit>(ctx, std::forward<Sender>(sender), also, limit).has_value();
}

}  // namespace loopback
}  // namespace ucxx
}  // namespace eux

#endif  // in the reference tree
#endif  // AXON_ROCM_LOOPBACK_AM_CONTEXT_HPP_
