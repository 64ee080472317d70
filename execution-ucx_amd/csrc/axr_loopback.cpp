// Loopback active-message context: the AM-bundle surface of the reference's
// ucx_am_context for one process without UCX.  Semantics and reference lines
// are given with the declarations in axon_rocm.h.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <set>

#include "axr_internal.h"

using namespace axr;

namespace {

struct Piece {
  const void* data;
  size_t size;
};

struct Request {
  std::atomic<int> done{0};        // 1 complete, -1 cancelled or failed
  hipEvent_t event = nullptr;      // set by an asynchronous fetch: done once it has fired
  bool claimed = false;            // a receiver has begun to fetch the payload: too late to cancel
  std::mutex mu;
  ~Request() {
    if (event) (void)hipEventDestroy(event);
  }
};

struct Message {
  uint64_t key = 0;
  uint64_t conn_id = 0;
  std::vector<uint8_t> header;
  std::vector<uint8_t> eager;
  std::vector<Piece> pieces;       // rendezvous: the sender's buffers
  uint64_t data_length = 0;
  bool rndv = false;
  int buffer_type = AXR_MEM_HOST;
  std::shared_ptr<Request> request;
};

// 0 pending, 1 complete, -1 cancelled or failed; an asynchronous fetch completes with its event.
int poll_request(Request* r) {
  int st = r->done.load();
  if (st == 0) {
    std::lock_guard<std::mutex> rl(r->mu);
    if (r->event) {
      const hipError_t q = hipEventQuery(r->event);
      if (q == hipSuccess) st = 1;
      else if (q != hipErrorNotReady) st = -1;
      if (st != 0) r->done.store(st);
    }
  }
  return st;
}

bool host_type(int t) { return t == AXR_MEM_HOST || t == AXR_MEM_ROCM_MANAGED; }
bool known_type(int t) { return host_type(t) || t == AXR_MEM_ROCM; }

constexpr size_t kMaxInFlight = 256;

std::atomic<uint64_t> g_next_id{1};

// Contexts that exist.  An endpoint is a plain pointer to its peer; a send looks the
// peer up here (and delivers under this lock), so that a peer destroyed in the
// meantime is an error and not a dangling pointer.
std::mutex g_contexts_mu;
std::set<const void*> g_contexts;

}  // namespace

struct axr_am_context {
  std::string name;
  size_t zcopy_thresh = 4096;
  // Held from the decision "this message goes out now" until it lies in the peer's queue, in
  // deliver() and in progress(): with several sending threads the order in which messages
  // reach the peer is then the order in which that decision was taken, and a message that
  // progress() has just taken off the waiting queue cannot be overtaken by a newer send.
  // Taken before `mu`, never while `mu` is held.
  std::mutex send_mu;
  std::mutex mu;
  std::deque<std::unique_ptr<Message>> arrived;          // not yet seen by recv_header
  std::map<uint64_t, std::unique_ptr<Message>> parked;   // handed out, awaiting fetch/release
  std::map<uint64_t, std::unique_ptr<Message>> borrowed; // payload lent to the receiver, awaiting release
  std::map<uint64_t, axr_am_context*> endpoints;         // conn id -> peer
  std::map<uint64_t, std::shared_ptr<Request>> requests;
  // Sends that have started and not completed (rendezvous sends whose payload has not been
  // fetched): at most kMaxInFlight, as the reference's context admits 256 operations
  // (kCompletionQueueEntryCount, ucx_am_context.hpp:94,836-839).  Further sends wait here, in
  // order, and start as completions make room (pendingIoQueue_, ucx_am_context.cpp:271-274).
  std::vector<std::shared_ptr<Request>> in_flight;
  struct Waiting {
    uint64_t conn_id;
    std::unique_ptr<Message> message;
  };
  std::deque<Waiting> waiting;
};

namespace {

size_t env_zcopy_thresh() {
  const char* val = std::getenv("UCX_ZCOPY_THRESH");
  if (!val) return 4096;
  char* end = nullptr;
  const long long v = std::strtoll(val, &end, 10);
  if (end == val || v <= 0) return 4096;
  return static_cast<size_t>(v);
}

int copy_piece(int dst_type, void* dst, int src_type, const void* src, size_t n, hipStream_t s) {
  if (n == 0) return AXR_OK;
  if (host_type(dst_type) && host_type(src_type)) {
    std::memcpy(dst, src, n);
    return AXR_OK;
  }
  if (dst_type == AXR_MEM_ROCM && src_type == AXR_MEM_ROCM && tunables().loopback_copy_kernel != 0) {
    // same GPU on both sides: the copy kernel (cacheable while the payload fits the last-level
    // cache, as the bundle kernels treat a payload)
    // (source and destination both take room there)
    const bool nt = 2 * static_cast<uint64_t>(n) > static_cast<uint64_t>(tunables().payload_cache_bytes);
    return launch_stream_copy(dst, src, n, nt, s);
  }
  return check_hip(hipMemcpyAsync(dst, src, n, hipMemcpyDefault, s), "hipMemcpyAsync(loopback)");
}

// Puts the message into the peer's arrival queue.  ctx->mu is NOT held.
int hand_over(axr_am_context* peer, std::unique_ptr<Message> m) {
  std::lock_guard<std::mutex> alive(g_contexts_mu);
  if (!g_contexts.count(peer)) {
    m->request->done.store(-1);
    return fail(AXR_ERR_INVALID, "the connection's peer context has been destroyed");
  }
  std::lock_guard<std::mutex> lock(peer->mu);
  peer->arrived.push_back(std::move(m));
  return AXR_OK;
}

// Forgets completed sends and starts waiting ones while there is room, in order.
// ctx->send_mu is held by the caller.
void progress_locked(axr_am_context* ctx) {
  for (;;) {
    axr_am_context* peer = nullptr;
    std::unique_ptr<Message> m;
    {
      std::lock_guard<std::mutex> lock(ctx->mu);
      auto& fl = ctx->in_flight;
      fl.erase(std::remove_if(fl.begin(), fl.end(),
                              [](const std::shared_ptr<Request>& r) { return poll_request(r.get()) != 0; }),
               fl.end());
      // cancelled while waiting: dropped without ever reaching the peer
      ctx->waiting.erase(std::remove_if(ctx->waiting.begin(), ctx->waiting.end(),
                                        [](const axr_am_context::Waiting& w) {
                                          return w.message->request->done.load() == -1;
                                        }),
                         ctx->waiting.end());
      if (ctx->waiting.empty()) return;
      Message* front = ctx->waiting.front().message.get();
      const bool counts = front->rndv;
      if (counts && fl.size() >= kMaxInFlight) return;
      auto it = ctx->endpoints.find(ctx->waiting.front().conn_id);
      peer = it == ctx->endpoints.end() ? nullptr : it->second;
      m = std::move(ctx->waiting.front().message);
      ctx->waiting.pop_front();
      if (counts) fl.push_back(m->request);
    }
    if (!peer) {
      m->request->done.store(-1);
      continue;
    }
    (void)hand_over(peer, std::move(m));   // a destroyed peer fails the request; the rest goes on
  }
}

void progress(axr_am_context* ctx) {
  std::lock_guard<std::mutex> order(ctx->send_mu);
  progress_locked(ctx);
}

int deliver(axr_am_context* ctx, uint64_t conn_id, std::unique_ptr<Message> m, uint64_t* request) {
  std::lock_guard<std::mutex> order(ctx->send_mu);
  progress_locked(ctx);
  axr_am_context* peer = nullptr;
  bool wait = false;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->endpoints.find(conn_id);
    if (it == ctx->endpoints.end()) return fail(AXR_ERR_INVALID, "unknown connection id");
    peer = it->second;
    const uint64_t rid = g_next_id++;
    ctx->requests[rid] = m->request;
    if (request) *request = rid;
    m->key = g_next_id++;
    m->conn_id = conn_id;
    // behind sends that wait (order is kept), or when the context is full
    wait = !ctx->waiting.empty() || (m->rndv && ctx->in_flight.size() >= kMaxInFlight);
    if (wait) {
      ctx->waiting.push_back({conn_id, std::move(m)});
    } else if (m->rndv) {
      ctx->in_flight.push_back(m->request);
    }
  }
  if (wait) return AXR_OK;
  return hand_over(peer, std::move(m));
}

}  // namespace

extern "C" {

static int am_context_create_body(const char* name, size_t zcopy_thresh, axr_am_context_t** ctx) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_context_create: null result");
  axr_am_context* c = new (std::nothrow) axr_am_context();
  if (!c) return fail(AXR_ERR_NOMEM, "axr_am_context_create: out of host memory");
  c->name = name ? name : "";
  c->zcopy_thresh = zcopy_thresh ? zcopy_thresh : env_zcopy_thresh();
  {
    std::lock_guard<std::mutex> alive(g_contexts_mu);
    g_contexts.insert(c);
  }
  *ctx = c;
  return AXR_OK;
}
int axr_am_context_create(const char* name, size_t zcopy_thresh, axr_am_context_t** ctx) {
  return guarded([&] { return am_context_create_body(name, zcopy_thresh, ctx); });
}

static int am_context_destroy_body(axr_am_context_t* ctx) {
  if (!ctx) return AXR_OK;
  {
    std::lock_guard<std::mutex> alive(g_contexts_mu);   // no delivery is under way past this
    g_contexts.erase(ctx);
  }
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    for (auto& m : ctx->arrived) m->request->done.store(-1);
    for (auto& kv : ctx->parked) kv.second->request->done.store(-1);
    for (auto& kv : ctx->borrowed) kv.second->request->done.store(1);   // the receiver is gone: nothing reads on
    for (auto& w : ctx->waiting) w.message->request->done.store(-1);
  }
  delete ctx;
  return AXR_OK;
}
int axr_am_context_destroy(axr_am_context_t* ctx) {
  return guarded([&] { return am_context_destroy_body(ctx); });
}

static int am_connect_body(axr_am_context_t* from, axr_am_context_t* to, uint64_t* conn_id) {
  if (!from || !to || !conn_id) return fail(AXR_ERR_INVALID, "axr_am_connect: null argument");
  const uint64_t id = g_next_id++;
  std::lock_guard<std::mutex> lock(from->mu);
  from->endpoints[id] = to;
  *conn_id = id;
  return AXR_OK;
}
int axr_am_connect(axr_am_context_t* from, axr_am_context_t* to, uint64_t* conn_id) {
  return guarded([&] { return am_connect_body(from, to, conn_id); });
}

static int am_send_body(axr_am_context_t* ctx, uint64_t conn_id, const axr_am_data_t* d,
                        void* stream, uint64_t* request) {
  if (!ctx || !d) return fail(AXR_ERR_INVALID, "axr_am_send: null argument");
  if (!d->header.data || d->header.size == 0)
    return fail(AXR_ERR_INVALID, "axr_am_send: the header must not be empty");
  if ((d->buffer.data == nullptr) != (d->buffer.size == 0))
    return fail(AXR_ERR_INVALID, "axr_am_send: buffer pointer and size disagree");
  if (!known_type(d->buffer_type)) return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory type");
  std::unique_ptr<Message> m(new Message());
  m->request = std::make_shared<Request>();
  const uint8_t* h = static_cast<const uint8_t*>(d->header.data);
  m->header.assign(h, h + d->header.size);
  m->data_length = d->buffer.size;
  m->buffer_type = d->buffer_type;
  // a zero-length rendezvous is treated as eager (ucx_am_context.hpp:1955-1958)
  m->rndv = d->buffer.size >= ctx->zcopy_thresh && d->buffer.size > 0;
  if (m->rndv) {
    m->pieces.push_back({d->buffer.data, d->buffer.size});
  } else {
    m->eager.resize(d->buffer.size);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = copy_piece(AXR_MEM_HOST, m->eager.data(), d->buffer_type, d->buffer.data,
                        d->buffer.size, s);
    if (rc) return rc;
    if (!host_type(d->buffer_type) && d->buffer.size) {
      rc = check_hip(hipStreamSynchronize(s), "hipStreamSynchronize");
      if (rc) return rc;
    }
    m->request->done.store(1);   // eager: the sender's buffer is free again
  }
  return deliver(ctx, conn_id, std::move(m), request);
}
int axr_am_send(axr_am_context_t* ctx,
                uint64_t conn_id,
                const axr_am_data_t* d,
                void* stream,
                uint64_t* request) {
  return guarded([&] { return am_send_body(ctx, conn_id, d, stream, request); });
}

static int am_send_iov_body(axr_am_context_t* ctx, uint64_t conn_id, const axr_am_iovec_t* d,
                            void* stream, uint64_t* request) {
  if (!ctx || !d) return fail(AXR_ERR_INVALID, "axr_am_send_iov: null argument");
  if (!d->header.data || d->header.size == 0)
    return fail(AXR_ERR_INVALID, "axr_am_send_iov: the header must not be empty");
  if ((d->buffer_vec == nullptr) != (d->buffer_count == 0))
    return fail(AXR_ERR_INVALID, "axr_am_send_iov: buffer vector and count disagree");
  if (!known_type(d->buffer_type)) return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory type");
  std::unique_ptr<Message> m(new Message());
  m->request = std::make_shared<Request>();
  const uint8_t* h = static_cast<const uint8_t*>(d->header.data);
  m->header.assign(h, h + d->header.size);
  m->buffer_type = d->buffer_type;
  for (size_t i = 0; i < d->buffer_count; ++i) {
    if (d->buffer_vec[i].size && !d->buffer_vec[i].data)
      return fail(AXR_ERR_INVALID, "axr_am_send_iov: null entry with a size");
    m->pieces.push_back({d->buffer_vec[i].data, d->buffer_vec[i].size});
    m->data_length += d->buffer_vec[i].size;
  }
  m->rndv = m->data_length > 0;   // always rendezvous; nothing to fetch when empty
  if (!m->rndv) m->request->done.store(1);
  return deliver(ctx, conn_id, std::move(m), request);
}
int axr_am_send_iov(axr_am_context_t* ctx,
                    uint64_t conn_id,
                    const axr_am_iovec_t* d,
                    void* stream,
                    uint64_t* request) {
  return guarded([&] { return am_send_iov_body(ctx, conn_id, d, stream, request); });
}

static int am_request_test_body(axr_am_context_t* ctx, uint64_t request, int* done) {
  if (!ctx || !done) return fail(AXR_ERR_INVALID, "axr_am_request_test: null argument");
  progress(ctx);
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->requests.find(request);
  if (it == ctx->requests.end()) return fail(AXR_ERR_INVALID, "axr_am_request_test: unknown request");
  const int st = poll_request(it->second.get());
  *done = st;
  if (st != 0) ctx->requests.erase(it);
  return AXR_OK;
}
int axr_am_request_test(axr_am_context_t* ctx, uint64_t request, int* done) {
  return guarded([&] { return am_request_test_body(ctx, request, done); });
}

static int am_recv_header_body(axr_am_context_t* ctx, axr_am_message_t* out) {
  if (!ctx || !out) return fail(AXR_ERR_INVALID, "axr_am_recv_header: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  // a rendezvous whose sender has cancelled it in the meantime never shows up
  while (!ctx->arrived.empty() && ctx->arrived.front()->rndv && ctx->arrived.front()->request->done.load() == -1)
    ctx->arrived.pop_front();
  if (ctx->arrived.empty()) return fail(AXR_ERR_NO_MESSAGE, "no message queued");
  std::unique_ptr<Message> m = std::move(ctx->arrived.front());
  ctx->arrived.pop_front();
  std::memset(out, 0, sizeof(*out));
  out->key = m->key;
  out->conn_id = m->conn_id;
  out->header = axr_buffer_t{m->header.data(), m->header.size()};
  out->data_length = m->data_length;
  out->is_rndv = m->rndv ? 1 : 0;
  out->buffer_type = m->buffer_type;
  if (!m->rndv) out->eager_data = axr_buffer_t{m->eager.empty() ? nullptr : m->eager.data(), m->eager.size()};
  const uint64_t key = m->key;
  ctx->parked[key] = std::move(m);
  return AXR_OK;
}
int axr_am_recv_header(axr_am_context_t* ctx, axr_am_message_t* out) {
  return guarded([&] { return am_recv_header_body(ctx, out); });
}

static int fetch(axr_am_context_t* ctx, uint64_t key, int dst_type, const axr_buffer_t* vec,
                 size_t count, void* stream, bool wait = true) {
  if (!known_type(dst_type)) return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory type");
  std::unique_ptr<Message> m;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->parked.find(key);
    if (it == ctx->parked.end()) return fail(AXR_ERR_NO_MESSAGE, "no message with this key");
    if (!it->second->rndv)
      return fail(AXR_ERR_NOT_IMPLEMENTED, "message was eager: its data came with the header");
    {
      // claim the payload, unless the sender has cancelled the send in the meantime
      Request* r = it->second->request.get();
      std::lock_guard<std::mutex> rl(r->mu);
      if (r->done.load() == -1) {
        ctx->parked.erase(it);
        return fail(AXR_ERR_CANCELED, "the sender cancelled this message");
      }
      r->claimed = true;
    }
    uint64_t room = 0;
    for (size_t i = 0; i < count; ++i) room += vec[i].size;
    if (room < it->second->data_length)
      return fail(AXR_ERR_LENGTH, "receive buffer is smaller than the message");
    m = std::move(it->second);
    ctx->parked.erase(it);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // stream the sender's pieces, in order, into the receiver's entries, in order
  size_t di = 0, doff = 0;
  int rc = AXR_OK;
  bool device_copy = false;
  for (const Piece& p : m->pieces) {
    size_t poff = 0;
    while (poff < p.size && rc == AXR_OK) {
      while (doff == vec[di].size) {
        ++di;
        doff = 0;
      }
      const size_t n = std::min(p.size - poff, vec[di].size - doff);
      rc = copy_piece(dst_type, static_cast<uint8_t*>(vec[di].data) + doff, m->buffer_type,
                      static_cast<const uint8_t*>(p.data) + poff, n, s);
      device_copy = device_copy || !(host_type(dst_type) && host_type(m->buffer_type));
      poff += n;
      doff += n;
    }
    if (rc) break;
  }
  if (rc == AXR_OK && device_copy && !wait) {
    // completion of the send = completion of the copies just enqueued
    std::lock_guard<std::mutex> lock(m->request->mu);
    rc = check_hip(hipEventCreateWithFlags(&m->request->event, hipEventDisableTiming), "hipEventCreate");
    if (rc == AXR_OK) rc = check_hip(hipEventRecord(m->request->event, s), "hipEventRecord");
    if (rc != AXR_OK) m->request->done.store(-1);
    return rc;
  }
  if (rc == AXR_OK && device_copy) rc = check_hip(hipStreamSynchronize(s), "hipStreamSynchronize");
  m->request->done.store(rc == AXR_OK ? 1 : -1);
  return rc;
}

static int am_recv_buffer_body(axr_am_context_t* ctx, uint64_t key, int dst_type, void* dst,
                               size_t dst_bytes, void* stream) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_recv_buffer: null context");
  if (!dst && dst_bytes) return fail(AXR_ERR_INVALID, "axr_am_recv_buffer: null buffer");
  axr_buffer_t one{dst, dst_bytes};
  return fetch(ctx, key, dst_type, &one, 1, stream);
}
int axr_am_recv_buffer(axr_am_context_t* ctx,
                       uint64_t key,
                       int dst_type,
                       void* dst,
                       size_t dst_bytes,
                       void* stream) {
  return guarded([&] { return am_recv_buffer_body(ctx, key, dst_type, dst, dst_bytes, stream); });
}

static int am_recv_buffer_async_body(axr_am_context_t* ctx, uint64_t key, int dst_type, void* dst,
                                     size_t dst_bytes, void* stream) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_recv_buffer_async: null context");
  if (!dst && dst_bytes) return fail(AXR_ERR_INVALID, "axr_am_recv_buffer_async: null buffer");
  axr_buffer_t one{dst, dst_bytes};
  return fetch(ctx, key, dst_type, &one, 1, stream, /*wait=*/false);
}
int axr_am_recv_buffer_async(axr_am_context_t* ctx,
                             uint64_t key,
                             int dst_type,
                             void* dst,
                             size_t dst_bytes,
                             void* stream) {
  return guarded([&] { return am_recv_buffer_async_body(ctx, key, dst_type, dst, dst_bytes,
                 stream); });
}

static int am_recv_buffer_iov_body(axr_am_context_t* ctx, uint64_t key, int dst_type,
                                   const axr_buffer_t* buffer_vec, size_t buffer_count,
                                   void* stream) {
  if (!ctx || !buffer_vec || buffer_count == 0)
    return fail(AXR_ERR_INVALID, "axr_am_recv_buffer_iov: null or empty buffer vector");
  for (size_t i = 0; i < buffer_count; ++i) {
    if (!buffer_vec[i].data || buffer_vec[i].size == 0)
      return fail(AXR_ERR_INVALID, "axr_am_recv_buffer_iov: every entry must be allocated and non-empty");
  }
  return fetch(ctx, key, dst_type, buffer_vec, buffer_count, stream);
}
int axr_am_recv_buffer_iov(axr_am_context_t* ctx,
                           uint64_t key,
                           int dst_type,
                           const axr_buffer_t* buffer_vec,
                           size_t buffer_count,
                           void* stream) {
  return guarded([&] { return am_recv_buffer_iov_body(ctx, key, dst_type, buffer_vec, buffer_count,
                 stream); });
}

static int am_recv_buffer_borrow_body(axr_am_context_t* ctx, uint64_t key, void** data, size_t* bytes,
                                      int* memory_type) {
  if (!ctx || !data || !bytes) return fail(AXR_ERR_INVALID, "axr_am_recv_buffer_borrow: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->parked.find(key);
  if (it == ctx->parked.end()) return fail(AXR_ERR_NO_MESSAGE, "no message with this key");
  Message* m = it->second.get();
  if (!m->rndv) return fail(AXR_ERR_NOT_IMPLEMENTED, "message was eager: its data came with the header");
  if (m->pieces.size() != 1)
    return fail(AXR_ERR_UNSUPPORTED, "only a contiguous payload can be borrowed: fetch an iov message with a copy");
  {
    Request* r = m->request.get();
    std::lock_guard<std::mutex> rl(r->mu);
    if (r->done.load() == -1) {
      ctx->parked.erase(it);
      return fail(AXR_ERR_CANCELED, "the sender cancelled this message");
    }
    r->claimed = true;
  }
  *data = const_cast<void*>(m->pieces[0].data);
  *bytes = m->pieces[0].size;
  if (memory_type) *memory_type = m->buffer_type;
  ctx->borrowed[key] = std::move(it->second);
  ctx->parked.erase(it);
  return AXR_OK;
}
int axr_am_recv_buffer_borrow(axr_am_context_t* ctx, uint64_t key, void** data, size_t* bytes, int* memory_type) {
  return guarded([&] { return am_recv_buffer_borrow_body(ctx, key, data, bytes, memory_type); });
}

static int am_borrow_release_body(axr_am_context_t* ctx, uint64_t key, void* stream) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_borrow_release: null context");
  std::unique_ptr<Message> m;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->borrowed.find(key);
    if (it == ctx->borrowed.end()) return fail(AXR_ERR_NO_MESSAGE, "no borrowed message with this key");
    m = std::move(it->second);
    ctx->borrowed.erase(it);
  }
  if (host_type(m->buffer_type)) {   // host readers have read by the time they say so
    m->request->done.store(1);
    return AXR_OK;
  }
  // completion of the send = completion of what the receiver's stream holds now
  std::lock_guard<std::mutex> lock(m->request->mu);
  int rc = check_hip(hipEventCreateWithFlags(&m->request->event, hipEventDisableTiming), "hipEventCreate");
  if (rc == AXR_OK) rc = check_hip(hipEventRecord(m->request->event, static_cast<hipStream_t>(stream)), "hipEventRecord");
  if (rc != AXR_OK) m->request->done.store(-1);
  return rc;
}
int axr_am_borrow_release(axr_am_context_t* ctx, uint64_t key, void* stream) {
  return guarded([&] { return am_borrow_release_body(ctx, key, stream); });
}

static int am_request_cancel_body(axr_am_context_t* ctx, uint64_t request) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_request_cancel: null context");
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->requests.find(request);
    if (it == ctx->requests.end()) return fail(AXR_ERR_INVALID, "axr_am_request_cancel: unknown request");
    // only a send that has not completed can be cancelled; the receiver then finds the message
    // gone (or fails its fetch), and the sender's buffers are its own again
    Request* r = it->second.get();
    std::lock_guard<std::mutex> rl(r->mu);
    if (!r->claimed && r->done.load() == 0) r->done.store(-1);
  }
  progress(ctx);   // room for a waiting send
  return AXR_OK;
}
int axr_am_request_cancel(axr_am_context_t* ctx, uint64_t request) {
  return guarded([&] { return am_request_cancel_body(ctx, request); });
}

static int am_progress_body(axr_am_context_t* ctx, size_t* in_flight, size_t* waiting) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_progress: null context");
  progress(ctx);
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (in_flight) *in_flight = ctx->in_flight.size();
  if (waiting) *waiting = ctx->waiting.size();
  return AXR_OK;
}
int axr_am_progress(axr_am_context_t* ctx, size_t* in_flight, size_t* waiting) {
  return guarded([&] { return am_progress_body(ctx, in_flight, waiting); });
}

static int am_message_release_body(axr_am_context_t* ctx, uint64_t key) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_message_release: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->parked.find(key);
  if (it == ctx->parked.end()) return AXR_OK;   // already fetched: nothing left to drop
  if (it->second->rndv) it->second->request->done.store(-1);
  ctx->parked.erase(it);
  return AXR_OK;
}
int axr_am_message_release(axr_am_context_t* ctx, uint64_t key) {
  return guarded([&] { return am_message_release_body(ctx, key); });
}

static int am_message_info_body(axr_am_context_t* ctx, uint64_t key, uint64_t* data_length, uint64_t* conn_id,
                                int* is_rndv) {
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_message_info: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->parked.find(key);
  if (it == ctx->parked.end()) return fail(AXR_ERR_NO_MESSAGE, "no message with this key");
  if (data_length) *data_length = it->second->data_length;
  if (conn_id) *conn_id = it->second->conn_id;
  if (is_rndv) *is_rndv = it->second->rndv ? 1 : 0;
  return AXR_OK;
}
int axr_am_message_info(axr_am_context_t* ctx, uint64_t key, uint64_t* data_length, uint64_t* conn_id, int* is_rndv) {
  return guarded([&] { return am_message_info_body(ctx, key, data_length, conn_id, is_rndv); });
}

static int am_pending_body(axr_am_context_t* ctx, size_t* count) {
  if (!ctx || !count) return fail(AXR_ERR_INVALID, "axr_am_pending: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  *count = ctx->arrived.size();
  return AXR_OK;
}
int axr_am_pending(axr_am_context_t* ctx, size_t* count) {
  return guarded([&] { return am_pending_body(ctx, count); });
}

}  // extern "C"
