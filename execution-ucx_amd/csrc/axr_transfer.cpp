// Streamed transfer of a large payload in chunks: pack -> loopback send -> unpack,
// double-buffered over two (or more) lanes, each lane a send slot and a receive slot.
// Chunk k uses lane k % lanes and runs on stream (k % lanes) % streams.  With one stream
// per lane, stream order alone makes a slot safe to reuse `lanes` chunks later and chunk
// k + 1's pack overlaps chunk k's wire copy and unpack; with fewer streams than lanes the
// chunks of one stream run back to back and the extra lanes only let the host queue ahead
// (all three stages are bound by HBM bandwidth, so on one GPU two stages that run at once
// contend: one stream with two lanes measured 8 % faster than two streams).  The caller
// keeps ONE sender plan and ONE receiver plan for all chunks of one geometry and moves them
// over the data with the per-chunk tensor deltas: nothing is planned, uploaded or allocated
// per chunk.
//
// The send goes through the same loopback context calls a caller would make
// (axr_am_send / axr_am_recv_header / axr_am_recv_buffer_borrow or axr_am_recv_buffer_async),
// which stand for
// connection_send (ucx_am_context.hpp:2234-2642) and connection_recv_buffer
// (ucx_am_context.hpp:1511-1844) of the reference.
#include <cstring>
#include <new>
#include <vector>

#include "axr_internal.h"

using namespace axr;

struct axr_transfer {
  struct Lane {
    void* stream = nullptr;
    void* done = nullptr;          // event after the lane's last unpack
    void* send_slot = nullptr;
    void* send_mem_h = nullptr;
    void* recv_slot = nullptr;
    uint64_t request = 0;
    bool in_flight = false;
  };
  axr_pool_t* pool = nullptr;
  size_t slot_bytes = 0;
  std::vector<Lane> lanes;
  axr_am_context_t* client = nullptr;
  axr_am_context_t* server = nullptr;
  uint64_t conn = 0;
  uint64_t submitted = 0;
  bool zero_copy = true;        // the receiver unpacks out of the sender's slot
  size_t streams = 1;           // lanes i and i + streams share a stream; the first `streams` lanes own them
};

namespace {

// Wait for the chunk that last used the lane and settle its send request.
int retire(axr_transfer* t, axr_transfer::Lane& lane) {
  if (!lane.in_flight) return AXR_OK;
  lane.in_flight = false;
  int rc = axr_event_synchronize(lane.done);
  if (rc) return rc;
  int done = 0;
  rc = axr_am_request_test(t->client, lane.request, &done);
  if (rc) return rc;
  if (done != 1) return fail(AXR_ERR_HIP, "a chunk's send did not complete");
  return AXR_OK;
}

void destroy(axr_transfer* t) {
  for (auto& lane : t->lanes)
    if (lane.stream) (void)axr_stream_synchronize(lane.stream);
  for (size_t i = 0; i < t->lanes.size(); ++i) {
    auto& lane = t->lanes[i];
    if (lane.send_slot) (void)axr_pool_free(t->pool, lane.send_slot);
    if (lane.recv_slot) (void)axr_pool_free(t->pool, lane.recv_slot);
    if (lane.done) (void)axr_event_destroy(lane.done);
    if (lane.stream && i < t->streams) (void)axr_stream_destroy(lane.stream);
  }
  if (t->client) (void)axr_am_context_destroy(t->client);
  if (t->server) (void)axr_am_context_destroy(t->server);
  delete t;
}

}  // namespace

extern "C" {

static int transfer_create_body(axr_pool_t* pool, size_t slot_bytes, int lanes, int streams,
                                axr_transfer_t** out) {
  if (!out) return fail(AXR_ERR_INVALID, "axr_transfer_create: null result");
  *out = nullptr;
  if (slot_bytes == 0) return fail(AXR_ERR_INVALID, "axr_transfer_create: slot_bytes must be positive");
  if (lanes < 1 || lanes > 8) return fail(AXR_ERR_INVALID, "axr_transfer_create: lanes must be in [1, 8]");
  if (streams < 1 || streams > lanes)
    return fail(AXR_ERR_INVALID, "axr_transfer_create: streams must be in [1, lanes]");
  if (!pool) {
    int rc = axr_pool_default(&pool);
    if (rc) return rc;
  }
  axr_transfer* t = new (std::nothrow) axr_transfer();
  if (!t) return fail(AXR_ERR_NOMEM, "axr_transfer_create: out of host memory");
  t->pool = pool;
  t->slot_bytes = slot_bytes;
  t->lanes.resize(static_cast<size_t>(lanes));
  int rc = AXR_OK;
  t->streams = static_cast<size_t>(streams);
  for (size_t i = 0; i < t->lanes.size(); ++i) {
    auto& lane = t->lanes[i];
    if (i >= t->streams) lane.stream = t->lanes[i % t->streams].stream;
    else if (!rc) rc = axr_stream_create(&lane.stream);
    if (!rc) rc = axr_event_create(&lane.done);
    if (!rc) rc = axr_pool_alloc(pool, slot_bytes, 256, &lane.send_slot, &lane.send_mem_h);
    // (receive slots are only needed by the copying mode and are allocated when it is chosen)
  }
  // rendezvous for every chunk with a payload: the wire copy is stream ordered
  if (!rc) rc = axr_am_context_create("transfer-sender", 1, &t->client);
  if (!rc) rc = axr_am_context_create("transfer-receiver", 1, &t->server);
  if (!rc) rc = axr_am_connect(t->client, t->server, &t->conn);
  if (rc) {
    destroy(t);
    return rc;
  }
  *out = t;
  return AXR_OK;
}
int axr_transfer_create(axr_pool_t* pool, size_t slot_bytes, int lanes, int streams,
                        axr_transfer_t** transfer) {
  return guarded([&] { return transfer_create_body(pool, slot_bytes, lanes, streams, transfer); });
}

static int transfer_submit_body(axr_transfer_t* t, axr_plan_t* send_plan, int64_t send_delta,
                                axr_plan_t* recv_plan, int64_t recv_delta) {
  if (!t || !send_plan || !recv_plan) return fail(AXR_ERR_INVALID, "axr_transfer_submit: null argument");
  uint64_t nbytes = 0, expect = 0;
  int rc = axr_plan_payload_bytes(send_plan, &nbytes);
  if (!rc) rc = axr_plan_payload_bytes(recv_plan, &expect);
  if (rc) return rc;
  if (nbytes > t->slot_bytes) return fail(AXR_ERR_LENGTH, "chunk is larger than a transfer slot");
  const void* header = nullptr;
  size_t header_bytes = 0;
  rc = axr_plan_header(send_plan, &header, &header_bytes);
  if (rc) return rc;
  const void* recv_header = nullptr;
  size_t recv_header_bytes = 0;
  rc = axr_plan_header(recv_plan, &recv_header, &recv_header_bytes);
  if (rc) return rc;
  if (nbytes != expect || header_bytes != recv_header_bytes ||
      std::memcmp(header, recv_header, header_bytes) != 0)
    return fail(AXR_ERR_MISMATCH, "the receiver's plan was not made from the sender's header");
  axr_transfer::Lane& lane = t->lanes[t->submitted % t->lanes.size()];
  rc = retire(t, lane);
  if (rc) return rc;
  ++t->submitted;

  if (!t->zero_copy && !lane.recv_slot) {
    rc = axr_pool_alloc(t->pool, t->slot_bytes, 256, &lane.recv_slot, nullptr);
    if (rc) return rc;
  }
  uint64_t borrowed_key = 0;
  void* source = t->zero_copy ? lane.send_slot : lane.recv_slot;
  axr_job_t job;
  std::memset(&job, 0, sizeof(job));
  // The payload side keeps the plans' own cache treatment (cacheable up to the size of the
  // last-level cache) while the wire copy streams: measured fastest for 256 MiB chunks
  // (8.0 ms for 8 GiB against 8.7 ms with everything streaming and 9.5 ms with a cacheable copy).
  job.plan = send_plan;
  job.unpack = 0;
  job.payload = lane.send_slot;
  job.payload_bytes = nbytes;
  job.tensor_delta = send_delta;
  rc = axr_submit(&job, 1, lane.stream);
  if (rc) return rc;
  auto give_up = [&](int status) {
    // the pack is on the lane's stream already: let it finish before the slot is reused
    (void)axr_stream_synchronize(lane.stream);
    return status;
  };
  if (nbytes) {
    axr_am_data_t am;
    std::memset(&am, 0, sizeof(am));
    am.header = axr_buffer_t{const_cast<void*>(header), header_bytes};
    am.buffer = axr_buffer_t{lane.send_slot, static_cast<size_t>(nbytes)};
    am.buffer_type = AXR_MEM_ROCM;
    am.mem_h = lane.send_mem_h;
    rc = axr_am_send(t->client, t->conn, &am, lane.stream, &lane.request);
    if (rc) return give_up(rc);
    // From here on a failure must not leave the send parked or its message queued: the
    // slot is reused by the chunk after next.
    axr_am_message_t msg;
    rc = axr_am_recv_header(t->server, &msg);
    if (rc) {
      (void)axr_am_request_cancel(t->client, lane.request);
      return give_up(rc);
    }
    // what arrived is what the receiver planned for (tests can make one chunk fail here)
    bool injected = false;
    {
      std::atomic<int64_t>& countdown = tunables().transfer_fail_after_send;
      int64_t left = countdown.load();
      while (left > 0 && !countdown.compare_exchange_weak(left, left - 1)) {
      }
      injected = left == 1;
    }
    if (injected || !msg.is_rndv || msg.data_length != nbytes || msg.header.size != recv_header_bytes ||
        std::memcmp(msg.header.data, recv_header, recv_header_bytes) != 0) {
      (void)axr_am_message_release(t->server, msg.key);
      (void)axr_am_request_cancel(t->client, lane.request);
      return give_up(fail(AXR_ERR_MISMATCH, "the received message does not match the receiver's plan"));
    }
    if (t->zero_copy) {
      void* lent = nullptr;
      size_t lent_bytes = 0;
      rc = axr_am_recv_buffer_borrow(t->server, msg.key, &lent, &lent_bytes, nullptr);
      if (!rc && (lent != lane.send_slot || lent_bytes != nbytes)) {
        (void)axr_am_borrow_release(t->server, msg.key, lane.stream);
        rc = fail(AXR_ERR_MISMATCH, "the borrowed payload is not the chunk that was sent");
      }
      if (!rc) {
        borrowed_key = msg.key;
        source = lent;
      }
    } else {
      rc = axr_am_recv_buffer_async(t->server, msg.key, AXR_MEM_ROCM, lane.recv_slot, t->slot_bytes,
                                    lane.stream);
    }
    if (rc) {
      (void)axr_am_message_release(t->server, msg.key);
      (void)axr_am_request_cancel(t->client, lane.request);
      // the lane's stream may already hold this chunk's pack: drain it, so that the slot is
      // quiet before the next chunk on this lane reuses it
      (void)axr_stream_synchronize(lane.stream);
      return rc;
    }
    lane.in_flight = true;
  }
  job.plan = recv_plan;
  job.unpack = 1;
  job.payload = source;
  job.tensor_delta = recv_delta;
  rc = axr_submit(&job, 1, lane.stream);
  // the send completes behind the scatter that reads its slot (also when the scatter was refused:
  // the lane must come back to a state in which retire() finds a completed send)
  if (borrowed_key) {
    const int released = axr_am_borrow_release(t->server, borrowed_key, lane.stream);
    if (!rc) rc = released;
  }
  const int recorded = axr_event_record(lane.done, lane.stream);
  if (rc || recorded) {
    // whatever was enqueued runs to its end before the error is reported: the lane's event and
    // send request are then settled and the next chunk finds the lane idle
    (void)axr_stream_synchronize(lane.stream);
    if (lane.in_flight) {
      int done = 0;
      (void)axr_am_request_test(t->client, lane.request, &done);
      lane.in_flight = false;
    }
    return rc ? rc : recorded;
  }
  return AXR_OK;
}
int axr_transfer_submit(axr_transfer_t* transfer, axr_plan_t* send_plan, int64_t send_delta,
                        axr_plan_t* recv_plan, int64_t recv_delta) {
  return guarded([&] { return transfer_submit_body(transfer, send_plan, send_delta, recv_plan, recv_delta); });
}

static int transfer_set_zero_copy_body(axr_transfer_t* t, int enable) {
  if (!t) return fail(AXR_ERR_INVALID, "axr_transfer_set_zero_copy: null transfer");
  for (auto& lane : t->lanes)
    if (lane.in_flight) return fail(AXR_ERR_BUSY, "axr_transfer_set_zero_copy: chunks are in flight; call axr_transfer_finish first");
  t->zero_copy = enable != 0;
  return AXR_OK;
}
int axr_transfer_set_zero_copy(axr_transfer_t* transfer, int enable) {
  return guarded([&] { return transfer_set_zero_copy_body(transfer, enable); });
}

static int transfer_finish_body(axr_transfer_t* t) {
  if (!t) return fail(AXR_ERR_INVALID, "axr_transfer_finish: null transfer");
  int first = AXR_OK;
  for (auto& lane : t->lanes) {
    int rc = retire(t, lane);
    if (!rc) rc = axr_stream_synchronize(lane.stream);
    if (rc && !first) first = rc;
  }
  return first;
}
int axr_transfer_finish(axr_transfer_t* transfer) {
  return guarded([&] { return transfer_finish_body(transfer); });
}

static int transfer_destroy_body(axr_transfer_t* t) {
  if (!t) return AXR_OK;
  const int rc = transfer_finish_body(t);
  destroy(t);
  return rc;
}
int axr_transfer_destroy(axr_transfer_t* transfer) {
  return guarded([&] { return transfer_destroy_body(transfer); });
}

}  // extern "C"
