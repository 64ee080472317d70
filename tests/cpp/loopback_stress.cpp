// Thread-safety stress of the loopback active-message context on host memory (no GPU),
// meant to be built with ThreadSanitizer (tests/test_host_cpp.py does that): several
// sender threads, each on a connection of its own, push eager and rendezvous messages
// at one server context while a receiver thread drains it and checks every payload,
// another sender cancels every other of its rendezvous sends right away, and another
// thread creates, connects and destroys unrelated contexts.  Two thirds of the messages
// are rendezvous sends, so that senders run into the 256 sends a context admits and the
// rest waits its turn.  The reference's
// context is reached from any thread with the work hopping to the context thread
// (ucx_context/ucx_am_context/ucx_am_context.hpp:2318-2392); here a mutex per context
// stands in for that hop.  Prints "loopback_stress ok <messages>" and exits 0.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "axon_rocm.h"

namespace {

constexpr int kSenders = 4;
constexpr int kPerSender = 400;

void die(const char* what, int rc) {
  std::fprintf(stderr, "loopback_stress: %s -> %d (%s)\n", what, rc, axr_last_error());
  std::exit(1);
}

struct Tag {   // the AM header of every message
  uint32_t sender, seq, bytes, pad;
};

uint8_t byte_of(uint32_t sender, uint32_t seq, size_t i) {
  return static_cast<uint8_t>(sender * 131u + seq * 7u + i);
}

}  // namespace

int main() {
  axr_am_context_t* server = nullptr;
  if (int rc = axr_am_context_create("server", 4096, &server)) die("create server", rc);
  std::atomic<int> received{0};
  std::atomic<bool> stop_churn{false};
  std::atomic<bool> canceller_done{false};
  std::atomic<int> cancelled_seen{0};

  std::vector<std::thread> threads;
  for (int s = 0; s < kSenders; ++s) {
    threads.emplace_back([s, server] {
      axr_am_context_t* client = nullptr;
      if (int rc = axr_am_context_create("client", 4096, &client)) die("create client", rc);
      uint64_t conn = 0;
      if (int rc = axr_am_connect(client, server, &conn)) die("connect", rc);
      // rendezvous sources must stay valid until the request completes
      std::vector<std::vector<uint8_t>> live(kPerSender);
      std::vector<uint64_t> requests(kPerSender);
      for (int q = 0; q < kPerSender; ++q) {
        const uint32_t bytes = (q % 3 != 2) ? 8192u + static_cast<uint32_t>(q) : static_cast<uint32_t>(q % 200);
        live[q].resize(bytes);
        for (size_t i = 0; i < bytes; ++i) live[q][i] = byte_of(s, q, i);
        Tag tag{static_cast<uint32_t>(s), static_cast<uint32_t>(q), bytes, 0};
        axr_am_data_t d;
        std::memset(&d, 0, sizeof(d));
        d.header.data = &tag;
        d.header.size = sizeof(tag);
        d.buffer.data = bytes ? live[q].data() : nullptr;
        d.buffer.size = bytes;
        d.buffer_type = AXR_MEM_HOST;
        if (int rc = axr_am_send(client, conn, &d, nullptr, &requests[q])) die("send", rc);
      }
      for (int q = 0; q < kPerSender; ++q) {
        int done = 0;
        while (!done) {
          if (int rc = axr_am_request_test(client, requests[q], &done)) die("request_test", rc);
          if (done < 0) die("request failed", done);
          if (!done) std::this_thread::yield();
        }
      }
      if (int rc = axr_am_context_destroy(client)) die("destroy client", rc);
    });
  }
  threads.emplace_back([server, &canceller_done] {   // sends and cancels
    axr_am_context_t* client = nullptr;
    if (int rc = axr_am_context_create("canceller", 4096, &client)) die("create canceller", rc);
    uint64_t conn = 0;
    if (int rc = axr_am_connect(client, server, &conn)) die("connect canceller", rc);
    constexpr int kCount = 300;
    std::vector<std::vector<uint8_t>> live(kCount);
    std::vector<uint64_t> requests(kCount);
    for (int q = 0; q < kCount; ++q) {
      const uint32_t bytes = 8192u + static_cast<uint32_t>(q);
      live[q].resize(bytes);
      for (size_t i = 0; i < bytes; ++i) live[q][i] = byte_of(kSenders, q, i);
      Tag tag{static_cast<uint32_t>(kSenders), static_cast<uint32_t>(q), bytes, 0};
      axr_am_data_t d;
      std::memset(&d, 0, sizeof(d));
      d.header.data = &tag;
      d.header.size = sizeof(tag);
      d.buffer.data = live[q].data();
      d.buffer.size = bytes;
      d.buffer_type = AXR_MEM_HOST;
      if (int rc = axr_am_send(client, conn, &d, nullptr, &requests[q])) die("send (canceller)", rc);
      if (q % 2) {
        if (int rc = axr_am_request_cancel(client, requests[q])) die("cancel", rc);
      }
    }
    for (int q = 0; q < kCount; ++q) {
      int done = 0;
      while (!done) {
        if (int rc = axr_am_request_test(client, requests[q], &done)) die("request_test (canceller)", rc);
        if (done < 0 && q % 2 == 0) die("a send that nobody cancelled failed", done);
        if (!done) std::this_thread::yield();
      }
    }
    size_t in_flight = 1, waiting = 1;
    if (int rc = axr_am_progress(client, &in_flight, &waiting)) die("progress", rc);
    if (in_flight || waiting) die("sends left behind", -1);
    if (int rc = axr_am_context_destroy(client)) die("destroy canceller", rc);
    canceller_done.store(true);
  });
  threads.emplace_back([server, &received, &canceller_done, &cancelled_seen] {
    std::vector<uint32_t> next(kSenders + 1, 0);
    std::vector<uint8_t> buf(16384);
    while (received.load() < kSenders * kPerSender || !canceller_done.load()) {
      axr_am_message_t m;
      const int rc = axr_am_recv_header(server, &m);
      if (rc == AXR_ERR_NO_MESSAGE) {
        std::this_thread::yield();
        continue;
      }
      if (rc) die("recv_header", rc);
      Tag tag;
      if (m.header.size != sizeof(tag)) die("header size", -1);
      std::memcpy(&tag, m.header.data, sizeof(tag));
      if (tag.sender > static_cast<uint32_t>(kSenders)) die("sender id", -1);
      if (tag.sender == static_cast<uint32_t>(kSenders)) {   // the canceller: some are missing, none out of order
        if (tag.seq < next[tag.sender]) die("order on the canceller's connection", -1);
        next[tag.sender] = tag.seq + 1;
      } else if (tag.seq != next[tag.sender]++) {
        die("order per connection", -1);
      }
      if (m.data_length != tag.bytes) die("length", -1);
      const uint8_t* got = nullptr;
      if (m.is_rndv) {
        const int rc2 = axr_am_recv_buffer(server, m.key, AXR_MEM_HOST, buf.data(), buf.size(), nullptr);
        if (rc2 == AXR_ERR_CANCELED && tag.sender == static_cast<uint32_t>(kSenders) && tag.seq % 2) {
          cancelled_seen.fetch_add(1);   // cancelled between its header and its fetch
          continue;
        }
        if (rc2) die("recv_buffer", rc2);
        got = buf.data();
      } else {
        got = static_cast<const uint8_t*>(m.eager_data.data);
      }
      for (size_t i = 0; i < tag.bytes; ++i)
        if (got[i] != byte_of(tag.sender, tag.seq, i)) die("payload", -1);
      if (!m.is_rndv) {
        if (int rc2 = axr_am_message_release(server, m.key)) die("release", rc2);
      }
      if (tag.sender < static_cast<uint32_t>(kSenders)) received.fetch_add(1);
    }
  });
  threads.emplace_back([&stop_churn] {   // unrelated contexts come and go
    while (!stop_churn.load()) {
      axr_am_context_t *a = nullptr, *b = nullptr;
      if (int rc = axr_am_context_create("a", 0, &a)) die("create a", rc);
      if (int rc = axr_am_context_create("b", 0, &b)) die("create b", rc);
      uint64_t conn = 0;
      if (int rc = axr_am_connect(a, b, &conn)) die("connect a b", rc);
      if (int rc = axr_am_context_destroy(b)) die("destroy b", rc);
      uint32_t word = 1;
      axr_am_data_t d;
      std::memset(&d, 0, sizeof(d));
      d.header.data = &word;
      d.header.size = sizeof(word);
      d.buffer_type = AXR_MEM_HOST;
      uint64_t req = 0;
      if (axr_am_send(a, conn, &d, nullptr, &req) != AXR_ERR_INVALID) die("send to a destroyed peer", -1);
      if (int rc = axr_am_context_destroy(a)) die("destroy a", rc);
    }
  });
  for (size_t i = 0; i + 1 < threads.size(); ++i) threads[i].join();
  stop_churn.store(true);
  threads.back().join();
  if (int rc = axr_am_context_destroy(server)) die("destroy server", rc);

  // Second phase: several threads send on ONE context (one connection each) while another
  // thread keeps calling axr_am_progress on it.  Every send is a rendezvous and nobody fetches
  // at first, so the context fills up (256 in flight) and the rest waits; then the receiver
  // drains.  Every sender's messages must arrive in the order that sender sent them: a message
  // that progress has just taken off the waiting queue must not be overtaken by a newer send.
  {
    axr_am_context_t *shared = nullptr, *sink = nullptr;
    if (int rc = axr_am_context_create("shared", 1, &shared)) die("create shared", rc);
    if (int rc = axr_am_context_create("sink", 1, &sink)) die("create sink", rc);
    constexpr int kThreads = 3, kEach = 300;
    std::atomic<bool> stop_progress{false};
    std::atomic<int> sent{0};
    std::vector<std::vector<uint64_t>> requests(kThreads, std::vector<uint64_t>(kEach));
    static uint8_t payload[64];
    std::vector<std::thread> phase;
    for (int s = 0; s < kThreads; ++s) {
      phase.emplace_back([s, shared, sink, &requests, &sent] {
        uint64_t conn = 0;
        if (int rc = axr_am_connect(shared, sink, &conn)) die("connect shared", rc);
        for (int q = 0; q < kEach; ++q) {
          Tag tag{static_cast<uint32_t>(s), static_cast<uint32_t>(q), sizeof(payload), 0};
          axr_am_data_t d;
          std::memset(&d, 0, sizeof(d));
          d.header.data = &tag;
          d.header.size = sizeof(tag);
          d.buffer.data = payload;
          d.buffer.size = sizeof(payload);
          d.buffer_type = AXR_MEM_HOST;
          if (int rc = axr_am_send(shared, conn, &d, nullptr, &requests[s][q])) die("send (shared)", rc);
          sent.fetch_add(1);
        }
      });
    }
    phase.emplace_back([shared, &stop_progress] {
      while (!stop_progress.load()) {
        if (int rc = axr_am_progress(shared, nullptr, nullptr)) die("progress (shared)", rc);
      }
    });
    std::vector<uint32_t> next(kThreads, 0);
    int got = 0;
    uint8_t into[64];
    while (got < kThreads * kEach) {
      axr_am_message_t m;
      const int rc = axr_am_recv_header(sink, &m);
      if (rc == AXR_ERR_NO_MESSAGE) {
        std::this_thread::yield();
        continue;
      }
      if (rc) die("recv_header (sink)", rc);
      Tag tag;
      std::memcpy(&tag, m.header.data, sizeof(tag));
      if (tag.sender >= static_cast<uint32_t>(kThreads) || tag.seq != next[tag.sender]++)
        die("order per sending thread on a shared context", -1);
      if (int rc2 = axr_am_recv_buffer(sink, m.key, AXR_MEM_HOST, into, sizeof(into), nullptr)) die("recv_buffer (sink)", rc2);
      ++got;
    }
    for (size_t i = 0; i < static_cast<size_t>(kThreads); ++i) phase[i].join();
    stop_progress.store(true);
    phase.back().join();
    for (int s = 0; s < kThreads; ++s)
      for (int q = 0; q < kEach; ++q) {
        int done = 0;
        if (int rc = axr_am_request_test(shared, requests[s][q], &done)) die("request_test (shared)", rc);
        if (done != 1) die("a send on the shared context did not complete", done);
      }
    if (int rc = axr_am_context_destroy(shared)) die("destroy shared", rc);
    if (int rc = axr_am_context_destroy(sink)) die("destroy sink", rc);
    received.fetch_add(got);
  }
  std::printf("loopback_stress ok %d\n", received.load());
  return 0;
}
