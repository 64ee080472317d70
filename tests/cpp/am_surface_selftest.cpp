// Runs the active-message bundle surface of execution-ucx_amd/host/loopback_am_context.hpp
// (connection_send / connection_recv / connection_recv_header / connection_recv_buffer with
// the reference's REAL UcxBuffer / UcxHeader / UcxAmData / UcxAmIovec / UcxBufferVec,
// ucx_context/ucx_context_data.hpp) on a GPU.  TEST INFRASTRUCTURE: built by oracle/Makefile
// into oracle/_ref/ with the execution-ucx tree on the include path; links the C oracle
// (liborc.so) as the checker.
//
//   PackTensors -> connection_send -> connection_recv_header -> ReceiveBufferFor ->
//   connection_recv_buffer -> UnpackTensors, payload compared with the oracle's pack
//
// for the host bundle of 64 fp32 tensors and for a device bundle, then the reference's edge
// rules (ucx_am_context.hpp:1570-1574, 1604-1621, 1643-1651, 1808-1818, 2275-2278), its
// known-answer cases (ucx_am_connection_test.cpp:1051-1108 iov -> contiguous and iov -> iov,
// ucx_am_context_test.cpp:321-333 send -> divide by two -> reply) and cancellation.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "loopback_am_context.hpp"
#include "reference_adapters.hpp"
#include "ucx_rocm_context.hpp"
#include "ucx_rocm_memory_manager.hpp"

#ifndef AXON_ROCM_HAVE_REFERENCE_MEMORY_RESOURCE
#error "build with -DAXON_ROCM_IN_REFERENCE_TREE and the execution-ucx tree on the include path"
#endif

extern "C" {
uint64_t orc_layout(const uint64_t* sizes, size_t n, uint64_t align, uint64_t* offsets);
int orc_pack(const void* const* srcs, const uint64_t* sizes, const uint64_t* offsets, size_t n, void* dst,
             uint64_t total);
}

using namespace eux::ucxx;
using namespace eux::ucxx::loopback;
using eux::axon::rocm::PackTensors;
using eux::axon::rocm::ReceiveBufferFor;
using eux::axon::rocm::UnpackTensors;

namespace {

int g_failures = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);           \
      std::fflush(stdout);                                                    \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

// A receiver that records how it was completed.
struct Outcome {
  int values = 0, errors = 0, dones = 0;
  std::error_code error;
};
struct Recorder {
  Outcome* out;
  template <typename... A>
  void set_value(A&&...) && { ++out->values; }
  void set_error(std::error_code ec) && {
    ++out->errors;
    out->error = ec;
  }
  void set_done() && { ++out->dones; }
};

std::vector<uint8_t> oracle_pack(const std::vector<std::vector<uint8_t>>& chunks, uint64_t align) {
  std::vector<uint64_t> sizes, offsets(chunks.size());
  std::vector<const void*> srcs;
  for (const auto& c : chunks) {
    sizes.push_back(c.size());
    srcs.push_back(c.data());
  }
  const uint64_t total = orc_layout(sizes.data(), sizes.size(), align, offsets.data());
  std::vector<uint8_t> out(total);
  if (orc_pack(srcs.data(), sizes.data(), offsets.data(), sizes.size(), out.data(), total) != 0) std::abort();
  return out;
}

struct Pair {
  UcxRocmMemoryResourceManager& mr;
  loopback_am_context client, server;
  LoopbackConnection to_server, to_client;
  explicit Pair(UcxRocmMemoryResourceManager& m)
      : mr(m), client(m, "client"), server(m, "server"), to_server(client.connect(server)),
        to_client(server.connect(client)) {}
};

axr_tensor_t describe(void* data, int32_t device_type, uint8_t code, uint8_t bits, int64_t* shape, int32_t ndim) {
  axr_tensor_t t;
  std::memset(&t, 0, sizeof(t));
  t.data = data;
  t.device_type = device_type;
  t.ndim = ndim;
  t.dtype_code = code;
  t.dtype_bits = bits;
  t.dtype_lanes = 1;
  t.shape = shape;
  return t;
}

// The whole path for one list of byte chunks living in host (kDLCPU) or device (kDLROCM)
// memory.  `own` sends an owning UcxAmData&& (the operation keeps the pool block until the
// send has completed), otherwise a borrowed ucx_am_data&.
void bundle_round_trip(Pair& p, const std::vector<std::vector<uint8_t>>& chunks, bool device, uint32_t align,
                       bool own) {
  UcxRocmMemoryResourceManager& mr = p.mr;
  const uint64_t blocks_before = mr.stats().live_blocks;
  const size_t n = chunks.size();
  std::vector<int64_t> shapes(n);
  std::vector<void*> src(n, nullptr), dst(n, nullptr);
  std::vector<std::vector<uint8_t>> outs(n);
  std::vector<axr_tensor_t> sdesc, ddesc;
  for (size_t i = 0; i < n; ++i) {
    shapes[i] = static_cast<int64_t>(chunks[i].size());
    outs[i].assign(chunks[i].size(), 0xEE);
    if (device && !chunks[i].empty()) {
      src[i] = mr.allocate(ucx_memory_type::ROCM, chunks[i].size(), 16);
      dst[i] = mr.allocate(ucx_memory_type::ROCM, chunks[i].size(), 16);
      mr.memcpy(ucx_memory_type::ROCM, src[i], ucx_memory_type::HOST, chunks[i].data(), chunks[i].size());
    } else if (!device) {
      src[i] = const_cast<uint8_t*>(chunks[i].data());
      dst[i] = outs[i].data();
    }
    sdesc.push_back(describe(src[i], device ? 10 : 1, 1, 8, &shapes[i], 1));
    ddesc.push_back(describe(dst[i], device ? 10 : 1, 1, 8, &shapes[i], 1));
  }
  const std::vector<uint8_t> want = oracle_pack(chunks, align);
  {
    // sender
    auto bundle = PackTensors(mr, sdesc.data(), n, align, p.client.stream());
    EXPECT(bundle.payload_bytes() == want.size());
    eux::axon::rocm::Check(axr_stream_synchronize(p.client.stream()), "axr_stream_synchronize");
    Outcome sent;
    ucx_am_data am = bundle.as_am_data();
    std::optional<UcxAmData> owned;
    if (own) {
      // header copy in host memory of the resource manager, the pool block handed over
      ucx_am_data raw = am;
      raw.header.data = mr.allocate(ucx_memory_type::HOST, am.header.size);
      std::memcpy(raw.header.data, am.header.data, am.header.size);
      const size_t bytes = bundle.payload_bytes();
      UcxRocmMemoryResourceManager* pmr = &mr;
      bundle.plan().reset();
      raw.buffer.data = bundle.detach();
      owned.emplace(mr, std::move(raw), /*own_header=*/true, /*own_buffer=*/true,
                    [pmr, bytes](void* q) { pmr->deallocate(ucx_memory_type::ROCM, q, bytes); });
    }
    auto send_op = own ? connect(connection_send(p.client.get_scheduler(), p.to_server, std::move(*owned)), Recorder{&sent})
                       : connect(connection_send(p.client.get_scheduler(), p.to_server.id(), am), Recorder{&sent});
    owned.reset();
    send_op.start();
    const bool rndv = want.size() >= 4096;
    EXPECT(sent.values == (rndv ? 0 : 1));   // a rendezvous send waits for the receiver's fetch

    // receiver
    auto first = sync_wait<recv_header_result_type>(p.server, connection_recv_header(p.server.get_scheduler()));
    EXPECT(first.has_value());
    if (!first) return;
    std::vector<uint8_t> header_bytes;
    std::optional<UcxBuffer> payload;
    if (rndv) {
      EXPECT(first->index() == 0);
      auto& keyed = std::get<0>(*first);
      header_bytes.assign(static_cast<uint8_t*>(keyed.second.data()),
                          static_cast<uint8_t*>(keyed.second.data()) + keyed.second.size());
      EXPECT(keyed.second.own_header());
      UcxBuffer room = ReceiveBufferFor(header_bytes.data(), header_bytes.size(), mr);
      EXPECT(room.size() == want.size());
      void* const block = room.data();
      auto got = sync_wait<active_message_buffer_bundle>(
          p.server, connection_recv_buffer(p.server.get_scheduler(), keyed.first, std::move(room)));
      EXPECT(got.has_value());
      if (!got) return;
      EXPECT(got->buffer().data() == block);                  // large enough: used as it is
      EXPECT(got->buffer().type() == ucx_memory_type::ROCM);
      EXPECT(got->connection().id() == p.to_server.id());
      payload.emplace(got->move_buffer());
      p.client.progress();
      EXPECT(sent.values == 1 && sent.errors == 0 && sent.dones == 0);
    } else {
      EXPECT(first->index() == 1);
      auto& whole = std::get<1>(*first);
      header_bytes.assign(static_cast<const uint8_t*>(whole.header().data()),
                          static_cast<const uint8_t*>(whole.header().data()) + whole.header().size());
      EXPECT(whole.buffer().type() == ucx_memory_type::HOST);   // eager payloads arrive in host memory
      EXPECT(whole.buffer().size() == want.size());
      // the unpack kernel reads device memory: move the eager payload there
      UcxBuffer room = ReceiveBufferFor(header_bytes.data(), header_bytes.size(), mr);
      if (want.size())
        mr.memcpy(ucx_memory_type::ROCM, room.data(), ucx_memory_type::HOST, whole.buffer().data(), want.size());
      payload.emplace(std::move(room));
    }
    // the payload is the oracle's pack of the same chunks
    std::vector<uint8_t> got_bytes(want.size());
    if (!want.empty())
      mr.memcpy(ucx_memory_type::HOST, got_bytes.data(), ucx_memory_type::ROCM, payload->data(), want.size());
    EXPECT(got_bytes == want);
    {
      auto rplan = UnpackTensors(header_bytes.data(), header_bytes.size(), payload->data(), payload->size(),
                                 ddesc.data(), n, p.server.stream());
    }   // destroying the plan waits for the kernel
    for (size_t i = 0; i < n; ++i) {
      if (device && !chunks[i].empty())
        mr.memcpy(ucx_memory_type::HOST, outs[i].data(), ucx_memory_type::ROCM, dst[i], chunks[i].size());
      EXPECT(outs[i] == chunks[i]);
    }
  }
  for (size_t i = 0; i < n; ++i) {
    if (device && src[i]) mr.deallocate(ucx_memory_type::ROCM, src[i], chunks[i].size());
    if (device && dst[i]) mr.deallocate(ucx_memory_type::ROCM, dst[i], chunks[i].size());
  }
  EXPECT(mr.stats().live_blocks == blocks_before);   // owned payloads were released at completion
}

// iov -> contiguous and iov -> iov with the reference's pattern: segments of 512 KiB, 256 KiB
// and 800 KiB (or 256/512/300 bytes), byte = running index % 256, header {1, 2, 3, 4}.
void iov_known_answers(Pair& p, const std::vector<size_t>& lens) {
  UcxRocmMemoryResourceManager& mr = p.mr;
  std::vector<std::vector<uint8_t>> segs;
  size_t cursor = 0, total = 0;
  for (size_t len : lens) {
    std::vector<uint8_t> s(len);
    for (auto& b : s) b = static_cast<uint8_t>(cursor++ % 256);
    segs.push_back(std::move(s));
    total += len;
  }
  uint8_t header[4] = {1, 2, 3, 4};
  std::vector<ucx_buffer_t> vec;
  for (auto& s : segs) vec.push_back(ucx_buffer_t{s.data(), s.size()});
  for (int pass = 0; pass < 2; ++pass) {
    ucx_am_iovec iov;
    std::memset(&iov, 0, sizeof(iov));
    iov.header = ucx_buffer_t{header, sizeof(header)};
    iov.buffer_vec = vec.data();
    iov.buffer_count = vec.size();
    iov.buffer_type = ucx_memory_type::HOST;
    Outcome sent;
    auto send_op = connect(connection_send(p.client.get_scheduler(), p.to_server, iov), Recorder{&sent});
    send_op.start();
    EXPECT(sent.values == 0);   // an iov payload is always a rendezvous (ucx_connection.cpp:417-419)
    if (pass == 0) {
      // contiguous receive: the flat concatenation
      auto got = sync_wait<active_message_bundle>(p.server, connection_recv(p.server.get_scheduler(), ucx_memory_type::HOST));
      EXPECT(got.has_value());
      if (!got) return;
      const ucx_am_data& d = got->get_raw_data();
      EXPECT(d.header.size == 4 && std::memcmp(d.header.data, header, 4) == 0);
      EXPECT(d.buffer.size == total && d.buffer_type == ucx_memory_type::HOST);
      bool same = d.buffer.size == total;
      for (size_t i = 0; same && i < total; ++i) same = static_cast<uint8_t*>(d.buffer.data)[i] == static_cast<uint8_t>(i % 256);
      EXPECT(same);
      EXPECT(got->data().owns_header() && got->data().own_buffer());
    } else {
      // iov receive with the same lengths: per-segment equality
      auto first = sync_wait<recv_header_result_type>(p.server, connection_recv_header(p.server.get_scheduler()));
      EXPECT(first && first->index() == 0);
      if (!first || first->index() != 0) return;
      const size_t key = std::get<0>(*first).first;
      // an iov whose entries are not allocated is refused and the message stays parked (:1808-1818)
      Outcome refused;
      std::vector<ucx_buffer_t> empty_entries(lens.size(), ucx_buffer_t{nullptr, 0});
      auto bad = connect(connection_recv_buffer(p.server.get_scheduler(), key,
                                                UcxBufferVec(mr, ucx_memory_type::HOST, std::move(empty_entries))),
                         Recorder{&refused});
      bad.start();
      EXPECT(refused.errors == 1 && refused.error == make_error_code(am_errc::invalid_param));
      auto got = sync_wait<active_message_iovec_buffer_bundle>(
          p.server, connection_recv_buffer(p.server.get_scheduler(), key, UcxBufferVec(mr, ucx_memory_type::HOST, lens)));
      EXPECT(got.has_value());
      if (!got) return;
      EXPECT(got->buffer().size() == lens.size());
      for (size_t i = 0; i < lens.size(); ++i) {
        EXPECT(got->buffer()[i].size == lens[i]);
        EXPECT(std::memcmp(got->buffer()[i].data, segs[i].data(), lens[i]) == 0);
      }
    }
    p.client.progress();
    EXPECT(sent.values == 1);
  }
}

void edge_rules(Pair& p) {
  UcxRocmMemoryResourceManager& mr = p.mr;
  // a send needs a header (ucx_am_context.hpp:2275-2278)
  {
    ucx_am_data d;
    std::memset(&d, 0, sizeof(d));
    Outcome o;
    auto op = connect(connection_send(p.client.get_scheduler(), p.to_server, d), Recorder{&o});
    op.start();
    EXPECT(o.errors == 1 && o.error == make_error_code(am_errc::invalid_param));
  }
  // unknown key: UCS_ERR_NO_MESSAGE (:1570-1574)
  {
    Outcome o;
    auto op = connect(connection_recv_buffer(p.server.get_scheduler(), 0xdeadbeefu, ucx_memory_type::HOST), Recorder{&o});
    op.start();
    EXPECT(o.errors == 1 && o.error == make_error_code(am_errc::no_message));
    EXPECT(o.error.message() == "UCS_ERR_NO_MESSAGE");
  }
  // the payload of an eager message comes with its header; asking for it by key is
  // UCS_ERR_NOT_IMPLEMENTED (:1643-1651)
  {
    uint8_t header[2] = {7, 9};
    std::vector<uint8_t> small(100, 0x5a);
    ucx_am_data d;
    std::memset(&d, 0, sizeof(d));
    d.header = ucx_buffer_t{header, 2};
    d.buffer = ucx_buffer_t{small.data(), small.size()};
    d.buffer_type = ucx_memory_type::HOST;
    EXPECT(sync_wait_void(p.client, connection_send(p.client.get_scheduler(), p.to_server, d)));   // complete at once
    axr_am_message_t m;
    EXPECT(axr_am_recv_header(p.server.handle(), &m) == AXR_OK && !m.is_rndv);
    Outcome o;
    auto op = connect(connection_recv_buffer(p.server.get_scheduler(), m.key, ucx_memory_type::HOST), Recorder{&o});
    op.start();
    EXPECT(o.errors == 1 && o.error == make_error_code(am_errc::not_implemented));
    EXPECT(axr_am_message_release(p.server.handle(), m.key) == AXR_OK);
    // the same message through connection_recv_header: a complete bundle, payload in host memory
    EXPECT(sync_wait_void(p.client, connection_send(p.client.get_scheduler(), p.to_server, d)));
    auto whole = sync_wait<recv_header_result_type>(p.server, connection_recv_header(p.server.get_scheduler()));
    EXPECT(whole && whole->index() == 1);
    if (whole && whole->index() == 1) {
      auto& b = std::get<1>(*whole);
      EXPECT(b.header().size() == 2 && std::memcmp(b.header().data(), header, 2) == 0);
      EXPECT(b.buffer().size() == 100 && std::memcmp(b.buffer().data(), small.data(), 100) == 0);
      EXPECT(b.buffer().type() == ucx_memory_type::HOST && b.buffer().own_buffer());
    }
    // and through connection_recv into device memory: copied there by the resource's memcpy (:1258-1260)
    EXPECT(sync_wait_void(p.client, connection_send(p.client.get_scheduler(), p.to_server, d)));
    auto dev = sync_wait<active_message_bundle>(p.server, connection_recv(p.server.get_scheduler(), ucx_memory_type::ROCM));
    EXPECT(dev.has_value());
    if (dev) {
      const ucx_am_data& r = dev->get_raw_data();
      EXPECT(r.buffer_type == ucx_memory_type::ROCM && r.buffer.size == 100);
      std::vector<uint8_t> back(100);
      mr.memcpy(ucx_memory_type::HOST, back.data(), ucx_memory_type::ROCM, r.buffer.data, 100);
      EXPECT(back == small);
    }
  }
  // a buffer that is too small is released and allocated again; its size becomes the
  // message's (:1604-1621).  A borrowed ucx_am_data with a header is refused (:1092-1095).
  {
    const size_t n = 1 << 20;
    std::vector<uint8_t> big(n);
    for (size_t i = 0; i < n; ++i) big[i] = static_cast<uint8_t>(i * 7);
    uint8_t header[1] = {1};
    ucx_am_data d;
    std::memset(&d, 0, sizeof(d));
    d.header = ucx_buffer_t{header, 1};
    d.buffer = ucx_buffer_t{big.data(), n};
    d.buffer_type = ucx_memory_type::HOST;
    Outcome sent;
    auto send_op = connect(connection_send(p.client.get_scheduler(), p.to_server, d), Recorder{&sent});
    send_op.start();
    auto first = sync_wait<recv_header_result_type>(p.server, connection_recv_header(p.server.get_scheduler()));
    EXPECT(first && first->index() == 0);
    if (first && first->index() == 0) {
      const uint64_t live = mr.stats().live_blocks;
      {
        UcxBuffer tiny(mr, ucx_memory_type::ROCM, 16);
        auto got = sync_wait<active_message_buffer_bundle>(
            p.server, connection_recv_buffer(p.server.get_scheduler(), std::get<0>(*first).first, std::move(tiny)));
        EXPECT(got.has_value());
        if (got) {
          EXPECT(got->buffer().size() == n && got->buffer().data() != nullptr);
          EXPECT(mr.stats().live_blocks == live + 1);   // the 16-byte block went back, one block of n bytes came
          std::vector<uint8_t> back(n);
          mr.memcpy(ucx_memory_type::HOST, back.data(), ucx_memory_type::ROCM, got->buffer().data(), n);
          EXPECT(back == big);
        }
      }
      EXPECT(mr.stats().live_blocks == live);
    }
    p.client.progress();
    EXPECT(sent.values == 1);
    ucx_am_data with_header;
    std::memset(&with_header, 0, sizeof(with_header));
    with_header.header = ucx_buffer_t{header, 1};
    Outcome o;
    auto op = connect(connection_recv(p.server.get_scheduler(), with_header), Recorder{&o});
    op.start();
    EXPECT(o.errors == 1 && o.error == make_error_code(am_errc::invalid_param));
    // borrowed receive into a buffer the caller provides: filled in place, header allocated for the caller
    Outcome again;
    auto second = connect(connection_send(p.client.get_scheduler(), p.to_server, d), Recorder{&again});
    second.start();
    std::vector<uint8_t> mine(n + 64, 0);
    ucx_am_data into;
    std::memset(&into, 0, sizeof(into));
    into.buffer = ucx_buffer_t{mine.data(), mine.size()};
    into.buffer_type = ucx_memory_type::HOST;
    auto got = sync_wait<active_message_bundle>(p.server, connection_recv(p.server.get_scheduler(), into), {&p.client});
    EXPECT(got.has_value());
    EXPECT(into.buffer.data == mine.data() && into.buffer.size == n);
    EXPECT(std::memcmp(mine.data(), big.data(), n) == 0);
    EXPECT(into.header.size == 1 && into.header.data && *static_cast<uint8_t*>(into.header.data) == 1);
    if (got) EXPECT(!got->data().owns_header() && !got->data().own_buffer());   // a view of the caller's descriptor
    if (into.header.data) mr.deallocate(ucx_memory_type::HOST, into.header.data, into.header.size);
    p.client.progress();
    EXPECT(again.values == 1);
    // a wait for a message that nobody sends ends with timed_out instead of spinning for ever
    bool timed_out = false;
    try {
      (void)sync_wait<recv_header_result_type>(p.server, connection_recv_header(p.server.get_scheduler()), {},
                                               std::chrono::milliseconds(20));
    } catch (const std::system_error& e) {
      timed_out = e.code() == std::make_error_code(std::errc::timed_out);
    }
    EXPECT(timed_out && p.server.progress() == 0);
  }
}

void cancellation(Pair& p) {
  // a receive that waits for a message is stopped: set_done, nothing else
  {
    Outcome o;
    auto op = connect(connection_recv_header(p.server.get_scheduler()), Recorder{&o});
    op.start();
    EXPECT(p.server.progress() == 1 && o.values + o.errors + o.dones == 0);
    op.request_stop();
    EXPECT(o.dones == 1 && o.values == 0 && o.errors == 0);
    EXPECT(p.server.progress() == 0);
    op.request_stop();                       // a second stop request changes nothing
    EXPECT(o.dones == 1);
  }
  // a rendezvous send that nobody has fetched is withdrawn: the receiver never sees it
  {
    std::vector<uint8_t> big(64 * 1024, 3);
    uint8_t header[1] = {5};
    ucx_am_data d;
    std::memset(&d, 0, sizeof(d));
    d.header = ucx_buffer_t{header, 1};
    d.buffer = ucx_buffer_t{big.data(), big.size()};
    d.buffer_type = ucx_memory_type::HOST;
    Outcome o;
    auto op = connect(connection_send(p.client.get_scheduler(), p.to_server, d), Recorder{&o});
    op.start();
    EXPECT(o.values == 0 && p.client.progress() == 1);
    op.request_stop();
    EXPECT(o.dones == 1 && o.values == 0);
    EXPECT(p.client.progress() == 0);
    Outcome r;
    auto rop = connect(connection_recv_header(p.server.get_scheduler()), Recorder{&r});
    rop.start();
    EXPECT(r.values == 0);                    // nothing arrived
    rop.request_stop();
  }
  // a parked receive is completed by progress() once a message has arrived
  {
    Outcome r;
    auto rop = connect(connection_recv(p.server.get_scheduler(), ucx_memory_type::HOST), Recorder{&r});
    rop.start();
    EXPECT(r.values == 0);
    uint8_t header[1] = {9};
    uint8_t body[8] = {1, 2, 3, 4, 5, 6, 7, 8};
    ucx_am_data d;
    std::memset(&d, 0, sizeof(d));
    d.header = ucx_buffer_t{header, 1};
    d.buffer = ucx_buffer_t{body, 8};
    d.buffer_type = ucx_memory_type::HOST;
    EXPECT(sync_wait_void(p.client, connection_send(p.client.get_scheduler(), p.to_server, d)));
    EXPECT(r.values == 0);
    p.server.progress();
    EXPECT(r.values == 1);
  }
}

// send float(i % 256), the server divides by two on the device and replies, the client
// expects (i % 256) / 2 exactly (ucx_am_context_test.cpp:321-333, 1893-1944)
void process_round_trip(Pair& p, size_t count) {
  UcxRocmMemoryResourceManager& mr = p.mr;
  std::vector<float> host(count);
  for (size_t i = 0; i < count; ++i) host[i] = static_cast<float>(i % 256);
  const size_t bytes = count * sizeof(float);
  UcxAmData request(mr, 4, bytes, ucx_memory_type::ROCM);
  std::memcpy(request.get()->header.data, "req", 4);
  mr.memcpy(ucx_memory_type::ROCM, request.get()->buffer.data, ucx_memory_type::HOST, host.data(), bytes);
  Outcome sent;
  auto send_op = connect(connection_send(p.client.get_scheduler(), p.to_server, std::move(request)), Recorder{&sent});
  send_op.start();
  auto got = sync_wait<active_message_bundle>(p.server, connection_recv(p.server.get_scheduler(), ucx_memory_type::ROCM),
                                              {&p.client});
  EXPECT(got.has_value());
  if (!got) return;
  p.client.progress();
  EXPECT(sent.values == 1);
  UcxAmData work = got->move_data();
  EXPECT(work.get()->buffer.size == bytes && work.get()->buffer_type == ucx_memory_type::ROCM);
  eux::axon::rocm::Check(axr_divide_by_two(static_cast<float*>(work.get()->buffer.data), count, p.server.stream()),
                         "axr_divide_by_two");
  eux::axon::rocm::Check(axr_stream_synchronize(p.server.stream()), "axr_stream_synchronize");
  Outcome replied;
  auto reply_op = connect(connection_send(p.server.get_scheduler(), got->connection().id() ? p.to_client : p.to_client,
                                          std::move(work)),
                          Recorder{&replied});
  reply_op.start();
  auto back = sync_wait<active_message_bundle>(p.client, connection_recv(p.client.get_scheduler(), ucx_memory_type::HOST),
                                               {&p.server});
  EXPECT(back.has_value());
  if (!back) return;
  p.server.progress();
  EXPECT(replied.values == 1);
  const ucx_am_data& r = back->get_raw_data();
  EXPECT(r.buffer.size == bytes && r.buffer_type == ucx_memory_type::HOST);
  bool exact = r.buffer.size == bytes;
  for (size_t i = 0; exact && i < count; ++i)
    exact = static_cast<float*>(r.buffer.data)[i] == static_cast<float>(i % 256) / 2.0f;
  EXPECT(exact);
}

}  // namespace

int main() {
  int count = 0;
  if (axr_device_count(&count) != AXR_OK || count == 0) {
    std::printf("am_surface_selftest: no device\n");
    return 2;
  }
  try {
    UcxAutoRocmDeviceContext context(0);
    auto active = context(nullptr, nullptr);
    UcxRocmMemoryResourceManager mr(0);
    {
      Pair p(mr);
      // the host bundle of 64 fp32 tensors of 16,384 elements, uniform [-1, 1) from a seed
      std::mt19937_64 rng(0);
      std::uniform_real_distribution<float> uni(-1.0f, 1.0f);
      std::vector<std::vector<uint8_t>> c1(64, std::vector<uint8_t>(16384 * sizeof(float)));
      for (auto& c : c1)
        for (size_t i = 0; i < 16384; ++i) {
          const float v = uni(rng);
          std::memcpy(c.data() + 4 * i, &v, 4);
        }
      std::printf("host bundle (64 x 64 KiB)\n");
      std::fflush(stdout);
      bundle_round_trip(p, c1, /*device=*/false, 1, /*own=*/false);
      bundle_round_trip(p, c1, /*device=*/false, 256, /*own=*/true);
      // a device bundle: long and short tensors (the short ones share wavefronts), an empty one
      std::vector<std::vector<uint8_t>> mixed;
      for (size_t len : {size_t(1000003), size_t(0), size_t(13), size_t(4096), size_t(77), size_t(300), size_t(1),
                         size_t(65536), size_t(257), size_t(8), size_t(8), size_t(100000)}) {
        std::vector<uint8_t> c(len);
        for (auto& b : c) b = static_cast<uint8_t>(rng());
        mixed.push_back(std::move(c));
      }
      std::printf("device bundle\n");
      std::fflush(stdout);
      for (uint32_t align : {1u, 256u})
        for (bool own : {false, true}) bundle_round_trip(p, mixed, /*device=*/true, align, own);
      // a bundle below the zero-copy threshold travels eagerly, header and payload together
      std::vector<std::vector<uint8_t>> tiny = {std::vector<uint8_t>(40, 1), std::vector<uint8_t>(24, 2)};
      bundle_round_trip(p, tiny, /*device=*/true, 1, /*own=*/false);
      std::printf("iov known answers\n");
      std::fflush(stdout);
      iov_known_answers(p, {256, 512, 300});
      iov_known_answers(p, {512 * 1024, 256 * 1024, 800 * 1024});
      std::printf("edge rules\n");
      std::fflush(stdout);
      edge_rules(p);
      std::printf("cancellation\n");
      std::fflush(stdout);
      cancellation(p);
      std::printf("process round trip\n");
      std::fflush(stdout);
      process_round_trip(p, 32);
      process_round_trip(p, 1 << 20);
    }
    EXPECT(mr.stats().live_blocks == 0);
  } catch (const std::exception& e) {
    std::printf("am_surface_selftest: exception: %s\n", e.what());
    return 1;
  }
  if (g_failures) {
    std::printf("am_surface_selftest: %d check(s) failed\n", g_failures);
    return 1;
  }
  std::printf("am_surface_selftest ok\n");
  return 0;
}
