// Round trip of a fresh 4096-tensor bundle timed from a C++ caller, C ABI only:
//   axr_plan_create + axr_plan_header -> axr_pack -> axr_stream_synchronize ->
//   axr_plan_from_header_bind -> axr_unpack -> axr_stream_synchronize
// (what ClientSendRequest_ and ProcessRndvBuffer_ would do per call for a bundle whose tensor
// list is new, axon/src/axon_worker.cpp:1424-1490 and :1098-1219).  The tensors follow the
// benchmark's mixed bundle: 4096 1-D tensors of 256 B to 64 KiB, log-uniform, five dtypes.
// A second loop times the arrangement a sender and a receiver in one process can use (the
// in-process transport): the receiver's plan is made from the header while the pack kernel
// runs, and the unpack follows the pack in stream order, so the host waits once.
// Prints one JSON line with the median phase times; exits non-zero when the tensors do not
// come back byte for byte.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "axon_rocm.h"

using Clock = std::chrono::steady_clock;
static double Us(Clock::time_point a, Clock::time_point b) {
  return std::chrono::duration<double, std::micro>(b - a).count();
}
#define CK(x)                                                              \
  do {                                                                     \
    int rc_ = (x);                                                         \
    if (rc_) {                                                             \
      std::fprintf(stderr, "%s -> %d: %s\n", #x, rc_, axr_last_error());   \
      return 1;                                                            \
    }                                                                      \
  } while (0)

int main(int argc, char** argv) {
  const int reps = argc > 1 ? std::atoi(argv[1]) : 100;
  const size_t n = 4096;
  std::mt19937_64 rng(1);
  std::vector<int64_t> shapes(n);
  std::vector<axr_tensor_t> src(n), dst(n);
  std::vector<uint64_t> offs(n), sizes(n);
  static const uint8_t kBits[5] = {16, 16, 32, 32, 8};
  static const uint8_t kCode[5] = {2, 4, 2, 0, 0};
  std::uniform_real_distribution<double> u(std::log(256.0), std::log(65536.0));
  uint64_t arena = 0;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t item = kBits[i % 5] / 8;
    sizes[i] = static_cast<uint64_t>(std::exp(u(rng))) / item * item;
    shapes[i] = static_cast<int64_t>(sizes[i] / item);
    offs[i] = arena;
    arena += (sizes[i] + 255) / 256 * 256 + 256 * (i % 3);   // gaps: the tensors do not lie back to back
  }
  void *a = nullptr, *b = nullptr, *payload = nullptr;
  CK(axr_mem_alloc(AXR_MEM_ROCM, arena, 256, &a));
  CK(axr_mem_alloc(AXR_MEM_ROCM, arena, 256, &b));
  std::vector<uint8_t> host(arena), back(arena);
  for (auto& x : host) x = static_cast<uint8_t>(rng());
  CK(axr_memcpy(AXR_MEM_ROCM, a, AXR_MEM_HOST, host.data(), arena));
  CK(axr_memset_async(b, 0, arena, nullptr));
  CK(axr_device_synchronize());
  for (size_t i = 0; i < n; ++i) {
    std::memset(&src[i], 0, sizeof(axr_tensor_t));
    src[i].data = static_cast<char*>(a) + offs[i];
    src[i].device_type = 10;   // kDLROCM
    src[i].ndim = 1;
    src[i].dtype_code = kCode[i % 5];
    src[i].dtype_bits = kBits[i % 5];
    src[i].dtype_lanes = 1;
    src[i].shape = &shapes[i];
    dst[i] = src[i];
    dst[i].data = static_cast<char*>(b) + offs[i];
  }
  axr_plan_t* probe = nullptr;
  CK(axr_plan_create(src.data(), n, 256, 0, &probe));
  uint64_t nbytes = 0;
  CK(axr_plan_payload_bytes(probe, &nbytes));
  CK(axr_plan_free(probe));
  CK(axr_mem_alloc(AXR_MEM_ROCM, nbytes, 256, &payload));
  void* stream = nullptr;
  CK(axr_stream_create(&stream));
  enum { kCreate, kPack, kWait1, kBind, kUnpack, kWait2, kFree, kTotal, kPhases };
  std::vector<double> t[kPhases];
  for (int it = 0; it < reps + 3; ++it) {
    CK(axr_stream_synchronize(stream));
    const auto t0 = Clock::now();
    axr_plan_t* p = nullptr;
    CK(axr_plan_create(src.data(), n, 256, 0, &p));
    const void* header = nullptr;
    size_t header_bytes = 0;
    CK(axr_plan_header(p, &header, &header_bytes));
    const auto t1 = Clock::now();
    CK(axr_pack(p, payload, nbytes, stream));
    const auto t2 = Clock::now();
    CK(axr_stream_synchronize(stream));
    const auto t3 = Clock::now();
    axr_plan_t* r = nullptr;
    CK(axr_plan_from_header_bind(header, header_bytes, dst.data(), n, &r));
    const auto t4 = Clock::now();
    CK(axr_unpack(r, payload, nbytes, stream));
    const auto t5 = Clock::now();
    CK(axr_stream_synchronize(stream));
    const auto t6 = Clock::now();
    CK(axr_plan_free(p));
    CK(axr_plan_free(r));
    const auto t7 = Clock::now();
    if (it >= 3) {
      t[kCreate].push_back(Us(t0, t1));
      t[kPack].push_back(Us(t1, t2));
      t[kWait1].push_back(Us(t2, t3));
      t[kBind].push_back(Us(t3, t4));
      t[kUnpack].push_back(Us(t4, t5));
      t[kWait2].push_back(Us(t5, t6));
      t[kFree].push_back(Us(t6, t7));
      t[kTotal].push_back(Us(t0, t6));
    }
  }
  std::vector<uint8_t> want(arena, 0);
  for (size_t i = 0; i < n; ++i) std::memcpy(want.data() + offs[i], host.data() + offs[i], sizes[i]);
  auto reproduced = [&]() {
    if (axr_memcpy(AXR_MEM_HOST, back.data(), AXR_MEM_ROCM, b, arena) != 0 || back != want) {
      std::fprintf(stderr, "the round trip did not reproduce the tensors\n");
      return false;
    }
    return true;
  };
  if (!reproduced()) return 2;
  // the same work with one wait: header decode and bind overlap the pack kernel
  std::vector<double> ordered;
  CK(axr_memset_async(b, 0, arena, stream));
  for (int it = 0; it < reps + 3; ++it) {
    CK(axr_stream_synchronize(stream));
    const auto t0 = Clock::now();
    axr_plan_t* p = nullptr;
    CK(axr_plan_create(src.data(), n, 256, 0, &p));
    const void* header = nullptr;
    size_t header_bytes = 0;
    CK(axr_plan_header(p, &header, &header_bytes));
    CK(axr_pack(p, payload, nbytes, stream));
    axr_plan_t* r = nullptr;
    CK(axr_plan_from_header_bind(header, header_bytes, dst.data(), n, &r));
    CK(axr_unpack(r, payload, nbytes, stream));
    CK(axr_stream_synchronize(stream));
    const auto t1 = Clock::now();
    CK(axr_plan_free(p));
    CK(axr_plan_free(r));
    if (it >= 3) ordered.push_back(Us(t0, t1));
  }
  if (!reproduced()) return 2;
  auto med = [](std::vector<double>& v) {
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
  };
  std::printf("{\"tensors\": %zu, \"payload_bytes\": %llu, \"repetitions\": %d, \"round_trip_us\": %.1f, "
              "\"us_per_1k_tensors\": %.2f, \"one_wait_round_trip_us\": %.1f, \"one_wait_us_per_1k_tensors\": %.2f, "
              "\"phases_us\": {\"plan_create_and_header\": %.1f, \"pack_call\": %.1f, "
              "\"wait_for_pack\": %.1f, \"plan_from_header_bind\": %.1f, \"unpack_call\": %.1f, "
              "\"wait_for_unpack\": %.1f, \"free_both_plans\": %.1f}}\n",
              n, static_cast<unsigned long long>(nbytes), reps, med(t[kTotal]), med(t[kTotal]) / (n / 1000.0),
              med(ordered), med(ordered) / (n / 1000.0),
              med(t[kCreate]), med(t[kPack]), med(t[kWait1]), med(t[kBind]), med(t[kUnpack]), med(t[kWait2]),
              med(t[kFree]));
  CK(axr_stream_destroy(stream));
  CK(axr_mem_free(AXR_MEM_ROCM, payload, nbytes));
  CK(axr_mem_free(AXR_MEM_ROCM, a, arena));
  CK(axr_mem_free(AXR_MEM_ROCM, b, arena));
  return 0;
}
