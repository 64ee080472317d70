// The host-side copy helper of the staging paths against plain memcpy: random job lists
// (many small pieces, a few large ones, empty ones), every thread count, with the bytes
// around every destination checked for overruns.  Built with AddressSanitizer by
// tests/test_host_cpp.py; needs no GPU.  Prints "host_copy_check ok <cases>".
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "axr_internal.h"

int main() {
  std::mt19937_64 rng(11);
  auto pick = [&](uint64_t lo, uint64_t hi) { return lo + rng() % (hi - lo + 1); };
  long cases = 0;
  for (int round = 0; round < 25; ++round) {
    const size_t njobs = pick(0, 40);
    std::vector<size_t> sizes(njobs);
    size_t total = 0;
    for (size_t& n : sizes) {
      const uint64_t kind = pick(0, 9);
      n = kind == 0 ? 0 : (kind < 7 ? pick(1, 70000) : pick(1u << 20, 5u << 20));
      total += n;
    }
    std::vector<uint8_t> src(total + 1), want(total + 64 * (njobs + 1), 0xEE), got;
    for (size_t i = 0; i < total; ++i) src[i] = static_cast<uint8_t>(rng());
    // destinations: 32 guard bytes between jobs
    std::vector<axr::HostCopyJob> jobs(njobs);
    got = want;
    size_t s_at = 0, d_at = 32;
    for (size_t j = 0; j < njobs; ++j) {
      std::memcpy(want.data() + d_at, src.data() + s_at, sizes[j]);
      jobs[j] = {got.data() + d_at, src.data() + s_at, sizes[j]};
      s_at += sizes[j];
      d_at += sizes[j] + 32;
    }
    for (int64_t threads : {1, 2, 3, 4, 7, 16}) {
      if (axr_tune_set("host_threads", threads) != AXR_OK) return 1;
      std::vector<uint8_t> out = got;   // fresh guard pattern every time
      std::vector<axr::HostCopyJob> mine = jobs;
      for (axr::HostCopyJob& job : mine)
        job.dst = out.data() + (static_cast<uint8_t*>(job.dst) - got.data());
      axr::host_copy(mine.data(), mine.size());
      if (out != want) {
        std::fprintf(stderr, "host_copy_check: mismatch in round %d with %lld threads\n", round,
                     static_cast<long long>(threads));
        return 1;
      }
      ++cases;
    }
  }
  std::printf("host_copy_check ok %ld\n", cases);
  return 0;
}
