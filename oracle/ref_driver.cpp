// ref_driver.cpp - thin extern "C" driver over the REAL reference classes.
//
// TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile together with the
// reference's own ucx_context/ucx_memory_resource.cpp, taken where it lies
// under the reference tree (REF=/root/reference), into oracle/_ref/.  It
// validates oracle/bundle_oracle.c and serves as the "reference" CPU baseline:
// every copy goes through DefaultUcxMemoryResourceManager::memcpy, i.e. a
// std::function wrapping std::memcpy (ucx_context/ucx_memory_resource.cpp:28-42,
// 106-110), in the loop shape of ucx_am_context_test.cpp:1740-1751.
#include <chrono>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <vector>
#include <algorithm>

#include "ucx_context/ucx_context_data.hpp"
#include "ucx_context/ucx_context_def.h"
#include "ucx_context/ucx_memory_resource.hpp"

using eux::ucxx::DefaultUcxMemoryResourceManager;
using eux::ucxx::UcxBuffer;
using eux::ucxx::UcxBufferVec;

namespace {
DefaultUcxMemoryResourceManager& mr() {
  static DefaultUcxMemoryResourceManager m;
  return m;
}
}  // namespace

extern "C" {

__attribute__((visibility("default"))) void ref_pack(const void* const* srcs,
                                                     const uint64_t* sizes, size_t n, void* dst) {
  size_t offset = 0;
  for (size_t i = 0; i < n; ++i) {
    mr().memcpy(ucx_memory_type::HOST, static_cast<char*>(dst) + offset, ucx_memory_type::HOST,
                srcs[i], sizes[i]);
    offset += sizes[i];
  }
}

__attribute__((visibility("default"))) void ref_unpack(const void* src, const uint64_t* sizes,
                                                       size_t n, void* const* dsts) {
  size_t offset = 0;
  for (size_t i = 0; i < n; ++i) {
    mr().memcpy(ucx_memory_type::HOST, dsts[i], ucx_memory_type::HOST,
                static_cast<const char*>(src) + offset, sizes[i]);
    offset += sizes[i];
  }
}

// UcxBuffer::to_buffer_vec over caller memory (non-owning).  0 ok, -1 length_error.
__attribute__((visibility("default"))) int ref_split(void* base, uint64_t size,
                                                     const uint64_t* sizes, size_t n,
                                                     void** views, uint64_t* view_sizes) {
  try {
    UcxBuffer buffer(mr(), ucx_memory_type::HOST, base, size, nullptr, false);
    std::vector<size_t> sz(sizes, sizes + n);
    UcxBufferVec vec = std::move(buffer).to_buffer_vec(sz);
    if (vec.size() != n) return -2;
    for (size_t i = 0; i < n; ++i) {
      views[i] = vec[i].data;
      view_sizes[i] = vec[i].size;
    }
    // the source must have been invalidated (ucx_context_data_test.cpp:72-74)
    if (buffer.data() != nullptr || buffer.size() != 0) return -3;
    return 0;
  } catch (const std::length_error&) {
    return -1;
  }
}

// Release-function ownership of the live UcxBuffer, the scenario of
// ucx_context_data_test.cpp:85-128: an external 16-byte block with a release
// callback is moved into a second buffer with own_buffer = `own`.  Returns how
// often the callback ran once both buffers are gone, or a negative number when
// an intermediate state differs from what that test expects.
__attribute__((visibility("default"))) int ref_release_count(int own) {
  int release_count = 0;
  auto* external = new uint8_t[16];
  int state = 0;
  {
    UcxBuffer buffer(mr(), ucx_memory_type::HOST, external, 16, nullptr, true,
                     [&release_count](void* ptr) {
                       ++release_count;
                       delete[] static_cast<uint8_t*>(ptr);
                     });
    auto moved = UcxBuffer(std::move(buffer), own != 0);
    if (buffer.data() != nullptr || buffer.own_buffer()) state = -1;
    if (moved.data() != external || moved.own_buffer() != (own != 0)) state = -2;
  }
  if (!own) delete[] external;
  return state ? state : release_count;
}

// Median seconds of one pack + unpack through the reference memcpy dispatch.
__attribute__((visibility("default"))) double ref_time_pack_unpack(
    const void* const* srcs, void* const* dsts, const uint64_t* sizes, size_t n, void* packed,
    int warmup, int reps) {
  std::vector<double> t;
  for (int r = -warmup; r < reps; ++r) {
    auto a = std::chrono::steady_clock::now();
    ref_pack(srcs, sizes, n, packed);
    ref_unpack(packed, sizes, n, dsts);
    auto b = std::chrono::steady_clock::now();
    if (r >= 0) t.push_back(std::chrono::duration<double>(b - a).count());
  }
  std::sort(t.begin(), t.end());
  return t[t.size() / 2];
}

}  // extern "C"
