// Host-side fuzz of the planner and the header codec through the C ABI, meant to be
// built with AddressSanitizer and UBSan (tests/test_host_cpp.py does that) and to
// run without a GPU: random tensor descriptors (any rank up to 8, zero and negative
// strides, empty extents, sub-byte and wide dtypes, host and device tensors), every
// inspection call on the resulting plan, a decode of its header, and decodes of
// mutated headers, which must fail cleanly or give a plan that re-encodes to the
// same bytes.  Prints "plan_fuzz ok: ..." with its counts and exits 0.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "axon_rocm.h"

namespace {

std::mt19937_64 rng;

uint64_t pick(uint64_t lo, uint64_t hi) {   // inclusive
  return lo + rng() % (hi - lo + 1);
}

void die(const char* what, int rc) {
  std::fprintf(stderr, "plan_fuzz: %s -> %d (%s)\n", what, rc, axr_last_error());
  std::exit(1);
}

struct Case {
  std::vector<axr_tensor_t> tensors;
  std::vector<int64_t> dims;   // shapes and strides, stable storage
};

void make_case(Case* c) {
  const size_t n = pick(0, 12);
  c->tensors.assign(n, axr_tensor_t{});
  c->dims.assign(n * 16, 0);
  static const uint8_t bits[] = {1, 4, 8, 16, 32, 64, 128};
  static const int32_t devices[] = {10, 10, 10, 11, 1};
  for (size_t i = 0; i < n; ++i) {
    axr_tensor_t& t = c->tensors[i];
    t.ndim = static_cast<int32_t>(pick(0, 8));
    t.dtype_code = static_cast<uint8_t>(pick(0, 6));
    t.dtype_bits = bits[pick(0, 6)];
    t.dtype_lanes = static_cast<uint16_t>(pick(1, 2));
    t.device_type = devices[pick(0, 4)];
    t.device_id = 0;
    t.byte_offset = pick(0, 3) == 0 ? pick(0, 64) : 0;
    t.data = reinterpret_cast<void*>(0x7f0000000000ull + (i << 32) + pick(0, 255) * 16);
    int64_t* shape = c->dims.data() + i * 16;
    int64_t* strides = shape + 8;
    const uint64_t cap = t.ndim <= 2 ? 5000 : (t.ndim <= 4 ? 40 : 6);
    int64_t acc = 1;
    for (int d = t.ndim - 1; d >= 0; --d) {
      shape[d] = static_cast<int64_t>(pick(0, 20) == 0 ? 0 : pick(1, cap));
      switch (pick(0, 9)) {
        case 0: strides[d] = 0; break;                                     // broadcast
        case 1: strides[d] = -acc; break;                                  // backwards
        case 2: strides[d] = acc * static_cast<int64_t>(pick(2, 5)); break;   // stepped
        default: strides[d] = acc; break;
      }
      acc *= shape[d] > 0 ? shape[d] + static_cast<int64_t>(pick(0, 3)) : 1;
    }
    if (pick(0, 3) == 0 && t.ndim > 1) {   // permute two dimensions
      const int a = static_cast<int>(pick(0, t.ndim - 1)), b = static_cast<int>(pick(0, t.ndim - 1));
      std::swap(shape[a], shape[b]);
      std::swap(strides[a], strides[b]);
    }
    t.shape = t.ndim ? shape : nullptr;
    t.strides = (t.ndim && pick(0, 4) != 0) ? strides : nullptr;
  }
}

bool inspect(axr_plan_t* plan, size_t n) {
  uint64_t payload = 0, data = 0;
  size_t count = 0;
  if (int rc = axr_plan_payload_bytes(plan, &payload)) die("payload_bytes", rc);
  if (int rc = axr_plan_data_bytes(plan, &data)) die("data_bytes", rc);
  if (int rc = axr_plan_num_tensors(plan, &count)) die("num_tensors", rc);
  if (count != n || data > payload) die("counts", -1);
  std::vector<uint64_t> off(n + 1), size(n + 1);
  if (int rc = axr_plan_layout(plan, off.data(), size.data())) die("layout", rc);
  for (size_t i = 0; i < n; ++i) {
    axr_tensor_t meta;
    if (int rc = axr_plan_tensor_meta(plan, i, &meta)) die("tensor_meta", rc);
    uint64_t nbytes = 0;
    if (int rc = axr_tensor_nbytes(&meta, &nbytes)) die("tensor_nbytes", rc);
    if (nbytes != size[i] || off[i] + size[i] > payload) die("layout consistency", -1);
  }
  // tables: unsupported layouts (2^31 runs in element mode ...) may be refused, never crash
  size_t nseg = 0;
  int rc = axr_plan_segments(plan, nullptr, 0, &nseg);
  if (rc == AXR_OK) {
    std::vector<axr_segment_info_t> segs(nseg + 1);
    if (int rc2 = axr_plan_segments(plan, segs.data(), nseg, &nseg)) die("segments", rc2);
    axr_launch_info_t info;
    if (int rc2 = axr_plan_launch_info(plan, &info)) die("launch_info", rc2);
    uint64_t tiles = 0;
    for (size_t i = 0; i < nseg; ++i)
      if (segs[i].mode != 4) tiles += segs[i].tiles;
    if (tiles != info.tiles) die("tile count", -1);
  } else if (rc != AXR_ERR_UNSUPPORTED && rc != AXR_ERR_INVALID) {
    die("segments", rc);
  }
  return rc == AXR_OK;
}

}  // namespace

int main(int argc, char** argv) {
  const uint64_t seed = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 1;
  const int rounds = argc > 2 ? std::atoi(argv[2]) : 3000;
  rng.seed(seed);
  static const uint32_t aligns[] = {1, 2, 16, 64, 256, 4096};
  long plans = 0, tables = 0, decodes = 0, accepted = 0;
  for (int r = 0; r < rounds; ++r) {
    Case c;
    make_case(&c);
    const size_t n = c.tensors.size();
    axr_plan_t* plan = nullptr;
    int rc = axr_plan_create(n ? c.tensors.data() : nullptr, n, aligns[pick(0, 5)], 0, &plan);
    if (rc != AXR_OK) {   // refused descriptors (overflowing sizes ...) leave nothing behind
      if (plan) die("plan set on failure", rc);
      continue;
    }
    ++plans;
    if (inspect(plan, n)) ++tables;
    const void* header = nullptr;
    size_t length = 0;
    if (int rc2 = axr_plan_header(plan, &header, &length)) die("header", rc2);
    std::vector<uint8_t> bytes(static_cast<const uint8_t*>(header),
                               static_cast<const uint8_t*>(header) + length);
    axr_plan_t* back = nullptr;
    if (int rc2 = axr_plan_from_header(bytes.data(), bytes.size(), &back)) die("from_header", rc2);
    uint64_t a = 0, b = 0;
    axr_plan_payload_bytes(plan, &a);
    axr_plan_payload_bytes(back, &b);
    if (a != b) die("decoded payload size", -1);
    // binding tensors of other shapes must be refused, the same shapes accepted
    rc = axr_plan_bind(back, n ? c.tensors.data() : nullptr, n);
    if (rc != AXR_OK && rc != AXR_ERR_MISMATCH) die("bind", rc);
    if (rc == AXR_OK) inspect(back, n);
    {   // the same in one pass: same result, same tables
      axr_plan_t* fused = nullptr;
      const int rc1 = axr_plan_from_header_bind(bytes.data(), bytes.size(), n ? c.tensors.data() : nullptr, n, &fused);
      if (rc1 != rc) die("from_header_bind result differs from from_header + bind", rc1);
      if (rc1 == AXR_OK) {
        inspect(fused, n);
        size_t c1 = 0, c2 = 0;
        axr_plan_segments(fused, nullptr, 0, &c1);
        axr_plan_segments(back, nullptr, 0, &c2);
        if (c1 != c2) die("from_header_bind segment count", -1);
        axr_plan_free(fused);
      } else if (fused) {
        die("plan set on failed from_header_bind", rc1);
      }
    }
    axr_plan_free(back);

    for (int m = 0; m < 8; ++m) {   // mutated headers
      std::vector<uint8_t> mutated = bytes;
      switch (pick(0, 4)) {
        case 0: mutated.resize(pick(0, mutated.size())); break;
        case 1: if (!mutated.empty()) mutated[pick(0, mutated.size() - 1)] ^= static_cast<uint8_t>(1u << pick(0, 7)); break;
        case 2: if (!mutated.empty()) mutated[pick(0, mutated.size() - 1)] = static_cast<uint8_t>(pick(0, 255)); break;
        case 3: mutated.insert(mutated.end(), pick(1, 40), static_cast<uint8_t>(pick(0, 255))); break;
        default:
          if (mutated.size() >= 16) {   // huge counts
            const uint32_t big = static_cast<uint32_t>(pick(0x7fffff00u, 0xffffffffu));
            std::memcpy(mutated.data() + (pick(0, 1) ? 8 : 12), &big, 4);
          }
      }
      axr_plan_t* p = nullptr;
      // exact-size heap copy so that a read past the end is an ASan error
      uint8_t* heap = static_cast<uint8_t*>(std::malloc(mutated.size() ? mutated.size() : 1));
      std::memcpy(heap, mutated.data(), mutated.size());
      {   // mutated headers through the one-pass call too (its result is only freed)
        axr_plan_t* q = nullptr;
        const int rq = axr_plan_from_header_bind(heap, mutated.size(), n ? c.tensors.data() : nullptr, n, &q);
        if (rq == AXR_OK) axr_plan_free(q);
        else if (q) die("plan set on failed from_header_bind", rq);
      }
      rc = axr_plan_from_header(heap, mutated.size(), &p);
      ++decodes;
      if (rc == AXR_OK) {
        ++accepted;
        const void* h2 = nullptr;
        size_t l2 = 0;
        if (int rc2 = axr_plan_header(p, &h2, &l2)) die("header of decoded", rc2);
        if (l2 != mutated.size() || std::memcmp(h2, heap, l2) != 0) die("accepted header does not re-encode", -1);
        axr_plan_free(p);
      } else if (p) {
        die("plan set on failed decode", rc);
      }
      std::free(heap);
    }
    axr_plan_free(plan);
  }
  {   // sizes that wrap 64 bits: refused at creation and in a crafted header
    int64_t huge = int64_t(1) << 62;
    axr_tensor_t t[2];
    std::memset(t, 0, sizeof(t));
    for (axr_tensor_t& x : t) {
      x.data = reinterpret_cast<void*>(0x1000);
      x.device_type = 10;
      x.ndim = 1;
      x.dtype_code = 1;
      x.dtype_bits = 16;
      x.dtype_lanes = 1;
      x.shape = &huge;
    }
    axr_plan_t* p = nullptr;
    if (axr_plan_create(t, 2, 1, 0, &p) != AXR_ERR_INVALID || p) die("wrapping sizes accepted", -1);
    uint8_t h[24 + 2 * 48];
    const uint32_t magic = 0x42545841u, n = 2, align = 1;
    const uint16_t version = 1, flags = 0;
    const uint64_t payload = 0, nbytes = uint64_t(1) << 63, zero = 0;
    uint8_t* w = h;
    auto emit = [&w](const void* src, size_t len) { std::memcpy(w, src, len); w += len; };
    emit(&magic, 4); emit(&version, 2); emit(&flags, 2); emit(&n, 4); emit(&align, 4); emit(&payload, 8);
    for (int i = 0; i < 2; ++i) {
      const uint64_t off = i ? nbytes : 0;
      const int32_t dev = 10, id = 0, ndim = 1;
      const uint8_t code = 1, bits = 16;
      const uint16_t lanes = 1;
      emit(&off, 8); emit(&nbytes, 8); emit(&dev, 4); emit(&id, 4); emit(&ndim, 4);
      emit(&code, 1); emit(&bits, 1); emit(&lanes, 2); emit(&zero, 8); emit(&huge, 8);
    }
    if (axr_plan_from_header(h, sizeof(h), &p) != AXR_ERR_HEADER || p) die("wrapping header accepted", -1);
  }
  std::printf("plan_fuzz ok: %ld plans, %ld with tables, %ld mutated headers decoded, %ld of them valid\n",
              plans, tables, decodes, accepted);
  return 0;
}
