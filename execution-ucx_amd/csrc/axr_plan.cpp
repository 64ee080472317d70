// Bundle planner: layout, header codec, segment-table construction and the
// pack / unpack entry points.
//
// Reference behaviour restated here:
//   - size rule     rpc_core/utils/tensor_meta.hpp:91-104 (CalculateTensorSize)
//   - tensor order  axon/python/src/bindings_runtime_helpers.hpp:351-414
//   - tight concat  ucx_context/ucx_am_context/ucx_am_connection_test.cpp:1051-1108
//   - split         ucx_context/ucx_context_data.hpp:641-665 (to_buffer_vec)
//
// Header wire format (all little-endian, no padding):
//   u32 magic 0x42545841 ("AXTB") | u16 version=1 | u16 flags=0 |
//   u32 n_tensors | u32 align | u64 payload_bytes
//   then per tensor:
//   u64 offset | u64 nbytes | i32 device_type | i32 device_id | i32 ndim |
//   u8 dtype_code | u8 dtype_bits | u16 dtype_lanes | u64 byte_offset (=0) |
//   i64 shape[ndim]
// These are the fields of TensorMeta (tensor_meta.hpp:77-82) plus the packed
// offset and size; strides are not sent because packed tensors are compact.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>

#include "axr_internal.h"

using namespace axr;

namespace {

// Storage the planner fills itself: growing it initialises nothing (a std::vector would
// clear hundreds of kilobytes per plan that the next loop overwrites), and elements are
// plain records.
template <typename T>
class RawVec {
 public:
  RawVec() = default;
  RawVec(const RawVec&) = delete;
  RawVec& operator=(const RawVec&) = delete;
  ~RawVec() { std::free(ptr_); }
  size_t size() const { return n_; }
  size_t capacity() const { return cap_; }
  bool empty() const { return n_ == 0; }
  T* data() { return ptr_; }
  const T* data() const { return ptr_; }
  T& operator[](size_t i) { return ptr_[i]; }
  const T& operator[](size_t i) const { return ptr_[i]; }
  T* begin() { return ptr_; }
  T* end() { return ptr_ + n_; }
  const T* begin() const { return ptr_; }
  const T* end() const { return ptr_ + n_; }
  void clear() { n_ = 0; }
  void reserve(size_t m) {
    if (m <= cap_) return;
    if (m > SIZE_MAX / sizeof(T)) throw std::bad_alloc();
    T* q = static_cast<T*>(std::realloc(ptr_, m * sizeof(T)));
    if (!q) throw std::bad_alloc();
    ptr_ = q;
    cap_ = m;
  }
  void resize(size_t m) {   // new elements hold whatever the memory held
    reserve(m);
    n_ = m;
  }
  void assign(const T* first, const T* last) {
    resize(static_cast<size_t>(last - first));
    if (n_) std::memcpy(ptr_, first, n_ * sizeof(T));
  }
  void swap(RawVec& o) {
    std::swap(ptr_, o.ptr_);
    std::swap(n_, o.n_);
    std::swap(cap_, o.cap_);
  }

 private:
  T* ptr_ = nullptr;
  size_t n_ = 0, cap_ = 0;
};

constexpr uint32_t kMagic = 0x42545841u;
constexpr uint16_t kVersion = 1;
constexpr size_t kFixedHeader = 24;
constexpr size_t kTensorHeader = 40;
constexpr int32_t kDLCPU = 1, kDLROCM = 10, kDLROCMHost = 11;
constexpr int kMaxNdim = 64;

struct TensorRec {          // 56 bytes
  uint64_t address = 0;     // data + byte_offset, 0 when unbound
  uint64_t offset = 0, nbytes = 0;
  uint32_t shape_at = 0;    // index into plan->dims64
  uint32_t strides_at = 0;
  int32_t device_type = 0, device_id = 0, ndim = 0;
  uint8_t code = 0, bits = 0;
  uint16_t lanes = 0;
  bool has_strides = false;
};

struct HostCopy {
  uint64_t host;
  uint64_t offset;
  uint64_t bytes;
};

// Host tensors travel through pinned staging blocks: one device copy per chunk
// of neighbouring pieces instead of one pageable copy per piece.
constexpr size_t kStageBytes = 8u << 20;
struct HostChunk {
  uint32_t first, count;     // range of host_copies
  uint64_t begin, end;       // payload byte range the chunk spans
};
struct HostStage {
  TableBlock block;
  hipEvent_t ready = nullptr;   // recorded after the device copy that uses the block
  bool pending = false;
};

template <typename T>
T get(const uint8_t* p) {
  T x;
  std::memcpy(&x, p, sizeof(T));
  return x;
}

// `a` is a power of two everywhere (check_align, table sections): no division per tensor
uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) & ~(a - 1); }

bool mul_overflow(uint64_t a, uint64_t b, uint64_t* out) {
  return __builtin_mul_overflow(a, b, out);
}

inline int nbytes_rule(int32_t ndim, const int64_t* shape, uint8_t bits, uint64_t* out) {
  if (ndim == 0) {   // the reference sizes a 0-d tensor as 0 bytes
    *out = 0;
    return AXR_OK;
  }
  if (ndim < 0 || ndim > kMaxNdim) return fail(AXR_ERR_INVALID, "tensor ndim out of range");
  if (!shape) return fail(AXR_ERR_INVALID, "tensor shape is null for ndim > 0");
  if (ndim == 1 && shape[0] >= 0 && shape[0] < (int64_t(1) << 56)) {   // the common case, no overflow possible
    *out = static_cast<uint64_t>(shape[0]) * ((static_cast<uint64_t>(bits) + 7) / 8);
    return AXR_OK;
  }
  uint64_t elems = 1;
  for (int32_t i = 0; i < ndim; ++i) {
    if (shape[i] < 0) return fail(AXR_ERR_INVALID, "negative tensor extent");
    if (mul_overflow(elems, static_cast<uint64_t>(shape[i]), &elems)) {
      // keep multiplying only to see whether a zero extent follows
      bool zero = false;
      for (int32_t j = 0; j < ndim; ++j) zero = zero || shape[j] == 0;
      if (!zero) return fail(AXR_ERR_INVALID, "tensor element count overflows 64 bits");
      elems = 0;
      break;
    }
  }
  const uint64_t item = (static_cast<uint64_t>(bits) + 7) / 8;
  if (mul_overflow(elems, item, out)) return fail(AXR_ERR_INVALID, "tensor size overflows 64 bits");
  return AXR_OK;
}

}  // namespace

struct axr_plan {
  uint32_t align = 1;
  RawVec<TensorRec> tensors;
  std::vector<int64_t> dims64;       // shapes and strides of all tensors
  RawVec<TensorRec> staged_tensors;  // axr_plan_bind fills these and swaps on success
  std::vector<int64_t> staged_dims64;
  uint64_t payload_bytes = 0, data_bytes = 0;
  RawVec<uint8_t> header;
  bool bound = false;
  bool receiver = false;             // made by axr_plan_from_header: tiles are anchored on the tensor side

  // device tables
  bool tables_built = false;
  bool device_built = false;         // the device built its tables itself from compact records
  std::vector<Seg> segs;
  std::vector<Dims> dims;
  std::vector<uint32_t> wave_seg;
  std::vector<uint32_t> seg_tensor;  // tensor index per segment (inspection)
  std::vector<uint8_t> group_blocks; // kGroupBlockBytes per group tile: GroupHead, then Member records
  std::vector<uint32_t> member_tensor;   // kGroupMaxMembers tensor indices per block (inspection)
  bool groups_only = false;          // every tile is a group tile: the kernel walks the blocks directly
  bool pinned_host_tensors = false;  // some tensor lies in device-visible host memory (kDLROCMHost)
  std::vector<HostCopy> host_copies;
  std::vector<uint32_t> host_copy_tensor;
  std::vector<HostChunk> host_chunks;
  HostStage stage[2];
  bool overlapping_dst = false;      // some tensor has a zero stride over an extent > 1
  uint32_t ntiles = 0;
  uint64_t shared_line_tiles = 0;    // tiles of transposed blocks whose rows straddle 128-byte lines
  LaunchConfig cfg;
  TableBlock block;
  size_t table_bytes = 0;
  size_t dims_at = 0, wave_at = 0, members_at = 0;
  bool uploaded = false;
  bool resident = false;             // upload known to be complete (axr_plan_prepare)
  size_t stage_bytes = 0;            // longest host chunk: size of the staging blocks
  std::unique_ptr<InlineTables> inline_tables;   // the tables as a kernel argument (small bundles)
  bool inline_ready = false;
  uint64_t launches = 0;             // kernel launches since the tables were built
  hipEvent_t upload_event = nullptr;   // from event_acquire
  int upload_event_device = -1;
  hipStream_t upload_stream = nullptr;
  struct BusyStream {
    hipStream_t stream;
    uint64_t mark;   // stream_mark_launch() of the plan's latest launch there
  };
  std::vector<BusyStream> busy_streams;    // streams with launches since the last quiesce

  const int64_t* shape_of(const TensorRec& t) const { return dims64.data() + t.shape_at; }
  const int64_t* strides_of(const TensorRec& t) const {
    return t.has_strides ? dims64.data() + t.strides_at : nullptr;
  }
};

namespace {

// Plans of thousands of tensors hold about a megabyte in vectors; fresh ones of that size
// come from mmap and are paged in on first touch, which costs more than filling them.  A few
// released plans are therefore kept, emptied, and handed out again with their capacity.
struct PlanShells {
  std::mutex mu;
  std::vector<axr_plan*> idle;
  ~PlanShells() {
    for (axr_plan* p : idle) delete p;
  }
};
PlanShells& plan_shells() {
  static PlanShells shells;
  return shells;
}
constexpr size_t kMaxIdlePlans = 8;
constexpr size_t kMaxIdlePlanBytes = 32u << 20;

axr_plan* plan_new() {
  {
    PlanShells& shells = plan_shells();
    std::lock_guard<std::mutex> lock(shells.mu);
    if (!shells.idle.empty()) {
      axr_plan* p = shells.idle.back();
      shells.idle.pop_back();
      return p;
    }
  }
  return new (std::nothrow) axr_plan();
}

// The plan owns no device resource any more; keeps the vectors' capacity, resets the rest.
void plan_delete(axr_plan* p) {
  auto keep = [](auto& v) {
    v.clear();
    return v.capacity() * sizeof(v[0]);
  };
  RawVec<TensorRec> tensors, tensors2;
  std::vector<int64_t> dims64, dims64_2;
  RawVec<uint8_t> header;
  std::vector<Seg> segs;
  std::vector<Dims> dims;
  std::vector<uint32_t> wave_seg, seg_tensor, member_tensor;
  std::vector<uint8_t> group_blocks;
  tensors.swap(p->tensors);
  dims64.swap(p->dims64);
  tensors2.swap(p->staged_tensors);
  dims64_2.swap(p->staged_dims64);
  header.swap(p->header);
  segs.swap(p->segs);
  dims.swap(p->dims);
  wave_seg.swap(p->wave_seg);
  seg_tensor.swap(p->seg_tensor);
  member_tensor.swap(p->member_tensor);
  group_blocks.swap(p->group_blocks);
  const size_t bytes = keep(tensors) + keep(dims64) + keep(header) + keep(segs) + keep(dims) + keep(wave_seg) +
                       keep(tensors2) + keep(dims64_2) + keep(seg_tensor) + keep(member_tensor) + keep(group_blocks);
  if (bytes > kMaxIdlePlanBytes) {
    delete p;
    return;
  }
  p->~axr_plan();
  new (p) axr_plan();
  tensors.swap(p->tensors);
  dims64.swap(p->dims64);
  tensors2.swap(p->staged_tensors);
  dims64_2.swap(p->staged_dims64);
  header.swap(p->header);
  segs.swap(p->segs);
  dims.swap(p->dims);
  wave_seg.swap(p->wave_seg);
  seg_tensor.swap(p->seg_tensor);
  member_tensor.swap(p->member_tensor);
  group_blocks.swap(p->group_blocks);
  PlanShells& shells = plan_shells();
  std::lock_guard<std::mutex> lock(shells.mu);
  if (shells.idle.size() < kMaxIdlePlans) {
    shells.idle.push_back(p);
    return;
  }
  delete p;   // (under the lock: rare, and the plan is empty)
}

// A plan under construction: given back to the shells unless it is released to the caller,
// also when an allocation throws on the way.
struct PlanInProgress {
  axr_plan* p;
  explicit PlanInProgress(axr_plan* plan) : p(plan) {}
  PlanInProgress(const PlanInProgress&) = delete;
  PlanInProgress& operator=(const PlanInProgress&) = delete;
  ~PlanInProgress() {
    if (p) plan_delete(p);
  }
  axr_plan* release() {
    axr_plan* out = p;
    p = nullptr;
    return out;
  }
};

// One tensor's record of the header, as it lies on the wire (little-endian targets only).
#pragma pack(push, 1)
struct WireTensor {
  uint64_t offset, nbytes;
  int32_t device_type, device_id, ndim;
  uint8_t code, bits;
  uint16_t lanes;
  uint64_t byte_offset;
};
#pragma pack(pop)
static_assert(sizeof(WireTensor) == kTensorHeader, "header record layout");

// The fixed part of the header; the per-tensor records are written while the tensors are read.
void encode_preamble(axr_plan* p) {
  uint8_t* w = p->header.data();
  const uint32_t magic = kMagic, n = static_cast<uint32_t>(p->tensors.size()), align = p->align;
  const uint16_t version = kVersion, flags = 0;
  std::memcpy(w, &magic, 4);
  std::memcpy(w + 4, &version, 2);
  std::memcpy(w + 6, &flags, 2);
  std::memcpy(w + 8, &n, 4);
  std::memcpy(w + 12, &align, 4);
  std::memcpy(w + 16, &p->payload_bytes, 8);
}

int check_align(uint32_t align) {
  if (align == 0 || (align & (align - 1)) || align > kMaxAlign)
    return fail(AXR_ERR_INVALID, "align must be a power of two in [1, 4096]");
  return AXR_OK;
}

void invalidate_tables(axr_plan* p) {
  p->tables_built = false;
  p->device_built = false;
  p->uploaded = false;
  p->resident = false;
  p->inline_ready = false;
  p->launches = 0;
  p->segs.clear();
  p->dims.clear();
  p->wave_seg.clear();
  p->seg_tensor.clear();
  p->group_blocks.clear();
  p->member_tensor.clear();
  p->groups_only = false;
  p->pinned_host_tensors = false;
  p->host_copies.clear();
  p->host_copy_tensor.clear();
  p->host_chunks.clear();
  p->overlapping_dst = false;
  p->ntiles = 0;
  p->shared_line_tiles = 0;
  p->cfg.lds_per_wave = 0;
}

// Wait until the device no longer reads the plan's tables.  No event is
// recorded per launch (it would put a barrier packet between back-to-back
// bundles); the streams used since the last call are drained instead.  A stream
// that axr_stream_destroy has destroyed in the meantime is not touched again
// (HIP dereferences the handle): hipStreamDestroy may return before the
// stream's work has finished, so the whole device is drained for it.
void quiesce(axr_plan* p) {
  bool whole_device = false;
  for (const axr_plan::BusyStream& b : p->busy_streams) {
    hipStream_t s = b.stream;
    if (s && stream_retired(s)) {
      whole_device = true;
    } else if (stream_drained(s, b.mark)) {
      // axr_stream_synchronize has seen the stream pass the plan's last launch
    } else {
      const uint64_t reached = stream_launch_mark();
      if (hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        whole_device = true;
      } else {
        stream_note_drained(s, reached);
      }
    }
  }
  if (whole_device) (void)hipDeviceSynchronize();
  p->busy_streams.clear();
}

// The plan has just enqueued work on `stream`.
void remember_stream(axr_plan* p, hipStream_t stream) {
  const uint64_t mark = stream_mark_launch();
  for (axr_plan::BusyStream& b : p->busy_streams) {
    if (b.stream == stream) {
      b.mark = mark;
      return;
    }
  }
  p->busy_streams.push_back({stream, mark});
}

// ------------------------------------------------------------ table building

// Outer (strided) dimensions and the contiguous inner run of one tensor, in
// fixed storage: planning a bundle of thousands of tensors must not allocate
// per tensor.
struct Collapsed {
  uint64_t extent[kMaxNdim];   // outer dims, outermost first
  int64_t stride[kMaxNdim];    // bytes
  size_t nd = 0;
  uint64_t run_bytes = 0;
};

// Reduce (shape, element strides) to the fewest strided outer dimensions plus
// one contiguous inner run.  Extent-1 dims vanish; adjacent dims that together
// address a regular span merge.
void collapse(const TensorRec& t, const int64_t* shape, const int64_t* strides, uint64_t item,
              Collapsed* c) {
  c->nd = 0;
  // merged dims, innermost first
  uint64_t me[kMaxNdim];
  int64_t ms[kMaxNdim];
  size_t nm = 0;
  int64_t dense = static_cast<int64_t>(item);   // row-major stride of the current dim
  for (int32_t d = t.ndim - 1; d >= 0; --d) {
    const int64_t row_major = dense;
    dense *= shape[d];
    if (shape[d] == 1) continue;
    const int64_t st = strides ? strides[d] * static_cast<int64_t>(item) : row_major;
    if (nm && st == ms[nm - 1] * static_cast<int64_t>(me[nm - 1])) {
      me[nm - 1] *= static_cast<uint64_t>(shape[d]);   // this dim continues the inner one
    } else {
      me[nm] = static_cast<uint64_t>(shape[d]);
      ms[nm] = st;
      ++nm;
    }
  }
  size_t first_outer = 0;
  if (nm && ms[0] == static_cast<int64_t>(item)) {
    c->run_bytes = me[0] * item;
    first_outer = 1;
  } else {
    c->run_bytes = item;
  }
  for (size_t i = nm; i-- > first_outer;) {
    c->extent[c->nd] = me[i];
    c->stride[c->nd] = ms[i];
    ++c->nd;
  }
}

// Largest power of two up to 16 that divides the run length.
uint32_t granule_of(uint64_t run_bytes) {
  uint32_t g = 16;
  while (g > 1 && (run_bytes % g) != 0) g >>= 1;
  return g;
}

// Runs shorter than this move in element mode.  With 16-byte granules (exact or ragged)
// element mode is ahead of run tiles up to runs of about 1 KiB and level with them from
// 1280 bytes on; narrower granules move fewer bytes per access and lose to the
// (length-agnostic) run-tile copy much earlier.
uint64_t element_mode_limit(uint64_t run_bytes) {
  const uint64_t limit = static_cast<uint64_t>(tunables().gather_run_bytes);
  if (granule_of(run_bytes) == 16) return limit;
  if (run_bytes >= kVecBytes && tunables().ragged_runs != 0) return limit;
  return (limit + 4) / 5;
}

struct Builder {
  axr_plan* p;
  uint32_t tile_bytes;    // rows * 1 KiB with rows a power of two
  uint32_t tile_shift;    // log2(tile_bytes)
  uint64_t head_align;    // 0 or a power of two up to 128
  uint64_t tiles = 0;
  uint64_t shared_line_tiles = 0;   // transposed blocks whose rows straddle 128-byte lines
  uint64_t group_bytes = 0;         // longest tensor that may share a wavefront (0: none)
  uint32_t slots_per_group = kGroupMaxSlots;
  // the group being collected (when open): the last block of p->group_blocks
  bool group_open = false;
  uint32_t group_count = 0;
  uint32_t group_slots = 0;
  uint64_t group_off = 0;
  uint64_t group_starts[2] = {0, 0};

  uint8_t* open_block() { return p->group_blocks.data() + p->group_blocks.size() - kGroupBlockBytes; }

  // A short contiguous device tensor joins the open group, which is closed first when the
  // tensor does not fit (16 members, 128 lane slots, offsets within 1 MiB of the first).
  // Returns false for a tensor that cannot be a member at all.
  bool add_member(uint32_t tensor, uint64_t ptr, uint64_t off, uint64_t nbytes, uint64_t pad, int* rc) {
    *rc = AXR_OK;
    if (group_bytes == 0 || nbytes == 0 || nbytes > group_bytes || nbytes > kGroupMaxMemberBytes || pad >= kMaxAlign)
      return false;
    const uint32_t need = group_data_slots(static_cast<uint32_t>(nbytes)) + group_pad_slots(static_cast<uint32_t>(pad));
    if (need > slots_per_group / 2) return false;
    if (group_open && (group_count >= kGroupMaxMembers || group_slots + need > slots_per_group ||
                       off < group_off || off - group_off >= (1ull << kMemberOffBits))) {
      *rc = close_group();
      if (*rc) return true;
    }
    if (!group_open) {
      group_open = true;
      group_count = 0;
      group_slots = 0;
      group_off = off;
      group_starts[0] = group_starts[1] = 0;
      p->group_blocks.resize(p->group_blocks.size() + kGroupBlockBytes, 0);
      p->member_tensor.resize(p->member_tensor.size() + kGroupMaxMembers, 0);
    }
    Member m;
    m.ptr = ptr;
    m.off_pad = static_cast<uint32_t>(off - group_off) | static_cast<uint32_t>(pad) << kMemberOffBits;
    m.nbytes = static_cast<uint16_t>(nbytes);
    m.begin = static_cast<uint16_t>(group_slots);
    std::memcpy(open_block() + sizeof(GroupHead) + group_count * sizeof(Member), &m, sizeof(m));
    p->member_tensor[p->member_tensor.size() - kGroupMaxMembers + group_count] = tensor;
    group_starts[group_slots >> 6] |= 1ull << (group_slots & 63u);
    ++group_count;
    group_slots += need;
    return true;
  }

  // Ends the open group: one tile for two members or more, an ordinary segment for one.
  int close_group() {
    if (!group_open) return AXR_OK;
    group_open = false;
    if (group_count == 1) {
      Member m;
      std::memcpy(&m, open_block() + sizeof(GroupHead), sizeof(m));
      const uint32_t tensor = p->member_tensor[p->member_tensor.size() - kGroupMaxMembers];
      p->group_blocks.resize(p->group_blocks.size() - kGroupBlockBytes);
      p->member_tensor.resize(p->member_tensor.size() - kGroupMaxMembers);
      int rc = add_seg(tensor, m.ptr, group_off, m.nbytes, 1, 0);
      if (!rc) p->segs.back().meta |= m.off_pad >> kMemberOffBits;
      return rc;
    }
    GroupHead head;
    head.starts[0] = group_starts[0];
    head.starts[1] = group_starts[1];
    head.off = group_off;
    head.members = group_count;
    head.slots = group_slots;
    std::memcpy(open_block(), &head, sizeof(head));
    const size_t index = p->group_blocks.size() / kGroupBlockBytes - 1;
    // `ptr` holds the index of the group's block until the table sections are laid out
    return add_seg(p->member_tensor[index * kGroupMaxMembers], index, group_off,
                   static_cast<uint64_t>(group_count) | static_cast<uint64_t>(group_slots) << 8, 1, kSegGroup);
  }

  int add_seg(uint32_t tensor, uint64_t ptr, uint64_t off, uint64_t run_bytes, uint64_t ntile,
              uint32_t dsel) {
    if (tiles + ntile > 0xffffffffull) return fail(AXR_ERR_UNSUPPORTED, "bundle has too many tiles");
    Seg s;
    s.ptr = ptr;
    s.off = off;
    s.run_bytes = run_bytes;
    s.tile_begin = static_cast<uint32_t>(tiles);
    s.meta = dsel << kSegDimsShift;
    p->segs.push_back(s);
    p->seg_tensor.push_back(tensor);
    tiles += ntile;
    return AXR_OK;
  }

  // Emit device segments for a strided block: `outer` strided dims (any count)
  // around one contiguous run.  More than kMaxOuterDims dims are peeled off on
  // the host, outermost first.
  int add_strided(uint32_t tensor, uint64_t ptr, uint64_t off, const uint64_t* ext,
                  const int64_t* str, size_t nd, uint64_t run_bytes) {
    if (nd == 0) {
      // Segments longer than a tile peel off their first bytes up to the next line of the
      // side that is written (the payload for a sender's plan, the tensor for a receiver's),
      // so that no two tiles write into one 128-byte line.
      uint64_t head = 0;
      if (head_align > 1 && run_bytes > tile_bytes && run_bytes <= kSegRunMask)
        head = (0 - (p->receiver ? ptr : off)) & (head_align - 1);
      int rc = add_seg(tensor, ptr, off, run_bytes | (head << kSegHeadShift),
                       (run_bytes - head + tile_bytes - 1) >> tile_shift, 0);
      return rc;
    }
    uint64_t inner_runs = 1;
    for (size_t d = 1; d < nd; ++d) inner_runs *= ext[d];
    if (nd > kMaxOuterDims) {
      for (uint64_t i = 0; i < ext[0]; ++i) {
        int rc = add_strided(tensor, ptr + static_cast<uint64_t>(static_cast<int64_t>(i) * str[0]),
                             off + i * inner_runs * run_bytes, ext + 1, str + 1, nd - 1, run_bytes);
        if (rc) return rc;
      }
      return AXR_OK;
    }
    const uint64_t runs = inner_runs * ext[0];
    const uint64_t nbytes = runs * run_bytes;
    Dims dm;
    std::memset(&dm, 0, sizeof(dm));
    dm.ndim = static_cast<uint32_t>(nd);
    dm.nbytes = nbytes;
    for (uint32_t d = 0; d < kMaxOuterDims; ++d) {
      dm.shape[d] = 1;
      dm.stride[d] = 0;
    }
    for (size_t d = 0; d < nd; ++d) {
      if (ext[d] > 0xffffffffull) return fail(AXR_ERR_UNSUPPORTED, "strided extent exceeds 32 bits");
      dm.shape[kMaxOuterDims - nd + d] = static_cast<uint32_t>(ext[d]);
      dm.stride[kMaxOuterDims - nd + d] = str[d];
    }
    uint64_t ntile;
    // A transposition: no contiguous inner run beyond one element, but some outer
    // dimension (B) is contiguous in the tensor.  Blocks of A x B go through LDS.
    size_t dim_b = nd;
    uint32_t edge_a = 0, edge_b = 0;
    if (nd >= 2 && run_bytes <= kVecBytes && (run_bytes & (run_bytes - 1)) == 0 &&
        tunables().transpose != 0) {
      for (size_t d = 0; d + 1 < nd; ++d) {
        if (str[d] == static_cast<int64_t>(run_bytes)) {
          dim_b = d;
          break;
        }
      }
    }
    if (dim_b < nd) {
      // Square blocks when both dimensions reach a block edge; otherwise the short
      // dimension is taken whole (up to an edge) and the other one stretches until
      // the block holds about 8 KiB.  Blocks under 1 KiB are not worth a wave:
      // such views stay in element mode.
      const uint32_t e = static_cast<uint32_t>(run_bytes);
      const uint64_t t = transpose_edge(e), ea = ext[nd - 1], eb = ext[dim_b];
      const uint64_t elems = kRectBlockBytes / e;
      if (ea >= t && eb >= t) {
        edge_a = edge_b = static_cast<uint32_t>(t);
      } else {
        // the long edge is a whole number of 16-byte vectors where it can be
        const uint64_t ev = kVecBytes / e;
        auto long_edge = [&](uint64_t extent, uint32_t short_edge) {
          uint64_t edge = std::min<uint64_t>({extent, kRectMaxEdge, elems / short_edge});
          if (edge >= ev) edge -= edge % ev;
          return static_cast<uint32_t>(edge);
        };
        if (ea <= eb) {
          edge_a = static_cast<uint32_t>(std::min(ea, t));
          edge_b = long_edge(eb, edge_a);
        } else {
          edge_b = static_cast<uint32_t>(std::min(eb, t));
          edge_a = long_edge(ea, edge_b);
        }
      }
      if (static_cast<uint64_t>(edge_a) * edge_b * e < 1024) dim_b = nd;
    }
    if (dim_b < nd) {
      const uint32_t e = static_cast<uint32_t>(run_bytes);
      const size_t dim_a = nd - 1;
      dm.mode = kModeTranspose;
      dm.granule = e;
      dm.ndim = static_cast<uint32_t>(nd - 2);
      for (uint32_t d = 0; d < kMaxOuterDims; ++d) {
        dm.shape[d] = 1;
        dm.stride[d] = 0;
      }
      // packed byte stride of dim d = element size * product of the inner extents
      uint64_t packed[kMaxOuterDims];
      uint64_t acc = e;
      for (size_t d = nd; d-- > 0;) {
        packed[d] = acc;
        acc *= ext[d];
      }
      uint64_t batches = 1;
      size_t slot = kMaxBatchDims;
      for (size_t d = nd; d-- > 0;) {
        if (d == dim_a || d == dim_b) continue;
        --slot;
        dm.shape[kMaxOuterDims - kMaxBatchDims + slot] = static_cast<uint32_t>(ext[d]);
        dm.stride[kMaxOuterDims - kMaxBatchDims + slot] = str[d];
        dm.pstride[slot] = packed[d];
        batches *= ext[d];
      }
      dm.stride_a = str[dim_a];
      dm.pstride_b = packed[dim_b];
      dm.ext_a = static_cast<uint32_t>(ext[dim_a]);
      dm.ext_b = static_cast<uint32_t>(ext[dim_b]);
      dm.edge_a = edge_a;
      dm.edge_b = edge_b;
      dm.tiles_a = (dm.ext_a + edge_a - 1) / edge_a;
      dm.tiles_b = (dm.ext_b + edge_b - 1) / edge_b;
      const uint64_t per_batch = static_cast<uint64_t>(dm.tiles_a) * dm.tiles_b;
      if (per_batch > 0xffffffffull || batches > 0xffffffffull / per_batch)
        return fail(AXR_ERR_UNSUPPORTED, "transposed tensor has too many blocks");
      ntile = batches * per_batch;
      // rows of one side plus a dword each, whichever direction needs more
      // (or one pad dword per 128 bytes, for blocks staged as one contiguous range)
      const uint32_t block_bytes = edge_a * edge_b * e;
      const uint32_t lds = block_bytes + std::max(4u * std::max(edge_a, edge_b), block_bytes / 32u + 16u);
      p->cfg.lds_per_wave = std::max<uint32_t>(p->cfg.lds_per_wave, (lds + 15u) & ~15u);
      // A side whose block rows start on 128-byte lines is read or written in whole lines and
      // may stream; a side with another pitch or base shares the first and last line of every
      // block row with the neighbouring blocks, and only a cacheable access lets the second
      // block find or complete the line in the die's L2 instead of going to memory again: the
      // bytes fetched and written for four 4097 x 4099 bf16 matrices fall from 1.38 to 1.1
      // times the payload and the pack + unpack rate rises from 3.65 to 3.87 TB/s (with the
      // die-contiguous tile ranges that finish_geometry then selects).
      const uint64_t line = kLineBytes - 1;
      bool tensor_lines = ((ptr | static_cast<uint64_t>(str[dim_a])) & line) == 0;
      bool payload_lines = ((off | packed[dim_b]) & line) == 0;
      for (size_t d = 0; d < nd; ++d) {
        if (d == dim_a || d == dim_b) continue;
        tensor_lines = tensor_lines && (static_cast<uint64_t>(str[d]) & line) == 0;
        payload_lines = payload_lines && (packed[d] & line) == 0;
      }
      dm.nt_allowed = ((tensor_lines ? 1u : 0u) | (payload_lines ? 2u : 0u)) * 5u;   // both directions
      if (!tensor_lines || !payload_lines) shared_line_tiles += ntile;
    } else if (run_bytes >= element_mode_limit(run_bytes)) {
      dm.mode = kModeRunTiles;
      const uint64_t tpr = (run_bytes + tile_bytes - 1) / tile_bytes;
      if (tpr > 0xffffffffull || runs > 0xffffffffull)
        return fail(AXR_ERR_UNSUPPORTED, "strided tensor has too many runs");
      dm.tiles_per_run = static_cast<uint32_t>(tpr);
      // granule is unused in this mode: it carries 1 + log2(tiles per run) when
      // that is a power of two, so the kernel can shift instead of divide
      dm.granule = (tpr & (tpr - 1)) == 0 ? 1u + static_cast<uint32_t>(__builtin_ctzll(tpr)) : 0u;
      ntile = runs * tpr;
    } else {
      dm.mode = kModeElements;
      // the kernel's per-granule index arithmetic is 32-bit
      if (runs > 0x7fffffffull) return fail(AXR_ERR_UNSUPPORTED, "strided tensor has too many runs");
      dm.granule = granule_of(run_bytes);
      // Rows shorter than a line use every line they touch only in part: such lines are
      // cheaper read and written through the cache than streamed (100-byte rows: +5 to 7 %).
      dm.nt_allowed = (run_bytes >= kLineBytes ? 3u : 2u) * 5u;   // the same in both directions
      const uint64_t element_tile = std::max<uint32_t>(tile_bytes, kMinElementTileBytes);
      const uint64_t granules_per_run = (run_bytes + kVecBytes - 1) / kVecBytes;
      if (run_bytes >= kVecBytes && tunables().ragged_runs != 0 &&
          (dm.granule != kVecBytes || (granules_per_run & 3) != 0)) {
        // ragged runs: ceil(run / 16) granules of 16 bytes per run, the last one covering
        // the run's final 16 bytes, in a whole number of four-lane groups; tiles count
        // lane slots
        dm.granule = kVecBytes;
        dm.lanes_per_run = static_cast<uint32_t>((granules_per_run + 3) & ~3ull);
        const uint64_t slots = runs * dm.lanes_per_run;
        dm.pstride[0] = slots;
        const uint64_t per_tile = element_tile / kVecBytes;
        ntile = (slots + per_tile - 1) / per_tile;
      } else {
        ntile = (nbytes + element_tile - 1) / element_tile;
      }
    }
    if (p->dims.size() + 1 >= kSegFillOnly)
      return fail(AXR_ERR_UNSUPPORTED, "too many strided tensors in one bundle");
    p->dims.push_back(dm);
    return add_seg(tensor, ptr, off, run_bytes, ntile, static_cast<uint32_t>(p->dims.size()));
  }

  // Host (kDLCPU) tensors move with one async copy per contiguous run.
  int add_host(uint32_t tensor, uint64_t ptr, uint64_t off, const uint64_t* ext,
               const int64_t* str, size_t nd, uint64_t run_bytes) {
    if (nd == 0) {
      // pieces of at most one staging block
      for (uint64_t done = 0; done < run_bytes; done += kStageBytes) {
        if (p->host_copies.size() >= (1u << 20))
          return fail(AXR_ERR_UNSUPPORTED, "host tensor needs more than 2^20 copies");
        p->host_copies.push_back({ptr + done, off + done, std::min<uint64_t>(kStageBytes, run_bytes - done)});
        p->host_copy_tensor.push_back(tensor);
      }
      return AXR_OK;
    }
    uint64_t inner = run_bytes;
    for (size_t d = 1; d < nd; ++d) inner *= ext[d];
    for (uint64_t i = 0; i < ext[0]; ++i) {
      int rc = add_host(tensor, ptr + static_cast<uint64_t>(static_cast<int64_t>(i) * str[0]),
                        off + i * inner, ext + 1, str + 1, nd - 1, run_bytes);
      if (rc) return rc;
    }
    return AXR_OK;
  }
};

int build_tables(axr_plan* p);

// A payload that streams to and from memory (larger than payload_cache_bytes, so written and
// read with non-temporal accesses) moves fastest in tiles of 1 KiB, one load and one store per
// lane, in workgroups of a single wavefront: the 1 GiB cache-block gather 6.02 -> 6.29 TB/s
// (pack 6.26 -> 6.51, unpack 5.80 -> 6.09), 1 GiB of pitched rows of 4-64 KiB 6.24-6.40 ->
// 6.59-6.61, the 405 MB layer bundle 6.43 -> 6.52.  Either change alone is slower than the
// 2 KiB tiles in workgroups of two wavefronts it replaces, and payloads that stay in the
// last-level cache lose 7-24 % with it (48 MB mixed bundle, 256 MiB chunk of pitched rows).
// Up to max_tiles tiles, i.e. 1 GiB.
bool streams_in_small_tiles(const axr_plan* p) {
  const Tunables& tn = tunables();
  return p->payload_bytes > static_cast<uint64_t>(tn.payload_cache_bytes) &&
         (p->payload_bytes >> 10) <= static_cast<uint64_t>(tn.max_tiles);
}

// Launch geometry of a bundle of p->ntiles tiles in nseg segments: one tile per wave until
// the grid would exceed max_waves, workgroup size, cache hints, and the size of the blocks of
// the tile-block index (about one segment each, a power of two up to 256 tiles: a bundle of
// few large tensors gets a tiny index, a bundle of many small ones an entry per few tiles).
void finish_geometry(axr_plan* p, uint32_t rows, size_t nseg, bool may_be_direct = false) {
  const Tunables& tn = tunables();
  uint64_t tpw = (p->ntiles + static_cast<uint64_t>(tn.max_waves) - 1) /
                 static_cast<uint64_t>(tn.max_waves);
  if (tpw == 0) tpw = 1;
  p->cfg.threads = tn.threads ? static_cast<uint32_t>(tn.threads)
                              : (rows == 1 && tn.tile_rows == 0 ? kWaveLanes : (p->ntiles < 65536 ? 256u : 128u));
  p->cfg.elements = false;
  bool ragged_rows = false, blocks = false;
  for (const Dims& dm : p->dims) {
    p->cfg.elements = p->cfg.elements || dm.mode != kModeRunTiles;
    ragged_rows = ragged_rows || (dm.mode == kModeElements && dm.lanes_per_run != 0);
    blocks = blocks || dm.mode == kModeTranspose;
  }
  if (p->cfg.elements) p->cfg.threads = std::min(p->cfg.threads, kMaxElementThreads);
  // Short rows that are no multiple of 16 bytes (lane slots left idle behind each run) run 2.5-5 %
  // faster in workgroups of one wavefront (rows of 250 B: 4.97 -> 5.22 TB/s, of 100 B: 3.06 ->
  // 3.14); rows of whole granules and transposed blocks are fastest at 256 threads.
  if (tn.threads == 0 && ragged_rows && !blocks) p->cfg.threads = kWaveLanes;
  if (p->cfg.lds_per_wave) {
    // transposed blocks: every wave of a workgroup owns a slice of at most 64 KiB of LDS
    const uint32_t fit = (64u * 1024u / p->cfg.lds_per_wave) * kWaveLanes;
    p->cfg.threads = std::min(p->cfg.threads, fit);
  }
  const uint32_t waves_per_wg = p->cfg.threads / kWaveLanes;
  const uint64_t per_wg = tpw * waves_per_wg;
  p->cfg.tiles_per_wave = static_cast<uint32_t>(tpw);
  p->cfg.workgroups = static_cast<uint32_t>((p->ntiles + per_wg - 1) / per_wg);
  // Each die a contiguous share of the tiles: slower for streams of whole lines, but it lets
  // transposed blocks whose rows straddle lines meet their neighbours in one L2 (automatic
  // when such blocks are half of the bundle or more).
  const bool remap = tn.xcd_remap > 0 ||
                     (tn.xcd_remap < 0 && p->shared_line_tiles != 0 && 2 * p->shared_line_tiles >= p->ntiles);
  p->cfg.xcd_remap = remap && p->cfg.workgroups >= 4 * kXcds;
  if (p->cfg.xcd_remap) p->cfg.workgroups = (p->cfg.workgroups + kXcds - 1) / kXcds * kXcds;
  p->cfg.tile_rows = rows;
  if (tn.nontemporal < 0) {
    p->cfg.nontemporal = p->payload_bytes > static_cast<uint64_t>(tn.payload_cache_bytes) ? 3u : 1u;
  } else {
    p->cfg.nontemporal = static_cast<uint32_t>(tn.nontemporal) & 3u;
  }
  uint32_t shift = 0;
  while (shift < 8 && (static_cast<uint64_t>(nseg) << (shift + 1)) <= p->ntiles) ++shift;
  // as many tiles as segments (none without a tile): tile t is segment t, no index to consult
  p->cfg.seg_shift = may_be_direct && nseg == p->ntiles ? kDirectSegShift : shift;
}

// Tile rows of a bundle whose tensors are all compact: 2 KiB tiles, doubled while the bundle
// would exceed max_tiles.
uint32_t rows_for_compact_bundle(const axr_plan* p) {
  const Tunables& tn = tunables();
  uint32_t rows = static_cast<uint32_t>(tn.tile_rows);
  if (rows) return rows;
  if (streams_in_small_tiles(p)) return 1;
  rows = 2;
  while (rows < kMaxTileRows &&
         p->payload_bytes / (static_cast<uint64_t>(rows) * kRowBytes) > static_cast<uint64_t>(tn.max_tiles))
    rows *= 2;
  return rows;
}

bool compact_strides(const int64_t* shape, const int64_t* strides, int32_t ndim) {
  int64_t expect = 1;
  for (int32_t d = ndim - 1; d >= 0; --d) {
    if (shape[d] == 1) continue;
    if (strides[d] != expect) return false;
    expect *= shape[d];
  }
  return true;
}

// Bundles of many contiguous device tensors: one pass over the tensors writes the segment
// records straight into pinned memory, and a kernel (one thread per segment) brings them to
// the device and writes the tile-block index, in front of the bundle kernel on the same
// stream: no strides to collapse, no index built on the host, no copy engine to wait for.
// Returns AXR_OK with *done set when the tables are on their way, AXR_OK with *done clear when
// the bundle does not qualify (the caller takes the general path), or an error.
int device_build_tables(axr_plan* p, hipStream_t stream, bool* done) {
  *done = false;
  const Tunables& tn = tunables();
  const size_t n = p->tensors.size();
  const int64_t least = tn.device_tables;
  if (least <= 0 || n < static_cast<uint64_t>(least) || n > (1u << 20) || !p->bound) return AXR_OK;
  if (tn.group_bytes > 0) {
    // a bundle in which a quarter of the tensors are short enough to share wavefronts takes the
    // general path, which builds group tiles
    const uint64_t limit = static_cast<uint64_t>(tn.group_bytes);
    size_t small = 0;
    for (size_t i = 0; i < n; ++i) small += (p->tensors[i].nbytes - 1) < limit ? 1 : 0;   // 1 .. limit
    if (small * 4 >= n) return AXR_OK;
  }
  const uint32_t rows = rows_for_compact_bundle(p);
  const uint32_t tile_bytes = rows * kRowBytes;
  const uint32_t tile_shift = static_cast<uint32_t>(__builtin_ctz(tile_bytes));
  const uint64_t head_align = static_cast<uint64_t>(tn.head_align);
  const uint64_t head_mask = head_align > 1 ? head_align - 1 : 0;
  // room for the index: with blocks of 2^shift tiles, shift < 8 means fewer than 2 n blocks
  const uint64_t tiles_bound = (p->payload_bytes >> tile_shift) + n;
  if (tiles_bound > 0xffffffffull) return AXR_OK;
  const size_t blocks_bound = std::max<size_t>(2 * n + 2, static_cast<size_t>(tiles_bound >> 8) + 2);
  const size_t wave_at = align_up((n + 1) * sizeof(Seg), 16);
  const size_t bytes = wave_at + blocks_bound * sizeof(uint32_t);
  if (p->block.host && p->block.bytes < bytes) {
    quiesce(p);
    table_block_release(&p->block);
  }
  if (!p->block.host) {
    int rc = table_block_acquire(bytes, &p->block);
    if (rc) return rc;
  } else {
    quiesce(p);   // earlier launches may still read the block
  }
  Seg* staged = static_cast<Seg*>(p->block.host);
  uint64_t tiles = 0;
  bool pinned = false;
  const bool receiver = p->receiver;
  const uint64_t align_mask = static_cast<uint64_t>(p->align) - 1;
  for (size_t i = 0; i < n; ++i) {
    const TensorRec& t = p->tensors[i];
    if ((t.device_type != kDLROCM && t.device_type != kDLROCMHost) || t.nbytes > kSegRunMask) return AXR_OK;
    pinned = pinned || t.device_type == kDLROCMHost;
    if (t.has_strides && t.nbytes && !compact_strides(p->shape_of(t), p->strides_of(t), t.ndim)) return AXR_OK;
    Seg& sg = staged[i];
    sg.ptr = t.address;
    sg.off = t.offset;
    sg.tile_begin = static_cast<uint32_t>(tiles);
    if (t.nbytes) {
      const uint64_t head =
          (head_mask && t.nbytes > tile_bytes) ? (0 - (receiver ? t.address : t.offset)) & head_mask : 0;
      const uint64_t stop = t.offset + t.nbytes;
      sg.run_bytes = t.nbytes | (head << kSegHeadShift);
      sg.meta = static_cast<uint32_t>(std::min((stop + align_mask) & ~align_mask, p->payload_bytes) - stop);
      tiles += (t.nbytes - head + tile_bytes - 1) >> tile_shift;
    } else {
      sg.run_bytes = 0;
      sg.meta = 0;
    }
  }
  if (tiles == 0 || tiles > 0xffffffffull) return AXR_OK;
  std::memset(&staged[n], 0, sizeof(Seg));
  staged[n].tile_begin = static_cast<uint32_t>(tiles);
  p->segs.clear();
  p->dims.clear();
  p->wave_seg.clear();
  p->ntiles = static_cast<uint32_t>(tiles);
  p->cfg.lds_per_wave = 0;
  p->pinned_host_tensors = pinned;
  finish_geometry(p, rows, n);
  p->dims_at = wave_at;
  p->wave_at = wave_at;
  p->table_bytes = wave_at + ((static_cast<size_t>(p->ntiles) >> p->cfg.seg_shift) + 1) * sizeof(uint32_t);
  uint8_t* d = static_cast<uint8_t*>(p->block.device);
  int rc = launch_expand_tables(staged, static_cast<uint32_t>(n), reinterpret_cast<Seg*>(d),
                                reinterpret_cast<uint32_t*>(d + wave_at), p->cfg.seg_shift, stream);
  if (rc) return rc;
  if (!p->upload_event) {
    rc = event_acquire(reinterpret_cast<void**>(&p->upload_event), &p->upload_event_device);
    if (rc) return rc;
  }
  rc = check_hip(hipEventRecord(p->upload_event, stream), "hipEventRecord");
  if (rc) return rc;
  remember_stream(p, stream);
  p->upload_stream = stream;
  p->uploaded = true;
  p->device_built = true;
  *done = true;
  return AXR_OK;
}

// Tables for a launch on `stream`: what is there already, else built by the device when the
// bundle qualifies and the stream is not capturing, else built on the host.
int ensure_tables(axr_plan* p, hipStream_t stream, bool capturing) {
  if (p->tables_built || p->device_built) return AXR_OK;
  if (!capturing) {
    bool done = false;
    int rc = device_build_tables(p, stream, &done);
    if (rc || done) return rc;
  }
  return build_tables(p);
}

int build_tables(axr_plan* p) {
  if (p->tables_built) return AXR_OK;
  if (!p->bound) return fail(AXR_ERR_INVALID, "plan has no tensor addresses bound");
  if (p->device_built) quiesce(p);   // the host tables replace the device-built ones at the next launch
  invalidate_tables(p);
  const Tunables& tn = tunables();
  uint32_t rows = static_cast<uint32_t>(tn.tile_rows);
  if (rows == 0) {
    rows = 2;
    // A bundle made only of strided views with one short run length (pitched
    // rows, small cache blocks) gets one tile per run: fewer waves, no split runs.
    // Only while the payload is small enough to be left in the last-level cache
    // (payload_cache_bytes): a pack followed by the unpack of the same payload then runs
    // 5-9 % faster with whole-run tiles (rows of 4-16 KiB, 256 MiB: 6.46-6.64 against
    // 6.10-6.30 TB/s), whereas a payload that streams to and from memory is moved 8-10 %
    // faster in 2 KiB tiles (1 GiB of 8 KiB or 16 KiB cache blocks: 5.68 and 5.59 against
    // 5.25 and 5.10 TB/s).
    uint64_t common_run = 0;
    bool uniform_runs = !p->tensors.empty();
    for (const TensorRec& t : p->tensors) {
      if (t.nbytes == 0) continue;
      if (!t.has_strides) {   // a compact tensor: not a bundle of strided views
        uniform_runs = false;
        break;
      }
      const uint64_t item = (static_cast<uint64_t>(t.bits) + 7) / 8;
      Collapsed c;
      collapse(t, p->shape_of(t), p->strides_of(t), item, &c);
      if (c.nd == 0 || (common_run && c.run_bytes != common_run)) {
        uniform_runs = false;
        break;
      }
      common_run = c.run_bytes;
    }
    if (uniform_runs && common_run >= 2 * kRowBytes && common_run <= kMaxTileRows * kRowBytes &&
        p->payload_bytes <= static_cast<uint64_t>(tn.payload_cache_bytes)) {
      while (rows < kMaxTileRows && rows * kRowBytes < common_run) rows *= 2;
    }
    if (streams_in_small_tiles(p)) {
      // only for bundles of compact tensors and strided views that move as run tiles
      bool run_tiles_only = true;
      for (const TensorRec& t : p->tensors) {
        if (t.nbytes == 0 || !t.has_strides) continue;
        const uint64_t item = (static_cast<uint64_t>(t.bits) + 7) / 8;
        Collapsed c;
        collapse(t, p->shape_of(t), p->strides_of(t), item, &c);
        if (c.nd != 0 && c.run_bytes < static_cast<uint64_t>(tn.gather_run_bytes)) {
          run_tiles_only = false;
          break;
        }
      }
      if (run_tiles_only) rows = 1;
    }
    while (rows < kMaxTileRows &&
           p->payload_bytes / (static_cast<uint64_t>(rows) * kRowBytes) >
               static_cast<uint64_t>(tn.max_tiles))
      rows *= 2;
  }
  Builder b{p, rows * kRowBytes, static_cast<uint32_t>(__builtin_ctz(rows * kRowBytes)),
            static_cast<uint64_t>(tn.head_align)};
  b.group_bytes = static_cast<uint64_t>(tn.group_bytes);
  b.slots_per_group = static_cast<uint32_t>(tn.group_slots);
  p->segs.reserve(p->tensors.size() + 1);
  p->seg_tensor.reserve(p->tensors.size());

  for (size_t i = 0; i < p->tensors.size(); ++i) {
    const TensorRec& t = p->tensors[i];
    if (t.nbytes == 0) continue;
    const uint64_t item = (static_cast<uint64_t>(t.bits) + 7) / 8;
    const uint64_t end = t.offset + t.nbytes;
    const uint64_t pad = std::min<uint64_t>(align_up(end, p->align), p->payload_bytes) - end;
    const int64_t* shape = p->shape_of(t);
    const int64_t* strides = p->strides_of(t);
    if (strides) {
      for (int32_t d = 0; d < t.ndim; ++d)
        if (strides[d] == 0 && shape[d] > 1) p->overlapping_dst = true;
    }
    Collapsed c;
    if (!strides) {   // compact by definition: one run, nothing to collapse
      c.nd = 0;
      c.run_bytes = t.nbytes;
    } else {
      collapse(t, shape, strides, item, &c);
    }
    int rc;
    if (t.device_type == kDLROCMHost) p->pinned_host_tensors = true;
    if (t.device_type == kDLROCM || t.device_type == kDLROCMHost) {
      if (c.nd == 0 && b.add_member(static_cast<uint32_t>(i), t.address, t.offset, t.nbytes, pad, &rc)) {
        if (rc) return rc;
        continue;
      }
      rc = b.close_group();
      if (rc) return rc;
      rc = b.add_strided(static_cast<uint32_t>(i), t.address, t.offset, c.extent, c.stride, c.nd,
                         c.run_bytes);
      if (rc) return rc;
      if (pad) p->segs.back().meta |= static_cast<uint32_t>(pad);
    } else if (t.device_type == kDLCPU) {
      rc = b.close_group();
      if (rc) return rc;
      rc = b.add_host(static_cast<uint32_t>(i), t.address, t.offset, c.extent, c.stride, c.nd,
                      c.run_bytes);
      if (rc) return rc;
      if (pad) {
        rc = b.add_seg(static_cast<uint32_t>(i), 0, end, 0, 1, kSegFillOnly);
        if (rc) return rc;
        p->segs.back().meta |= static_cast<uint32_t>(pad);
      }
    } else {
      return fail(AXR_ERR_UNSUPPORTED,
                  "Unsupported memory type: DLPack device " + std::to_string(t.device_type));
    }
  }
  {
    int rc = b.close_group();
    if (rc) return rc;
  }
  // Group neighbouring host pieces (in payload order, at most an alignment gap
  // apart) into chunks that fit one staging block.
  for (uint32_t i = 0; i < p->host_copies.size(); ++i) {
    const HostCopy& hc = p->host_copies[i];
    if (!p->host_chunks.empty()) {
      HostChunk& c = p->host_chunks.back();
      if (hc.offset >= c.end && hc.offset - c.end < kMaxAlign &&
          hc.offset + hc.bytes - c.begin <= kStageBytes) {
        c.end = hc.offset + hc.bytes;
        ++c.count;
        continue;
      }
    }
    p->host_chunks.push_back({i, 1, hc.offset, hc.offset + hc.bytes});
  }
  p->stage_bytes = 0;
  for (const HostChunk& c : p->host_chunks)
    p->stage_bytes = std::max<size_t>(p->stage_bytes, static_cast<size_t>(c.end - c.begin));
  p->ntiles = static_cast<uint32_t>(b.tiles);
  p->shared_line_tiles = b.shared_line_tiles;
  Seg sentinel;
  std::memset(&sentinel, 0, sizeof(sentinel));
  sentinel.tile_begin = p->ntiles;
  p->segs.push_back(sentinel);

  const size_t nseg = p->segs.size() - 1;
  bool one_tile_each = true;
  for (size_t i = 0; i < nseg && one_tile_each; ++i)
    one_tile_each = p->segs[i + 1].tile_begin - p->segs[i].tile_begin == 1;
  finish_geometry(p, rows, nseg, one_tile_each);
  // group tiles only: the kernel finds tile t's block at a fixed stride, without the segment
  // records and the index
  p->groups_only = nseg != 0 && p->group_blocks.size() == nseg * kGroupBlockBytes;
  if (p->groups_only) p->cfg.seg_shift = kGroupBlocksShift;

  // Tile-block index: entry k = segment that holds tile k << seg_shift.  Blocks
  // are sized to about one segment each (a power of two, at most 256 tiles), so
  // a bundle of few large tensors gets a tiny index and a bundle of many small
  // ones one entry per few tiles; a wave walks at most a segment or two forward.
  const uint32_t shift = p->cfg.seg_shift;
  const bool no_index = shift == kDirectSegShift || shift == kGroupBlocksShift;
  const size_t nblocks = no_index ? 1 : (static_cast<size_t>(p->ntiles) >> shift) + 1;
  p->wave_seg.assign(nblocks, 0);
  size_t s = 0;
  for (size_t k = 0; k < nblocks && !no_index; ++k) {
    const uint64_t t0 = static_cast<uint64_t>(k) << shift;
    if (t0 >= p->ntiles) break;
    while (s + 1 < nseg && p->segs[s + 1].tile_begin <= t0) ++s;
    p->wave_seg[k] = static_cast<uint32_t>(s);
  }

  p->dims_at = align_up(p->segs.size() * sizeof(Seg), 16);
  p->wave_at = align_up(p->dims_at + p->dims.size() * sizeof(Dims), 16);
  p->members_at = align_up(p->wave_at + p->wave_seg.size() * sizeof(uint32_t), 16);
  p->table_bytes = p->members_at + p->group_blocks.size();
  if (!p->group_blocks.empty()) {
    // a group's segment names its block by the block's offset in the table block
    if (p->table_bytes > 0xffffffffull) return fail(AXR_ERR_UNSUPPORTED, "bundle tables exceed 4 GiB");
    for (size_t i = 0; i < nseg; ++i) {
      Seg& sg = p->segs[i];
      if ((sg.meta >> kSegDimsShift) == kSegGroup) sg.ptr = p->members_at + sg.ptr * kGroupBlockBytes;
    }
  }
  p->tables_built = true;
  return AXR_OK;
}

// Where the kernel's `dims` argument points inside the table block: at the Dims records, or,
// for a bundle of group tiles only, at the group blocks.
size_t dims_arg_at(const axr_plan* p) { return p->groups_only ? p->members_at : p->dims_at; }

// The host-built tables laid out as one block (segments, dims, tile-block index, group blocks).
void write_tables(const axr_plan* p, uint8_t* h) {
  std::memcpy(h, p->segs.data(), p->segs.size() * sizeof(Seg));
  if (!p->dims.empty()) std::memcpy(h + p->dims_at, p->dims.data(), p->dims.size() * sizeof(Dims));
  std::memcpy(h + p->wave_at, p->wave_seg.data(), p->wave_seg.size() * sizeof(uint32_t));
  if (!p->group_blocks.empty()) std::memcpy(h + p->members_at, p->group_blocks.data(), p->group_blocks.size());
}

int ensure_uploaded(axr_plan* p, hipStream_t stream) {
  if (p->ntiles == 0) return AXR_OK;
  if (!p->uploaded) {
    if (p->block.host && (p->block.bytes < p->table_bytes)) {
      quiesce(p);
      table_block_release(&p->block);
    }
    if (!p->block.host) {
      int rc = table_block_acquire(p->table_bytes, &p->block);
      if (rc) return rc;
    } else {
      quiesce(p);   // previous launches may still read the old tables
    }
    uint8_t* h = static_cast<uint8_t*>(p->block.host);
    write_tables(p, h);
    int rc = check_hip(hipMemcpyAsync(p->block.device, h, p->table_bytes, hipMemcpyHostToDevice,
                                      stream),
                       "hipMemcpyAsync(plan tables)");
    if (rc) return rc;
    if (!p->upload_event) {
      rc = event_acquire(reinterpret_cast<void**>(&p->upload_event), &p->upload_event_device);
      if (rc) return rc;
    }
    rc = check_hip(hipEventRecord(p->upload_event, stream), "hipEventRecord");
    if (rc) return rc;
    p->upload_stream = stream;
    p->uploaded = true;
  } else if (stream != p->upload_stream) {
    int rc = check_hip(hipStreamWaitEvent(stream, p->upload_event, 0), "hipStreamWaitEvent");
    if (rc) return rc;
  }
  return AXR_OK;
}

int stage_ready(HostStage* st) {   // block until the staging block's last device copy is done
  if (!st->pending) return AXR_OK;
  st->pending = false;
  return check_hip(hipEventSynchronize(st->ready), "hipEventSynchronize(staging)");
}

int stage_acquire(HostStage* st, size_t bytes) {
  if (st->block.host && st->block.bytes < bytes) {   // a rebound plan with longer chunks
    int rc = stage_ready(st);
    if (rc) return rc;
    table_block_release(&st->block);
  }
  if (!st->block.host) {
    int rc = table_block_acquire(bytes, &st->block);
    if (rc) return rc;
  }
  if (!st->ready) {
    int rc = check_hip(hipEventCreateWithFlags(&st->ready, hipEventDisableTiming), "hipEventCreate");
    if (rc) return rc;
  }
  return stage_ready(st);
}

// kDLCPU tensors.  Pack: the pieces of a chunk are copied into a pinned block on
// the calling thread (gaps zeroed: they are alignment padding or are rewritten by
// the kernel that follows on the stream), then one asynchronous device copy moves
// the chunk.  Unpack: one device copy per chunk into a pinned block; while the
// next chunk is in flight the calling thread copies the previous one out, so the
// call returns when the host tensors hold their data (as a copy into pageable
// memory does).  Two blocks alternate.
int move_host_tensors(axr_plan* p, bool pack, uint8_t* payload, hipStream_t stream) {
  const size_t nchunks = p->host_chunks.size();
  std::vector<HostCopyJob> jobs;
  auto pieces_out = [p, &jobs](const HostChunk& c, const uint8_t* staged) {
    jobs.clear();
    for (uint32_t i = c.first; i < c.first + c.count; ++i) {
      const HostCopy& hc = p->host_copies[i];
      jobs.push_back({reinterpret_cast<void*>(hc.host), staged + (hc.offset - c.begin), hc.bytes});
    }
    host_copy(jobs.data(), jobs.size());
  };
  for (size_t k = 0; k < nchunks; ++k) {
    const HostChunk& c = p->host_chunks[k];
    HostStage* st = &p->stage[k & 1];
    if (!pack && k >= 2) {   // the block still holds chunk k - 2
      int rc = stage_ready(st);
      if (rc) return rc;
      pieces_out(p->host_chunks[k - 2], static_cast<const uint8_t*>(st->block.host));
    }
    const size_t span = static_cast<size_t>(c.end - c.begin);
    // a block as long as the plan's longest chunk (8 MiB at most), not 8 MiB for all
    int rc = stage_acquire(st, p->stage_bytes);
    if (rc) return rc;
    uint8_t* staged = static_cast<uint8_t*>(st->block.host);
    if (pack) {
      uint64_t at = c.begin;
      jobs.clear();
      for (uint32_t i = c.first; i < c.first + c.count; ++i) {
        const HostCopy& hc = p->host_copies[i];
        if (hc.offset > at) std::memset(staged + (at - c.begin), 0, hc.offset - at);
        jobs.push_back({staged + (hc.offset - c.begin), reinterpret_cast<const void*>(hc.host), hc.bytes});
        at = hc.offset + hc.bytes;
      }
      host_copy(jobs.data(), jobs.size());
      rc = check_hip(hipMemcpyAsync(payload + c.begin, staged, span, hipMemcpyDefault, stream),
                     "hipMemcpyAsync(host tensors -> payload)");
    } else {
      rc = check_hip(hipMemcpyAsync(staged, payload + c.begin, span, hipMemcpyDefault, stream),
                     "hipMemcpyAsync(payload -> host tensors)");
    }
    if (rc) return rc;
    rc = check_hip(hipEventRecord(st->ready, stream), "hipEventRecord(staging)");
    if (rc) return rc;
    st->pending = true;
  }
  if (!pack) {
    for (size_t k = nchunks >= 2 ? nchunks - 2 : 0; k < nchunks; ++k) {
      HostStage* st = &p->stage[k & 1];
      int rc = stage_ready(st);
      if (rc) return rc;
      pieces_out(p->host_chunks[k], static_cast<const uint8_t*>(st->block.host));
    }
  }
  return AXR_OK;
}

// Small bundles with the default launch geometry can carry their tables inside the
// kernel arguments (3.5 KiB at most) instead of a device block.
bool tables_fit_kernel_arguments(const axr_plan* p) {
  const int64_t limit = tunables().inline_tables;
  return limit > 0 && p->tables_built && p->ntiles <= static_cast<uint64_t>(limit) &&
         p->table_bytes + kInlineTablesHead <= kInlineTableBytes && p->cfg.tile_rows == 2 &&
         (p->cfg.nontemporal & 3u) == 1u && !p->cfg.xcd_remap;
}

void fill_inline_tables(axr_plan* p) {
  if (!p->inline_tables) p->inline_tables.reset(new InlineTables());
  uint8_t* b = p->inline_tables->bytes;
  std::memset(b, 0, kInlineTablesHead);
  std::memcpy(b, &kInlineTablesMark, sizeof(kInlineTablesMark));
  write_tables(p, b + kInlineTablesHead);
  p->inline_ready = true;
}

// The cache hint bits a job runs with: the plan's own, or with the payload side forced.
uint32_t effective_nontemporal(const axr_plan* p, uint32_t job_flags) {
  uint32_t nt = p->cfg.nontemporal & 3u;
  if (job_flags & AXR_JOB_PAYLOAD_STREAMING) nt |= 2u;
  else if (job_flags & AXR_JOB_PAYLOAD_CACHED) nt &= ~2u;
  return nt;
}

int run(axr_plan* p, bool pack, void* payload, size_t payload_bytes, void* stream_, int64_t delta = 0,
        uint32_t job_flags = 0) {
  if (!p) return fail(AXR_ERR_INVALID, "null plan");
  if (!p->bound) return fail(AXR_ERR_INVALID, "plan has no tensor addresses bound");
  if (payload_bytes < p->payload_bytes)
    return fail(AXR_ERR_LENGTH, "payload buffer is smaller than the plan's payload");
  if (p->payload_bytes == 0) return AXR_OK;
  if (!payload) return fail(AXR_ERR_INVALID, "null payload");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  // Under stream capture only the kernel launch may be recorded: the tables must be
  // resident already (axr_plan_prepare) and nothing may wait on the host.
  bool capturing = false;
  int rc = AXR_OK;
  if (stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    rc = check_hip(hipStreamIsCapturing(stream, &status), "hipStreamIsCapturing");
    if (rc) return rc;
    capturing = status == hipStreamCaptureStatusActive;
  }
  rc = ensure_tables(p, stream, capturing);
  if (rc) return rc;
  if (!pack && p->overlapping_dst)
    return fail(AXR_ERR_INVALID, "unpack destination has overlapping elements (zero stride)");
  if (capturing) {
    if (!p->host_chunks.empty())
      return fail(AXR_ERR_UNSUPPORTED, "a bundle with host (kDLCPU) tensors cannot be captured in a graph");
  }
  if (!p->host_chunks.empty()) {
    if (delta != 0)
      return fail(AXR_ERR_UNSUPPORTED, "a tensor address delta cannot be applied to host (kDLCPU) tensors");
    rc = move_host_tensors(p, pack, static_cast<uint8_t*>(payload), stream);
    remember_stream(p, stream);
    if (rc) return rc;
  }
  if (p->ntiles == 0) return AXR_OK;
  KernelArgs a;
  a.payload = static_cast<uint8_t*>(payload);
  a.nseg = p->segs.empty() ? 0u : static_cast<uint32_t>(p->segs.size() - 1);
  a.ntiles = p->ntiles;
  a.tiles_per_wave = p->cfg.tiles_per_wave;
  a.xcd_remap = p->cfg.xcd_remap ? p->cfg.workgroups / kXcds : 0;
  a.seg_shift = p->cfg.seg_shift;
  a.tensor_delta = delta;
  LaunchConfig cfg = p->cfg;
  cfg.nontemporal = effective_nontemporal(p, job_flags);
  if (delta == 0 && cfg.nontemporal == (p->cfg.nontemporal & 3u) &&
      (capturing ? !p->resident : p->launches == 0 && !p->uploaded) && tables_fit_kernel_arguments(p)) {
    // Small bundle, first launch: the tables ride in the kernel arguments.  The launch
    // owns its copy, so a capturing stream may record it.  A plan that is launched again
    // is being reused: from the second launch on it pays one upload and then the shorter
    // argument list (a 3.5 KiB argument costs 0.4 us per launch, the upload 4 us on the
    // host and 4 us on the device, once).
    if (!p->inline_ready) fill_inline_tables(p);
    rc = launch_bundle_kernel_inline(pack, a, p->cfg, *p->inline_tables,
                                     static_cast<uint32_t>(dims_arg_at(p)),
                                     static_cast<uint32_t>(p->wave_at), stream);
    if (rc) return rc;
    ++p->launches;
    if (!pack && p->pinned_host_tensors) stream_note_host_writes(stream);
    // The launch needs nothing of the plan any more, but callers rely on axr_plan_free and
    // axr_plan_bind returning only when the plan's launches are done (they release the
    // payload or the tensors next), so the stream is remembered all the same.
    if (!capturing) remember_stream(p, stream);
    return AXR_OK;
  }
  if (capturing && !p->resident)
    return fail(AXR_ERR_INVALID, "call axr_plan_prepare before capturing this plan in a graph");
  if (!p->resident) {
    rc = ensure_uploaded(p, stream);
    if (rc) return rc;
  }
  uint8_t* d = static_cast<uint8_t*>(p->block.device);
  a.segs = reinterpret_cast<const Seg*>(d);
  a.dims = reinterpret_cast<const Dims*>(d + dims_arg_at(p));
  a.wave_seg = reinterpret_cast<const uint32_t*>(d + p->wave_at);
  rc = launch_bundle_kernel(pack, a, cfg, stream);
  if (rc) return rc;
  ++p->launches;
  if (!pack && p->pinned_host_tensors) stream_note_host_writes(stream);
  // a capturing stream cannot be drained later; the caller keeps the plan alive
  // for as long as the graph can run
  if (!capturing) remember_stream(p, stream);
  return AXR_OK;
}

int store_tensor(std::vector<int64_t>& dims64, const axr_tensor_t& in, TensorRec* rec) {
  rec->device_type = in.device_type;
  rec->device_id = in.device_id;
  rec->ndim = in.ndim;
  rec->code = in.dtype_code;
  rec->bits = in.dtype_bits;
  rec->lanes = in.dtype_lanes;
  int rc = nbytes_rule(in.ndim, in.shape, in.dtype_bits, &rec->nbytes);
  if (rc) return rc;
  rec->shape_at = static_cast<uint32_t>(dims64.size());
  rec->strides_at = 0;
  rec->has_strides = in.strides != nullptr && in.ndim > 0;
  if (in.ndim == 1) {
    dims64.push_back(in.shape[0]);
    if (rec->has_strides) {
      rec->strides_at = rec->shape_at + 1;
      dims64.push_back(in.strides[0]);
    }
  } else {
    dims64.insert(dims64.end(), in.shape, in.shape + in.ndim);
    if (rec->has_strides) {
      rec->strides_at = static_cast<uint32_t>(dims64.size());
      dims64.insert(dims64.end(), in.strides, in.strides + in.ndim);
    }
  }
  if (rec->nbytes != 0 && in.data == nullptr)
    return fail(AXR_ERR_INVALID, "tensor data pointer is null");
  rec->address = reinterpret_cast<uint64_t>(in.data) + in.byte_offset;
  return AXR_OK;
}

}  // namespace

extern "C" {

static int tensor_nbytes_body(const axr_tensor_t* t, uint64_t* nbytes) {
  if (!t || !nbytes) return fail(AXR_ERR_INVALID, "axr_tensor_nbytes: null argument");
  return nbytes_rule(t->ndim, t->shape, t->dtype_bits, nbytes);
}
int axr_tensor_nbytes(const axr_tensor_t* t, uint64_t* nbytes) {
  return guarded([&] { return tensor_nbytes_body(t, nbytes); });
}

static int plan_create_body(const axr_tensor_t* tensors, size_t n, uint32_t align, uint32_t flags,
                            axr_plan_t** plan) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_create: null result");
  *plan = nullptr;
  if (n && !tensors) return fail(AXR_ERR_INVALID, "axr_plan_create: null tensor array");
  if (n > 0xffffffffull) return fail(AXR_ERR_INVALID, "axr_plan_create: too many tensors");
  if (flags != 0) return fail(AXR_ERR_INVALID, "axr_plan_create: flags are reserved and must be 0");
  int rc = check_align(align);
  if (rc) return rc;
  PlanInProgress guard(plan_new());
  axr_plan* p = guard.p;
  if (!p) return fail(AXR_ERR_NOMEM, "axr_plan_create: out of host memory");
  p->align = align;
  p->tensors.resize(n);
  p->dims64.clear();
  p->dims64.reserve(2 * n);
  // one pass: tensor record, layout and header record (the header grows as shapes come in)
  RawVec<uint8_t>& h = p->header;
  h.resize(kFixedHeader + n * (kTensorHeader + 16));
  uint8_t* w = h.data() + kFixedHeader;
  uint64_t off = 0, data = 0, end = 0;
  const uint64_t mask = static_cast<uint64_t>(align) - 1;
  for (size_t i = 0; i < n; ++i) {
    TensorRec& t = p->tensors[i];
    rc = store_tensor(p->dims64, tensors[i], &t);
    if (rc) {
      return rc;
    }
    {
      // room for this record and every fixed part still to come
      const size_t at = static_cast<size_t>(w - h.data());
      const size_t need = at + 8 * static_cast<size_t>(t.ndim) + (n - i) * kTensorHeader;
      if (need > h.size()) {
        h.resize(std::max(need, h.size() + h.size() / 2));
        w = h.data() + at;
      }
    }
    if (__builtin_add_overflow(off, mask, &off) || (off &= ~mask, __builtin_add_overflow(off, t.nbytes, &end))) {
      return fail(AXR_ERR_INVALID, "axr_plan_create: bundle size overflows 64 bits");
    }
    t.offset = off;
    off = end;
    data += t.nbytes;
    WireTensor rec;
    rec.offset = t.offset;
    rec.nbytes = t.nbytes;
    rec.device_type = t.device_type;
    rec.device_id = t.device_id;
    rec.ndim = t.ndim;
    rec.code = t.code;
    rec.bits = t.bits;
    rec.lanes = t.lanes;
    rec.byte_offset = 0;   // the packed copy starts at its offset
    std::memcpy(w, &rec, kTensorHeader);
    w += kTensorHeader;
    if (t.ndim == 1) {   // the common case without a call
      std::memcpy(w, tensors[i].shape, 8);
      w += 8;
    } else if (t.ndim) {
      std::memcpy(w, tensors[i].shape, 8 * static_cast<size_t>(t.ndim));
      w += 8 * static_cast<size_t>(t.ndim);
    }
  }
  h.resize(static_cast<size_t>(w - h.data()));
  p->payload_bytes = end;
  p->data_bytes = data;
  encode_preamble(p);
  p->bound = true;
  *plan = guard.release();
  return AXR_OK;
}
int axr_plan_create(const axr_tensor_t* tensors,
                    size_t n,
                    uint32_t align,
                    uint32_t flags,
                    axr_plan_t** plan) {
  return guarded([&] { return plan_create_body(tensors, n, align, flags, plan); });
}

static int plan_free_body(axr_plan_t* plan) {
  if (!plan) return AXR_OK;
  quiesce(plan);
  if (plan->uploaded && plan->upload_event) (void)hipEventSynchronize(plan->upload_event);
  table_block_release(&plan->block);
  event_release(plan->upload_event, plan->upload_event_device);   // fired, or never recorded
  plan->upload_event = nullptr;
  for (HostStage& st : plan->stage) {
    table_block_release(&st.block);
    if (st.ready) (void)hipEventDestroy(st.ready);
  }
  plan_delete(plan);
  return AXR_OK;
}
int axr_plan_free(axr_plan_t* plan) {
  return guarded([&] { return plan_free_body(plan); });
}

static int plan_num_tensors_body(const axr_plan_t* plan, size_t* n) {
  if (!plan || !n) return fail(AXR_ERR_INVALID, "axr_plan_num_tensors: null argument");
  *n = plan->tensors.size();
  return AXR_OK;
}
int axr_plan_num_tensors(const axr_plan_t* plan, size_t* n) {
  return guarded([&] { return plan_num_tensors_body(plan, n); });
}

static int plan_payload_bytes_body(const axr_plan_t* plan, uint64_t* bytes) {
  if (!plan || !bytes) return fail(AXR_ERR_INVALID, "axr_plan_payload_bytes: null argument");
  *bytes = plan->payload_bytes;
  return AXR_OK;
}
int axr_plan_payload_bytes(const axr_plan_t* plan, uint64_t* bytes) {
  return guarded([&] { return plan_payload_bytes_body(plan, bytes); });
}

static int plan_data_bytes_body(const axr_plan_t* plan, uint64_t* bytes) {
  if (!plan || !bytes) return fail(AXR_ERR_INVALID, "axr_plan_data_bytes: null argument");
  *bytes = plan->data_bytes;
  return AXR_OK;
}
int axr_plan_data_bytes(const axr_plan_t* plan, uint64_t* bytes) {
  return guarded([&] { return plan_data_bytes_body(plan, bytes); });
}

static int plan_layout_body(const axr_plan_t* plan, uint64_t* offsets, uint64_t* sizes) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_layout: null plan");
  for (size_t i = 0; i < plan->tensors.size(); ++i) {
    if (offsets) offsets[i] = plan->tensors[i].offset;
    if (sizes) sizes[i] = plan->tensors[i].nbytes;
  }
  return AXR_OK;
}
int axr_plan_layout(const axr_plan_t* plan, uint64_t* offsets, uint64_t* sizes) {
  return guarded([&] { return plan_layout_body(plan, offsets, sizes); });
}

static int plan_tensor_meta_body(const axr_plan_t* plan, size_t i, axr_tensor_t* meta) {
  if (!plan || !meta) return fail(AXR_ERR_INVALID, "axr_plan_tensor_meta: null argument");
  if (i >= plan->tensors.size()) return fail(AXR_ERR_INVALID, "axr_plan_tensor_meta: index out of range");
  const TensorRec& t = plan->tensors[i];
  meta->data = nullptr;
  meta->device_type = t.device_type;
  meta->device_id = t.device_id;
  meta->ndim = t.ndim;
  meta->dtype_code = t.code;
  meta->dtype_bits = t.bits;
  meta->dtype_lanes = t.lanes;
  meta->shape = t.ndim ? const_cast<int64_t*>(plan->shape_of(t)) : nullptr;
  meta->strides = const_cast<int64_t*>(plan->strides_of(t));
  meta->byte_offset = 0;
  return AXR_OK;
}
int axr_plan_tensor_meta(const axr_plan_t* plan, size_t i, axr_tensor_t* meta) {
  return guarded([&] { return plan_tensor_meta_body(plan, i, meta); });
}

static int plan_header_body(const axr_plan_t* plan, const void** header, size_t* length) {
  if (!plan || !header || !length) return fail(AXR_ERR_INVALID, "axr_plan_header: null argument");
  *header = plan->header.data();
  *length = plan->header.size();
  return AXR_OK;
}
int axr_plan_header(const axr_plan_t* plan, const void** header, size_t* length) {
  return guarded([&] { return plan_header_body(plan, header, length); });
}

// `bound` (may be null): the receiver's tensors, attached in the same pass (axr_plan_from_header
// followed by axr_plan_bind, without a second walk over the records).
static int plan_from_header_body(const void* header, size_t length, const axr_tensor_t* bound,
                                 size_t nbound, bool binding, axr_plan_t** plan) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_from_header: null result");
  *plan = nullptr;
  if (!header) return fail(AXR_ERR_INVALID, "axr_plan_from_header: null header");
  const uint8_t* h = static_cast<const uint8_t*>(header);
  if (length < kFixedHeader) return fail(AXR_ERR_HEADER, "bundle header shorter than its fixed part");
  if (get<uint32_t>(h) != kMagic) return fail(AXR_ERR_HEADER, "bundle header has a wrong magic");
  if (get<uint16_t>(h + 4) != kVersion) return fail(AXR_ERR_HEADER, "bundle header version not supported");
  if (get<uint16_t>(h + 6) != 0) return fail(AXR_ERR_HEADER, "bundle header has unknown flags");
  const uint32_t n = get<uint32_t>(h + 8);
  const uint32_t align = get<uint32_t>(h + 12);
  const uint64_t payload = get<uint64_t>(h + 16);
  if (check_align(align) != AXR_OK) return fail(AXR_ERR_HEADER, "bundle header has a bad alignment");
  if (static_cast<uint64_t>(n) * kTensorHeader > length - kFixedHeader)
    return fail(AXR_ERR_HEADER, "bundle header truncated");
  if (binding) {
    if (nbound != n) return fail(AXR_ERR_MISMATCH, "axr_plan_from_header_bind: tensor count differs from the header");
    if (n && !bound) return fail(AXR_ERR_INVALID, "axr_plan_from_header_bind: null tensor array");
  }
  PlanInProgress guard(plan_new());
  axr_plan* p = guard.p;
  if (!p) return fail(AXR_ERR_NOMEM, "axr_plan_from_header: out of host memory");
  p->align = align;
  p->tensors.resize(n);
  p->dims64.reserve((length - kFixedHeader - static_cast<size_t>(n) * kTensorHeader) / 8 * (binding ? 2 : 1));
  size_t at = kFixedHeader;
  uint64_t expect = 0, end = 0, data = 0;
  const uint64_t mask = static_cast<uint64_t>(align) - 1;
  if ((length - kFixedHeader - static_cast<size_t>(n) * kTensorHeader) / 8 > 0xffffffffull) {
    return fail(AXR_ERR_HEADER, "bundle header too long");
  }
  for (uint32_t i = 0; i < n; ++i) {
    if (length - at < kTensorHeader) {
      return fail(AXR_ERR_HEADER, "bundle header truncated");
    }
    TensorRec& t = p->tensors[i];
    WireTensor rec;
    std::memcpy(&rec, h + at, kTensorHeader);
    const uint64_t off = rec.offset, nb = rec.nbytes, byte_offset = rec.byte_offset;
    t.device_type = rec.device_type;
    t.device_id = rec.device_id;
    t.ndim = rec.ndim;
    t.code = rec.code;
    t.bits = rec.bits;
    t.lanes = rec.lanes;
    at += kTensorHeader;
    if (t.ndim < 0 || t.ndim > kMaxNdim ||
        static_cast<size_t>(t.ndim) * 8 > length - at || byte_offset != 0) {
      return fail(AXR_ERR_HEADER, "bundle header has a bad tensor record");
    }
    uint64_t rule = 0;
    int sized;
    if (!binding) {
      t.address = 0;
      t.strides_at = 0;
      t.has_strides = false;
      t.shape_at = static_cast<uint32_t>(p->dims64.size());
      if (t.ndim == 1) {
        p->dims64.push_back(get<int64_t>(h + at));
      } else if (t.ndim) {
        p->dims64.resize(t.shape_at + static_cast<size_t>(t.ndim));
        std::memcpy(p->dims64.data() + t.shape_at, h + at, 8 * static_cast<size_t>(t.ndim));
      }
      sized = nbytes_rule(t.ndim, p->dims64.data() + t.shape_at, t.bits, &rule);
    } else {
      int64_t sent_shape[kMaxNdim];   // the record's shape is only checked; the bound tensor's is kept
      if (t.ndim == 1) {
        std::memcpy(sent_shape, h + at, 8);
      } else {
        std::memcpy(sent_shape, h + at, 8 * static_cast<size_t>(t.ndim));
      }
      sized = nbytes_rule(t.ndim, sent_shape, t.bits, &rule);
    }
    at += static_cast<size_t>(t.ndim) * 8;
    if (sized != AXR_OK || rule != nb) {
      return fail(AXR_ERR_HEADER, "bundle header tensor size does not follow from its shape");
    }
    if (binding) {
      const uint32_t sent_item = (static_cast<uint32_t>(t.bits) + 7) / 8;
      int rc = store_tensor(p->dims64, bound[i], &t);   // size rule, null checks; replaces the record
      if (rc) {
        return rc;
      }
      if (t.nbytes != nb || (nb != 0 && (static_cast<uint32_t>(t.bits) + 7) / 8 != sent_item)) {
        return fail(AXR_ERR_MISMATCH, "axr_plan_from_header_bind: tensor " + std::to_string(i) +
                                          " does not match the header's size or element width");
      }
    }
    // the offset must be the one the layout rule gives (no wrapping of 64 bits on the way)
    uint64_t stop = 0;
    if (__builtin_add_overflow(expect, mask, &expect) || (expect &= ~mask, expect != off) ||
        __builtin_add_overflow(off, nb, &stop)) {
      return fail(AXR_ERR_HEADER, "bundle header offsets do not follow the layout rule");
    }
    expect = end = stop;
    data += nb;
    t.nbytes = nb;
    t.offset = off;
  }
  if (at != length) {
    return fail(AXR_ERR_HEADER, "bundle header has trailing bytes");
  }
  if (end != payload) {
    return fail(AXR_ERR_HEADER, "bundle header offsets do not follow the layout rule");
  }
  p->payload_bytes = end;
  p->data_bytes = data;
  p->header.assign(h, h + length);
  p->bound = binding;
  p->receiver = true;
  *plan = guard.release();
  return AXR_OK;
}
int axr_plan_from_header(const void* header, size_t length, axr_plan_t** plan) {
  return guarded([&] { return plan_from_header_body(header, length, nullptr, 0, false, plan); });
}
int axr_plan_from_header_bind(const void* header, size_t length, const axr_tensor_t* tensors, size_t n,
                              axr_plan_t** plan) {
  return guarded([&] { return plan_from_header_body(header, length, tensors, n, true, plan); });
}

static int plan_bind_body(axr_plan_t* plan, const axr_tensor_t* tensors, size_t n) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_bind: null plan");
  if (n != plan->tensors.size())
    return fail(AXR_ERR_MISMATCH, "axr_plan_bind: tensor count differs from the plan");
  if (n && !tensors) return fail(AXR_ERR_INVALID, "axr_plan_bind: null tensor array");
  // Everything is validated and staged first (in vectors the plan keeps for this): a
  // failure leaves the plan as it was.
  RawVec<TensorRec>& recs = plan->staged_tensors;
  std::vector<int64_t>& dims64 = plan->staged_dims64;
  recs.resize(n);
  dims64.clear();
  dims64.reserve(plan->dims64.size() * 2);
  for (size_t i = 0; i < n; ++i) {
    const TensorRec& t = plan->tensors[i];
    int rc = store_tensor(dims64, tensors[i], &recs[i]);   // size rule, null checks
    if (rc) return rc;
    if (recs[i].nbytes != t.nbytes ||
        (t.nbytes != 0 && (recs[i].bits + 7) / 8 != (t.bits + 7) / 8))
      return fail(AXR_ERR_MISMATCH, "axr_plan_bind: tensor " + std::to_string(i) +
                                        " does not match the plan's size or element width");
    recs[i].offset = t.offset;
  }
  quiesce(plan);
  invalidate_tables(plan);
  // The header keeps describing what was sent; the bound records describe memory.
  plan->tensors.swap(recs);
  plan->dims64.swap(dims64);
  plan->bound = true;
  return AXR_OK;
}
int axr_plan_bind(axr_plan_t* plan, const axr_tensor_t* tensors, size_t n) {
  return guarded([&] { return plan_bind_body(plan, tensors, n); });
}

static int plan_split_body(const axr_plan_t* plan, void* payload, size_t payload_bytes,
                           axr_buffer_t* views) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_split: null plan");
  if (plan->payload_bytes > payload_bytes)
    return fail(AXR_ERR_LENGTH, "Total size of chunks exceeds buffer size");
  if (plan->tensors.empty()) return AXR_OK;
  if (!views) return fail(AXR_ERR_INVALID, "axr_plan_split: null views");
  for (size_t i = 0; i < plan->tensors.size(); ++i) {
    views[i].data = static_cast<uint8_t*>(payload) + plan->tensors[i].offset;
    views[i].size = plan->tensors[i].nbytes;
  }
  return AXR_OK;
}
int axr_plan_split(const axr_plan_t* plan,
                   void* payload,
                   size_t payload_bytes,
                   axr_buffer_t* views) {
  return guarded([&] { return plan_split_body(plan, payload, payload_bytes, views); });
}

static int pack_body(axr_plan_t* plan, void* payload, size_t payload_bytes, void* stream) {
  return run(plan, true, payload, payload_bytes, stream);
}
int axr_pack(axr_plan_t* plan, void* payload, size_t payload_bytes, void* stream) {
  return guarded([&] { return pack_body(plan, payload, payload_bytes, stream); });
}

static int unpack_body(axr_plan_t* plan, const void* payload, size_t payload_bytes, void* stream) {
  return run(plan, false, const_cast<void*>(payload), payload_bytes, stream);
}
int axr_unpack(axr_plan_t* plan, const void* payload, size_t payload_bytes, void* stream) {
  return guarded([&] { return unpack_body(plan, payload, payload_bytes, stream); });
}

// Who used the static table area of a device last, and an event behind that use.
struct StaticAreaUse {
  std::mutex mu;
  hipEvent_t after_launch = nullptr;   // created at the first use, kept until the process ends
  hipStream_t last_stream = nullptr;
  bool used = false;
};
static StaticAreaUse& static_area_use(int device) {
  static StaticAreaUse uses[64];
  return uses[device >= 0 && device < 64 ? device : 0];
}

// axr_pack for callers that must not allocate device memory.  The tables ride in the
// kernel arguments when they fit; otherwise they are copied, on `stream`, into the static
// table area of the current device and the same kernel as axr_pack reads them there.
static int pack_noalloc_body(axr_plan_t* p, void* payload, size_t payload_bytes, void* stream_) {
  if (!p) return fail(AXR_ERR_INVALID, "null plan");
  if (!p->bound) return fail(AXR_ERR_INVALID, "plan has no tensor addresses bound");
  if (payload_bytes < p->payload_bytes)
    return fail(AXR_ERR_LENGTH, "payload buffer is smaller than the plan's payload");
  if (p->payload_bytes == 0) return AXR_OK;
  if (!payload) return fail(AXR_ERR_INVALID, "null payload");
  int rc = build_tables(p);   // host memory only
  if (rc) return rc;
  if (!p->host_chunks.empty())
    return fail(AXR_ERR_UNSUPPORTED,
                "axr_pack_noalloc: host (kDLCPU) tensors need pinned staging blocks; use axr_pack");
  if (p->ntiles == 0) return AXR_OK;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  bool capturing = false;
  if (stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    rc = check_hip(hipStreamIsCapturing(stream, &status), "hipStreamIsCapturing");
    if (rc) return rc;
    capturing = status == hipStreamCaptureStatusActive;
  }
  KernelArgs a;
  a.payload = static_cast<uint8_t*>(payload);
  a.nseg = static_cast<uint32_t>(p->segs.size() - 1);
  a.ntiles = p->ntiles;
  a.tiles_per_wave = p->cfg.tiles_per_wave;
  a.xcd_remap = p->cfg.xcd_remap ? p->cfg.workgroups / kXcds : 0;
  a.seg_shift = p->cfg.seg_shift;
  auto remember = [&] {
    if (!capturing) remember_stream(p, stream);
  };
  if (tables_fit_kernel_arguments(p)) {
    if (!p->inline_ready) fill_inline_tables(p);
    rc = launch_bundle_kernel_inline(true, a, p->cfg, *p->inline_tables,
                                     static_cast<uint32_t>(dims_arg_at(p)),
                                     static_cast<uint32_t>(p->wave_at), stream);
    if (rc) return rc;
    ++p->launches;
    remember();
    return AXR_OK;
  }
  if (p->table_bytes > kStaticTableBytes)
    return fail(AXR_ERR_LENGTH, "axr_pack_noalloc: the bundle's tables need " +
                                    std::to_string(p->table_bytes) + " bytes, the static table area holds " +
                                    std::to_string(kStaticTableBytes) + "; use axr_pack");
  if (capturing)
    return fail(AXR_ERR_UNSUPPORTED,
                "axr_pack_noalloc: tables beyond the kernel arguments cannot be recorded into a graph");
  void* area = nullptr;
  rc = static_table_area(&area);
  if (rc) return rc;
  uint8_t* d = static_cast<uint8_t*>(area);
  // Calls on one stream are ordered by the stream.  A call on ANOTHER stream than the area's
  // last user first waits (on the device, not on the host) for that user's launch: an event,
  // created once per device, is recorded behind every launch that reads the area.
  int device = 0;
  rc = check_hip(hipGetDevice(&device), "hipGetDevice");
  if (rc) return rc;
  StaticAreaUse& use = static_area_use(device);
  std::lock_guard<std::mutex> area_lock(use.mu);
  if (!use.after_launch) {
    rc = check_hip(hipEventCreateWithFlags(&use.after_launch, hipEventDisableTiming), "hipEventCreate(static table area)");
    if (rc) return rc;
  }
  if (use.used && use.last_stream != stream) {
    rc = check_hip(hipStreamWaitEvent(stream, use.after_launch, 0), "hipStreamWaitEvent(static table area)");
    if (rc) return rc;
  }
  // Copies out of the plan's own (pageable) vectors, ordered on `stream`.  The vectors live
  // until the plan is rebound or freed, and both drain the stream first; the launch mark is
  // taken once something has been enqueued, also when a later step fails.
  bool enqueued = false;
  auto copy = [&](size_t at, const void* src, size_t bytes, const char* what) {
    if (rc || bytes == 0) return;
    rc = check_hip(hipMemcpyAsync(d + at, src, bytes, hipMemcpyHostToDevice, stream), what);
    enqueued = enqueued || rc == AXR_OK;
  };
  copy(0, p->segs.data(), p->segs.size() * sizeof(Seg), "hipMemcpyAsync(segment table -> static area)");
  copy(p->dims_at, p->dims.data(), p->dims.size() * sizeof(Dims), "hipMemcpyAsync(dims table -> static area)");
  copy(p->wave_at, p->wave_seg.data(), p->wave_seg.size() * sizeof(uint32_t), "hipMemcpyAsync(tile index -> static area)");
  copy(p->members_at, p->group_blocks.data(), p->group_blocks.size(), "hipMemcpyAsync(group blocks -> static area)");
  if (!rc) {
    a.segs = reinterpret_cast<const Seg*>(d);
    a.dims = reinterpret_cast<const Dims*>(d + dims_arg_at(p));
    a.wave_seg = reinterpret_cast<const uint32_t*>(d + p->wave_at);
    rc = launch_bundle_kernel(true, a, p->cfg, stream);
    if (!rc) ++p->launches;
  }
  if (enqueued) {
    remember();
    use.used = true;
    use.last_stream = stream;
    const int recorded = check_hip(hipEventRecord(use.after_launch, stream), "hipEventRecord(static table area)");
    if (!rc) rc = recorded;
  }
  return rc;
}
int axr_pack_noalloc(axr_plan_t* plan, void* payload, size_t payload_bytes, void* stream) {
  return guarded([&] { return pack_noalloc_body(plan, payload, payload_bytes, stream); });
}

// Several bundles on one stream, neighbours of one launch geometry sharing a launch.
static int submit_body(const axr_job_t* jobs, size_t n, void* stream_) {
  if (n == 0) return AXR_OK;
  if (!jobs) return fail(AXR_ERR_INVALID, "axr_submit: null job array");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  bool capturing = false;
  if (stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    int rc = check_hip(hipStreamIsCapturing(stream, &status), "hipStreamIsCapturing");
    if (rc) return rc;
    capturing = status == hipStreamCaptureStatusActive;
  }
  // Everything is checked, and every table built, before the first launch: a refused job
  // leaves nothing half submitted.
  for (size_t i = 0; i < n; ++i) {
    const axr_job_t& j = jobs[i];
    axr_plan* p = j.plan;
    if (!p) return fail(AXR_ERR_INVALID, "axr_submit: null plan in job " + std::to_string(i));
    if ((j.flags & ~(AXR_JOB_PAYLOAD_STREAMING | AXR_JOB_PAYLOAD_CACHED)) ||
        (j.flags & (AXR_JOB_PAYLOAD_STREAMING | AXR_JOB_PAYLOAD_CACHED)) ==
            (AXR_JOB_PAYLOAD_STREAMING | AXR_JOB_PAYLOAD_CACHED))
      return fail(AXR_ERR_INVALID, "axr_submit: bad flags in job " + std::to_string(i));
    if (!p->bound) return fail(AXR_ERR_INVALID, "plan has no tensor addresses bound");
    if (j.payload_bytes < p->payload_bytes)
      return fail(AXR_ERR_LENGTH, "payload buffer is smaller than the plan's payload");
    if (p->payload_bytes && !j.payload) return fail(AXR_ERR_INVALID, "null payload");
    for (size_t k = 0; k < i; ++k)
      if (jobs[k].plan == p) return fail(AXR_ERR_INVALID, "axr_submit: one plan appears in two jobs");
    int rc = ensure_tables(p, stream, capturing);
    if (rc) return rc;
    if (j.unpack && p->overlapping_dst)
      return fail(AXR_ERR_INVALID, "unpack destination has overlapping elements (zero stride)");
    if (!p->host_chunks.empty() && (capturing || j.tensor_delta != 0))
      return fail(AXR_ERR_UNSUPPORTED, "a bundle with host (kDLCPU) tensors can neither be captured nor rebased");
    if (capturing && p->ntiles && !p->resident)
      return fail(AXR_ERR_INVALID, "call axr_plan_prepare before capturing this plan in a graph");
  }
  auto batchable = [](const axr_plan* p) {
    return p->ntiles != 0 && p->host_chunks.empty() && !p->cfg.xcd_remap &&
           (!p->cfg.elements || p->cfg.tile_rows == 2);
  };
  auto same_geometry = [](const axr_job_t& jx, const axr_job_t& jy) {
    const axr_plan *x = jx.plan, *y = jy.plan;
    return x->cfg.tile_rows == y->cfg.tile_rows && x->cfg.threads == y->cfg.threads &&
           effective_nontemporal(x, jx.flags) == effective_nontemporal(y, jy.flags) &&
           (!(x->cfg.elements || y->cfg.elements) || (x->cfg.tile_rows == 2 && x->cfg.threads <= kMaxElementThreads));
  };
  size_t i = 0;
  while (i < n) {
    axr_plan* first = jobs[i].plan;
    size_t end = i + 1;
    if (batchable(first)) {
      while (end < n && end - i < kMaxJobs && batchable(jobs[end].plan) &&
             same_geometry(jobs[i], jobs[end]))
        ++end;
    }
    if (end - i == 1) {
      const axr_job_t& j = jobs[i];
      int rc = run(j.plan, j.unpack == 0, j.payload, j.payload_bytes, stream_, j.tensor_delta, j.flags);
      if (rc) return rc;
      i = end;
      continue;
    }
    JobTable table;
    std::memset(&table, 0, sizeof(table));
    LaunchConfig cfg = first->cfg;
    cfg.nontemporal = effective_nontemporal(first, jobs[i].flags);
    uint32_t wg = 0;
    // The jobs of a call do not depend on each other, so their order inside the launch is free:
    // gathers take the first workgroups, scatters follow.  A scatter then mostly runs while the
    // payload its gather wrote a launch earlier is still in the last-level cache and the new
    // gather's tensor reads are under way (48 MB mixed bundle: 6.37 against 6.15 TB/s the other
    // way round).
    size_t order[kMaxJobs];
    size_t slots = 0;
    for (int unpacks = 0; unpacks < 2; ++unpacks)
      for (size_t k = i; k < end; ++k)
        if ((jobs[k].unpack != 0) == (unpacks != 0)) order[slots++] = k;
    for (size_t slot = 0; slot < slots; ++slot) {
      const size_t k = order[slot];
      const axr_job_t& j = jobs[k];
      axr_plan* p = j.plan;
      if (!p->resident) {
        int rc = ensure_uploaded(p, stream);
        if (rc) return rc;
      }
      const uint8_t* d = static_cast<const uint8_t*>(p->block.device);
      JobDesc& jd = table.job[slot];
      jd.segs = reinterpret_cast<uint64_t>(d);
      jd.dims = reinterpret_cast<uint64_t>(d + dims_arg_at(p));
      jd.wave_seg = reinterpret_cast<uint64_t>(d + p->wave_at);
      jd.payload = reinterpret_cast<uint64_t>(j.payload);
      jd.tensor_delta = j.tensor_delta;
      jd.ntiles = p->ntiles;
      jd.tiles_per_wave = p->cfg.tiles_per_wave;
      jd.seg_shift = p->cfg.seg_shift;
      jd.wg_begin = wg;
      jd.unpack = j.unpack ? 1u : 0u;
      if (static_cast<uint64_t>(wg) + p->cfg.workgroups > 0x7fffffffull)
        return fail(AXR_ERR_UNSUPPORTED, "axr_submit: the jobs' grids exceed one launch");
      wg += p->cfg.workgroups;
      cfg.elements = cfg.elements || p->cfg.elements;
      cfg.lds_per_wave = std::max(cfg.lds_per_wave, p->cfg.lds_per_wave);
    }
    table.count = static_cast<uint32_t>(end - i);
    for (uint32_t k = 0; k < kMaxJobs; ++k) table.begins[k] = k < table.count ? table.job[k].wg_begin : kNoJobBegin;
    const int64_t interleave = tunables().submit_interleave;
    if (interleave != 0 && (cfg.nontemporal & 2u) != 0 && end - i == 2 &&   // the streaming instantiations carry the code
        jobs[i + 1].plan->cfg.workgroups == first->cfg.workgroups) {
      const uint64_t cache = static_cast<uint64_t>(tunables().payload_cache_bytes);
      const bool beyond_cache = first->payload_bytes > cache && jobs[i + 1].plan->payload_bytes > cache;
      table.interleaved = (beyond_cache || interleave > 1) ? 1u : 0u;
    }
    table.lds_per_wave = cfg.lds_per_wave;
    table.nt_bits = (cfg.nontemporal & 3u) | (cfg.threads / kWaveLanes) << 8;   // hints, wavefronts per workgroup
    cfg.workgroups = wg;
    if (cfg.lds_per_wave) {
      // every plan sized its workgroups for its own LDS need; the launch uses the largest
      const uint32_t fit = (64u * 1024u / cfg.lds_per_wave) * kWaveLanes;
      if (cfg.threads > fit)
        return fail(AXR_ERR_UNSUPPORTED, "axr_submit: jobs with transposed views of different block sizes");
    }
    int rc = launch_bundle_jobs(table, cfg, stream);
    if (rc) return rc;
    for (size_t k = i; k < end; ++k) {
      axr_plan* p = jobs[k].plan;
      ++p->launches;
      if (jobs[k].unpack && p->pinned_host_tensors) stream_note_host_writes(stream);
      if (!capturing) remember_stream(p, stream);
    }
    i = end;
  }
  return AXR_OK;
}
int axr_submit(const axr_job_t* jobs, size_t n, void* stream) {
  return guarded([&] { return submit_body(jobs, n, stream); });
}

static int plan_launch_info_body(axr_plan_t* plan, axr_launch_info_t* info) {
  if (!plan || !info) return fail(AXR_ERR_INVALID, "axr_plan_launch_info: null argument");
  int rc = build_tables(plan);
  if (rc) return rc;
  info->workgroups = plan->cfg.workgroups;
  info->threads_per_workgroup = plan->cfg.threads;
  info->tiles = plan->ntiles;
  info->tile_bytes = plan->cfg.tile_rows * kRowBytes;
  info->segments = static_cast<uint32_t>(plan->segs.size() - 1);
  info->table_bytes = static_cast<uint32_t>(plan->table_bytes);
  info->host_copies = static_cast<uint32_t>(plan->host_copies.size());
  info->host_chunks = static_cast<uint32_t>(plan->host_chunks.size());
  info->inline_tables = plan->ntiles && !plan->uploaded && plan->launches == 0 &&
                                tables_fit_kernel_arguments(plan)
                            ? 1u
                            : 0u;
  info->reserved = 0;
  return AXR_OK;
}
static int plan_prepare_body(axr_plan_t* plan, void* stream_) {
  if (!plan) return fail(AXR_ERR_INVALID, "axr_plan_prepare: null plan");
  if (!plan->bound) return fail(AXR_ERR_INVALID, "plan has no tensor addresses bound");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  int rc = ensure_tables(plan, stream, false);
  if (rc) return rc;
  if (plan->ntiles == 0 || plan->resident) return AXR_OK;
  rc = ensure_uploaded(plan, stream);
  if (rc) return rc;
  rc = check_hip(hipEventSynchronize(plan->upload_event), "hipEventSynchronize(plan tables)");
  if (rc) return rc;
  plan->resident = true;
  return AXR_OK;
}
int axr_plan_prepare(axr_plan_t* plan, void* stream) {
  return guarded([&] { return plan_prepare_body(plan, stream); });
}

int axr_plan_launch_info(axr_plan_t* plan, axr_launch_info_t* info) {
  return guarded([&] { return plan_launch_info_body(plan, info); });
}

static int plan_segments_body(axr_plan_t* plan, axr_segment_info_t* out, size_t capacity,
                              size_t* count) {
  if (!plan || !count) return fail(AXR_ERR_INVALID, "axr_plan_segments: null argument");
  int rc = build_tables(plan);
  if (rc) return rc;
  const size_t nseg = plan->segs.size() - 1;
  size_t groups = 0;
  for (size_t i = 0; i < nseg; ++i) groups += (plan->segs[i].meta >> kSegDimsShift) == kSegGroup ? 1 : 0;
  size_t members = 0;
  for (size_t g = 0; g < groups; ++g) {
    GroupHead head;
    std::memcpy(&head, plan->group_blocks.data() + g * kGroupBlockBytes, sizeof(head));
    members += head.members;
  }
  *count = nseg - groups + members + plan->host_copies.size();
  size_t w = 0;
  for (size_t i = 0; i < nseg && out && w < capacity; ++i, ++w) {
    const Seg& s = plan->segs[i];
    if ((s.meta >> kSegDimsShift) == kSegGroup) {
      // one entry per member; the group's single tile is counted with its first member
      const size_t block = (s.ptr - plan->members_at) / kGroupBlockBytes, n = s.run_bytes & 0xffu;
      for (size_t k = 0; k < n && w < capacity; ++k, ++w) {
        Member m;
        std::memcpy(&m, plan->group_blocks.data() + block * kGroupBlockBytes + sizeof(GroupHead) + k * sizeof(Member),
                    sizeof(m));
        axr_segment_info_t& o = out[w];
        std::memset(&o, 0, sizeof(o));
        o.tensor = plan->member_tensor[block * kGroupMaxMembers + k];
        o.mode = 6;
        o.address = m.ptr;
        o.offset = s.off + (m.off_pad & ((1u << kMemberOffBits) - 1u));
        o.run_bytes = o.nbytes = m.nbytes;
        o.pad = m.off_pad >> kMemberOffBits;
        o.tiles = k == 0 ? 1u : 0u;
        o.granule = m.begin;
        o.lanes_per_run = group_data_slots(m.nbytes) + group_pad_slots(o.pad);
      }
      --w;   // the loop header steps once more
      continue;
    }
    axr_segment_info_t& o = out[w];
    std::memset(&o, 0, sizeof(o));
    o.tensor = plan->seg_tensor[i];
    o.address = s.ptr;
    o.offset = s.off;
    o.run_bytes = s.run_bytes;
    o.pad = s.meta & kSegPadMask;
    o.tiles = plan->segs[i + 1].tile_begin - s.tile_begin;
    const uint32_t dsel = s.meta >> kSegDimsShift;
    if (dsel == 0) {
      o.mode = 0;
      o.run_bytes = s.run_bytes & kSegRunMask;
      o.head = static_cast<uint32_t>(s.run_bytes >> kSegHeadShift);
      o.nbytes = o.run_bytes;
    } else if (dsel == kSegFillOnly) {
      o.mode = 3;
    } else {
      const Dims& dm = plan->dims[dsel - 1];
      o.mode = dm.mode == kModeRunTiles ? 1 : (dm.mode == kModeElements ? 2 : 5);
      o.nbytes = dm.nbytes;
      o.ndim = dm.ndim;
      o.granule = dm.granule;
      o.lanes_per_run = dm.mode == kModeElements ? dm.lanes_per_run : 0;
      for (uint32_t d = 0; d < dm.ndim; ++d) {
        o.shape[d] = dm.shape[kMaxOuterDims - dm.ndim + d];
        o.stride_bytes[d] = dm.stride[kMaxOuterDims - dm.ndim + d];
      }
      if (dm.mode == kModeTranspose) {
        // all dims in packed (C) order: the batch dims with B, the dim that is
        // contiguous in the tensor, at its place among them, then A
        struct Dim { uint32_t extent; int64_t stride; uint64_t packed; };
        Dim all[kMaxOuterDims];
        uint32_t n = 0;
        for (uint32_t d = 0; d < dm.ndim; ++d) {
          const uint32_t slot = kMaxBatchDims - dm.ndim + d;
          all[n++] = {dm.shape[kMaxOuterDims - kMaxBatchDims + slot],
                      dm.stride[kMaxOuterDims - kMaxBatchDims + slot], dm.pstride[slot]};
        }
        all[n++] = {dm.ext_b, static_cast<int64_t>(dm.granule), dm.pstride_b};
        std::sort(all, all + n, [](const Dim& x, const Dim& y) { return x.packed > y.packed; });
        all[n++] = {dm.ext_a, dm.stride_a, dm.granule};
        for (uint32_t d = 0; d < n; ++d) {
          o.shape[d] = all[d].extent;
          o.stride_bytes[d] = all[d].stride;
        }
        o.ndim = n;
      }
    }
  }
  for (size_t i = 0; i < plan->host_copies.size() && out && w < capacity; ++i, ++w) {
    axr_segment_info_t& o = out[w];
    std::memset(&o, 0, sizeof(o));
    o.tensor = plan->host_copy_tensor[i];
    o.mode = 4;
    o.address = plan->host_copies[i].host;
    o.offset = plan->host_copies[i].offset;
    o.run_bytes = o.nbytes = plan->host_copies[i].bytes;
  }
  return AXR_OK;
}
int axr_plan_segments(axr_plan_t* plan, axr_segment_info_t* out, size_t capacity, size_t* count) {
  return guarded([&] { return plan_segments_body(plan, out, capacity, count); });
}

}  // extern "C"
