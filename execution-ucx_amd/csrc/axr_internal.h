// Internal declarations shared by the planner (host only), the runtime shim
// and the HIP kernels.  Nothing here is part of the C ABI.
#ifndef AXR_INTERNAL_H_
#define AXR_INTERNAL_H_

#include <stddef.h>
#include <stdint.h>

#include <atomic>
#include <new>
#include <string>
#include <vector>

#include "axon_rocm.h"

namespace axr {

// ---------------------------------------------------------------- device tables
//
// One pack or unpack is ONE kernel launch that walks a segment table resident
// in HBM.  A segment is one tensor (or one slice of a tensor with many strided
// outer dimensions); it is cut into tiles of at most kTileBytes that never
// cross a contiguous run, and tiles are numbered consecutively over the whole
// bundle.  Each wavefront owns a contiguous range of tile ids.

constexpr uint32_t kWaveLanes = 64;
constexpr uint32_t kVecBytes = 16;                           // one dwordx4 per lane
constexpr uint32_t kRowBytes = kWaveLanes * kVecBytes;       // 1 KiB per wave-wide access
constexpr uint32_t kMaxTileRows = 16;
constexpr uint32_t kMaxThreadsPerWorkgroup = 1024;
constexpr uint32_t kMaxElementThreads = 256;   // kernels that decode elements or transpose: more registers
constexpr uint32_t kXcds = 8;   // accelerator dies; workgroup i is dispatched to die i % 8
constexpr uint32_t kMaxOuterDims = 6;

constexpr uint32_t kSegPadMask = 0xfffu;         // meta bits 0..11: zero bytes after segment
constexpr uint32_t kSegDimsShift = 12;           // meta bits 12..31: 1 + dims index
constexpr uint32_t kSegFillOnly = 0xfffffu;      // dims field value: segment only writes zeros
constexpr uint32_t kSegGroup = 0xffffeu;         // dims field value: one tile that holds several short tensors
constexpr uint32_t kMaxAlign = 4096;
constexpr uint32_t kDirectSegShift = 0xffu;      // seg_shift value: every segment is exactly one tile
constexpr uint32_t kGroupBlocksShift = 0xfeu;    // seg_shift value: every tile is a group block at a fixed stride
// run_bytes of a contiguous (not strided) segment carries, in its top byte, the number
// of leading bytes (< 128) that tile 0 moves in addition to its own range: with them
// peeled off, every tile of the segment starts on a 128-byte line of the written side.
constexpr uint32_t kSegHeadShift = 56;
constexpr uint64_t kSegRunMask = (1ull << kSegHeadShift) - 1;
constexpr uint32_t kLineBytes = 128;

struct Seg {              // 32 bytes
  uint64_t ptr;           // tensor-side address of the first element
  uint64_t off;           // payload offset of the segment's first byte
  uint64_t run_bytes;     // bytes per contiguous run (whole segment when not strided)
  uint32_t tile_begin;    // id of the segment's first tile
  uint32_t meta;          // pad | (dims index + 1) << 12
};
static_assert(sizeof(Seg) == 32, "Seg layout");

// A group tile: several whole short contiguous tensors that follow each other in the bundle
// are moved by ONE wavefront.  Every group has a block of kGroupBlockBytes in the table block
// (behind the tile-block index): a GroupHead, then up to kGroupMaxMembers Member records.  The
// group's Seg carries, in `ptr`, the byte offset of that block from the start of the segment
// table.  A bundle that consists of group tiles only needs neither its Seg records nor the
// index on the device: tile t's block lies at t * kGroupBlockBytes (seg_shift ==
// kGroupBlocksShift; the kernel's `dims` argument then points at the blocks), which takes
// one dependent memory access out of every wavefront's path.
// A member of n bytes followed by `pad` zero bytes occupies max(1, ceil(n / 16)) data slots,
// then ceil(pad / 16) zero slots when pad >= 16; a slot is one 16-byte access of one lane, the
// last data (zero) slot covering the member's (gap's) final 16 bytes.  Members shorter than 16
// bytes and gaps shorter than 16 bytes move in pieces of 8, 4, 2 and 1 bytes in the lane of
// the member's last data slot.
constexpr uint32_t kGroupMaxMembers = 16;
constexpr uint32_t kGroupMaxSlots = 128;         // two 16-byte accesses per lane
constexpr uint32_t kGroupMaxMemberBytes = 1023;
struct Member {           // 16 bytes
  uint64_t ptr;           // tensor-side address
  uint32_t off_pad;       // bits 0-19: payload offset from the group's first byte; bits 20-31: pad
  uint16_t nbytes;        // 1 .. kGroupMaxMemberBytes
  uint16_t begin;         // first slot of the member
};
static_assert(sizeof(Member) == 16, "Member layout");
struct GroupHead {        // 32 bytes
  uint64_t starts[2];     // bit j of starts[r]: lane slot 64 r + j is the first slot of a member, so
                          // that a slot finds its member by counting bits instead of searching
  uint64_t off;           // payload offset of the group's first member
  uint32_t members;
  uint32_t slots;
};
static_assert(sizeof(GroupHead) == 32, "GroupHead layout");
constexpr uint32_t kGroupBlockBytes = sizeof(GroupHead) + kGroupMaxMembers * sizeof(Member);   // 288
constexpr uint32_t kMemberOffBits = 20;
constexpr uint32_t group_data_slots(uint32_t nbytes) { return nbytes >= kVecBytes ? (nbytes + kVecBytes - 1) / kVecBytes : 1u; }
constexpr uint32_t group_pad_slots(uint32_t pad) { return pad >= kVecBytes ? (pad + kVecBytes - 1) / kVecBytes : 0u; }

constexpr uint32_t kModeRunTiles = 0;   // every tile is a piece of one contiguous run
constexpr uint32_t kModeElements = 1;   // tile covers packed bytes; lanes decode granules
constexpr uint32_t kModeTranspose = 2;  // tile is a square block transposed through LDS

// Transposed blocks are T x T elements; a block row is 128 bytes (eight 16-byte
// vectors) for elements up to 4 bytes and 256 bytes for wider ones, so that a
// block is 4 to 16 KiB.  In LDS every row carries one dword of padding.
constexpr uint32_t transpose_edge(uint32_t element_bytes) {
  return (element_bytes <= 4 ? 128u : 256u) / element_bytes;   // 128, 64, 32, 32, 16
}
constexpr uint32_t transpose_lds_pitch(uint32_t element_bytes) {
  return transpose_edge(element_bytes) * element_bytes + 4u;
}
// When one of the two block dimensions is shorter than a square block's edge the
// block becomes a rectangle of about this many bytes, its long edge capped.
constexpr uint32_t kRectBlockBytes = 8192;
constexpr uint32_t kRectMaxEdge = 1024;
constexpr uint32_t kMaxBatchDims = 4;
constexpr uint32_t kMinElementTileBytes = 8192;   // element-mode work unit (measured: 8 KiB beats 2, 4 and 16)

struct Dims {             // 176 bytes, one per strided segment
  uint32_t mode;
  uint32_t ndim;          // outer (non-run) dimensions after collapsing, <= kMaxOuterDims;
                          // kModeTranspose: batch dimensions (<= kMaxBatchDims)
  uint32_t tiles_per_run; // kModeRunTiles
  uint32_t granule;       // kModeElements: bytes moved per lane access (1,2,4,8,16);
                          // kModeRunTiles: 1 + log2(tiles_per_run) when a power of two;
                          // kModeTranspose: element size
  uint64_t nbytes;        // bytes of the whole segment
  uint32_t shape[kMaxOuterDims];
  int64_t stride[kMaxOuterDims];   // bytes, outermost first, right-aligned
  // kModeTranspose: A is the innermost packed dimension (strided in the tensor), B the
  // dimension that is contiguous in the tensor; the rest are batch dimensions.
  uint64_t pstride[kMaxBatchDims]; // packed byte strides of the batch dims (aligned with shape[2..5])
  int64_t stride_a;                // tensor byte stride of A
  uint64_t pstride_b;              // packed byte stride of B
  uint32_t ext_a, ext_b;
  uint32_t tiles_a, tiles_b;
  uint32_t edge_a, edge_b;         // block extent along A and B (elements)
  uint32_t lanes_per_run;          // kModeElements: 0, or the lane slots a ragged run occupies (its
                                   // 16-byte granules rounded up to a multiple of four)
  uint32_t nt_allowed;             // kModeElements, kModeTranspose: sides that may keep the launch's
                                   // non-temporal hint when packing (bit 0 tensor, bit 1 payload) and when
                                   // unpacking (bits 2, 3).  Transposed block rows that straddle 128-byte
                                   // lines share them with the neighbouring blocks and are written through
                                   // the cache; rows shorter than a line are read and written through it
};
static_assert(sizeof(Dims) == 176, "Dims layout");

struct KernelArgs {
  const Seg* segs;            // nseg + 1 entries, last is a sentinel with tile_begin == ntiles
  const Dims* dims;
  const uint32_t* wave_seg;   // segment holding tile (k << seg_shift), for every k
  uint8_t* payload;
  uint32_t nseg;
  uint32_t ntiles;
  uint32_t tiles_per_wave;
  uint32_t xcd_remap;         // 0 or the number of workgroups per die
  uint32_t seg_shift;         // log2 of the tile-block size of wave_seg
  int64_t tensor_delta = 0;   // added to every tensor-side address of the tables
};

// One launch serving several bundles: job k owns the workgroups [wg_begin[k], wg_begin[k+1]).
constexpr uint32_t kMaxJobs = 16;   // 1 KiB of kernel arguments
struct JobDesc {              // 64 bytes
  uint64_t segs, dims, wave_seg, payload;   // device addresses
  int64_t tensor_delta;
  uint32_t ntiles, tiles_per_wave, seg_shift, wg_begin;
  uint32_t unpack;            // 0: tensors -> payload, 1: payload -> tensors
  uint32_t reserved;
};
static_assert(sizeof(JobDesc) == 64, "JobDesc layout");
constexpr uint32_t kNoJobBegin = 0x7fffffffu;        // beyond every workgroup index of a launch
constexpr uint32_t kJobTableKernargOffset = 64;      // the table follows 14 scalar arguments, 16-byte aligned
struct alignas(16) JobTable {
  uint32_t count, lds_per_wave, nt_bits;
  uint32_t interleaved;       // 1: two jobs of equal grids, job = workgroup & 1, local workgroup = workgroup >> 1
  // first workgroup of every job once more, side by side (kNoJobBegin past the last job): the kernel
  // gets the first eleven as scalar arguments as well and reads the rest here, instead of walking
  // the descriptors with a dependent load per step
  uint32_t begins[kMaxJobs];
  JobDesc job[kMaxJobs];
};

// Tables of a small bundle handed to the kernel by value.  bytes[0..16) is a head
// (a mark the kernel checks, then padding), the Seg array follows at kInlineTablesHead,
// Dims and the tile-block index at the offsets the launch passes.
constexpr uint32_t kInlineTableBytes = 3584;
constexpr uint32_t kInlineTablesHead = 16;
constexpr uint64_t kInlineTablesMark = 0x31454c4254525841ull;   // "AXRTBLE1"
struct alignas(16) InlineTables {
  uint8_t bytes[kInlineTableBytes];
};

struct LaunchConfig {
  uint32_t workgroups = 0;
  uint32_t tiles_per_wave = 0;
  uint32_t tile_rows = 2;
  uint32_t threads = 128;   // per workgroup, a multiple of 64
  uint32_t seg_shift = 0;   // wave_seg has one entry per 2^seg_shift tiles
  uint32_t nontemporal = 3;   // bit 0: tensor-side accesses, bit 1: payload-side accesses
  bool elements = false;   // some segment uses kModeElements or kModeTranspose
  uint32_t lds_per_wave = 0;   // bytes of LDS each wavefront needs (transposed tiles only)
  bool xcd_remap = false;  // give each die a contiguous share of the wave index space
};

// ---------------------------------------------------------------- tunables

// Read by planning threads while axr_tune_set may write: every knob is an atomic.
struct Tunables {
  // Tile = tile_rows KiB moved by one wavefront.  0 picks the smallest of
  // 2, 4, 8, 16 that keeps the bundle within max_tiles tiles (and one tile per
  // run for bundles of short strided runs): small tiles and a grid of one tile
  // per wave measured fastest on MI355X (the hardware dispatcher balances the
  // load); larger tiles only bound the grid for multi-GiB bundles.
  std::atomic<int64_t> tile_rows{0};
  std::atomic<int64_t> max_tiles{1 << 20};
  std::atomic<int64_t> max_waves{1 << 20};    // beyond this many tiles a wave takes several
  std::atomic<int64_t> threads{0};            // workgroup size; 0 = 256 below 65,536 tiles (fewer dispatches
                                  // for short kernels), 128 above (finer balance at the tail)
  // Non-temporal hint: bit 0 tensor-side accesses, bit 1 payload-side accesses;
  // -1 = automatic: tensors always stream (read or written once), the payload
  // streams only when it is larger than payload_cache_bytes.  A smaller payload
  // is written with ordinary stores so that it is still in the 256 MB
  // last-level cache when the consumer (unpack, or the transport's copy) reads it.
  std::atomic<int64_t> nontemporal{-1};
  std::atomic<int64_t> payload_cache_bytes{256ll << 20};
  // Strided runs shorter than this use element mode when they are 16 bytes or
  // longer (16-byte granules, exact or ragged), anything else up to a fifth of it
  // (measured crossovers).
  std::atomic<int64_t> gather_run_bytes{1280};
  std::atomic<int64_t> xcd_remap{-1};         // contiguous wave ranges per die: 1 always, 0 never, -1 when
                                  // transposed blocks that share lines with their neighbours dominate
  std::atomic<int64_t> transpose{1};          // move transposed views as square blocks through LDS
  std::atomic<int64_t> ragged_runs{1};        // short runs of 16+ bytes that are no multiple of 16 move in
                                  // 16-byte granules (the last one overlapping) instead of narrower ones
  // Contiguous segments longer than a tile start their tiles on a multiple of this many
  // bytes of the written side (0: tiles start at the segment's first byte).  Measured on the
  // 4096-tensor bundle: 16 lifts the tight layout by 2 % (every 16-byte store aligned) and
  // costs the 256-byte aligned layout nothing; 64 and 128 are no better for either.
  std::atomic<int64_t> head_align{16};
  // The loopback transport moves a device payload to device memory of the same GPU with the
  // library's copy kernel (1) or with hipMemcpyAsync (0).
  std::atomic<int64_t> loopback_copy_kernel{1};
  // Bundles of at least this many tensors, all of them contiguous device tensors, get their
  // tables in one pass over the tensors into pinned memory plus a kernel that brings them to
  // the device and writes the tile-block index (0: the general host path always).
  std::atomic<int64_t> device_tables{512};
  // axr_stream_synchronize may first poll, for up to this many microseconds, a word of pinned
  // memory that a one-wave kernel enqueued behind the stream's work writes, before it falls
  // back to the runtime's wait (0, the default: the runtime's wait only).  See the header.
  std::atomic<int64_t> spin_wait_us{0};
  std::atomic<int64_t> host_threads{4};       // threads (the caller included) for host-side staging copies
  // Contiguous device tensors of at most this many bytes that follow each other in a bundle
  // share wavefronts (group tiles, up to 64 tensors or 2 KiB of lane slots each); 0: every
  // tensor gets its own wavefronts.
  std::atomic<int64_t> group_bytes{512};
  std::atomic<int64_t> group_slots{kGroupMaxSlots};   // lane slots per group tile: 64 or 128
  // The two jobs of an axr_submit launch whose grids are equal and whose payloads are larger than
  // payload_cache_bytes take the workgroups in turn (even / odd) instead of one range each (1, the
  // default; 0: never; 2: also smaller payloads that were asked to stream).  With a pack and an
  // unpack in one launch the memory then sees reads and writes of both throughout: the 405 MB
  // layer bundle 6.50 -> 6.65 TB/s.  Smaller payloads are better off with the pack's range first,
  // cached (48 MB mixed bundle: 6.18 against 6.11 TB/s) or streaming (5.78 against 5.51).
  std::atomic<int64_t> submit_interleave{1};
  // Failure injection for tests of the streamed transfer's error handling: N > 0 makes the
  // N-th chunk submitted from now on fail after its send has been queued, as if the message
  // that arrived did not match the receiver's plan (and counts down to 0 = off).
  std::atomic<int64_t> transfer_fail_after_send{0};
  std::atomic<int64_t> inline_tables{16384};  // bundles of up to this many tiles whose tables fit the kernel
                                  // arguments are launched without a table upload; 0: never
};
Tunables& tunables();

// ---------------------------------------------------------------- errors

int fail(int status, const std::string& message);   // records thread-local message
int check_hip(int hip_error, const char* what);     // 0 or AXR_ERR_HIP
// Host-side copies of the staging paths (pageable memory <-> pinned blocks).  One core
// moves about 25 GB/s, less than the PCIe link; jobs of 2 MiB and more in total are cut
// into byte-balanced shares for up to `host_threads` short-lived threads.
struct HostCopyJob {
  void* dst;
  const void* src;
  size_t bytes;
};
void host_copy(const HostCopyJob* jobs, size_t count);

// True for a handle that axr_stream_destroy has destroyed (and no later
// axr_stream_create has returned again).
bool stream_retired(void* stream);
// Launch marks order what the library enqueues, process-wide.  A launch takes a mark after
// it has been enqueued; a wait reads the current mark before it starts, and once it has seen
// the stream drain, every launch on that stream with a mark up to that value is known to be
// finished, so that a plan released next need not wait for the stream again.
uint64_t stream_mark_launch();
uint64_t stream_launch_mark();
void stream_note_drained(void* stream, uint64_t mark);
bool stream_drained(void* stream, uint64_t mark);
void stream_forget(void* stream);   // the stream is being destroyed
// A kernel that writes device-visible HOST memory has been enqueued on `stream`: the next
// axr_stream_synchronize of that stream must be the runtime's wait (which makes such writes
// visible to the CPU), not the polled one.  take: true once per note, then forgotten.
void stream_note_host_writes(void* stream);
bool stream_take_host_writes(void* stream);
int fail_nothrow(int status, const char* message) noexcept;

// Every extern "C" entry point runs its body through this: no C++ exception
// (std::bad_alloc from a container, in practice) crosses the C boundary.
template <typename Body>
int guarded(Body&& body) noexcept {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return fail_nothrow(AXR_ERR_NOMEM, "out of host memory");
  } catch (...) {
    return fail_nothrow(AXR_ERR_INVALID, "unexpected C++ exception");
  }
}

// ---------------------------------------------------------------- kernels (axr_kernels.hip)

int launch_bundle_kernel(bool pack, const KernelArgs& args, const LaunchConfig& cfg,
                         void* stream);
// Same launch with the tables inside the kernel arguments (default geometry only:
// 2 KiB tiles, tensor side streaming, payload side cacheable, no die remapping).
int launch_bundle_kernel_inline(bool pack, const KernelArgs& args, const LaunchConfig& cfg,
                                const InlineTables& tables, uint32_t dims_at, uint32_t wave_at,
                                void* stream);
// One launch for up to kMaxJobs bundles that share `cfg` (tile size, workgroup size, cache
// hints; cfg.workgroups is the whole grid, cfg.lds_per_wave the largest need of any job).
int launch_bundle_jobs(const JobTable& jobs, const LaunchConfig& cfg, void* stream);
int launch_fill(void* dst, int value, size_t bytes, void* stream);
// Enqueues a one-wave kernel that stores `value` into *flag (pinned host memory).
int launch_notify(uint32_t* flag, uint32_t value, void* stream);
// staged: n + 1 segment records in device-accessible memory (pinned host memory will do);
// segs and wave_seg are device memory.  Copies the records and writes the tile-block index.
int launch_expand_tables(const Seg* staged, uint32_t n, Seg* segs, uint32_t* wave_seg, uint32_t seg_shift,
                         void* stream);
// dst[0, bytes) = src[0, bytes), both in device memory of the current device, no alignment needed.
int launch_stream_copy(void* dst, const void* src, size_t bytes, bool nontemporal, void* stream);
// Device address, on the current device, of the kStaticTableBytes bytes that hold the
// tables of axr_pack_noalloc (a __device__ array of the code object: never allocated,
// shared by every call on that device).
constexpr size_t kStaticTableBytes = 1u << 20;
int static_table_area(void** ptr);

// ---------------------------------------------------------------- runtime (axr_runtime.cpp)

int device_compute_units(int* cus);
// Cached pinned-host + device block pair used for plan tables.
struct TableBlock {
  void* host = nullptr;
  void* device = nullptr;
  size_t bytes = 0;
  int device_id = -1;
};
int table_block_acquire(size_t bytes, TableBlock* block);
void table_block_release(TableBlock* block);
// Events without timing for the current device, recycled: creating one costs more than a
// microsecond, and every fresh plan that uploads tables needs one.  An event goes back
// only once it has fired (or was never recorded).
int event_acquire(void** event, int* device);
void event_release(void* event, int device);

}  // namespace axr

#endif  // AXR_INTERNAL_H_
