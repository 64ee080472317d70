// Runtime shim: device selection, streams, events, copies and the slab pool.
// This file (with axr_kernels.hip) is the only place that includes HIP
// headers; host code above the C ABI never does.
#include <hip/hip_runtime_api.h>

#include <chrono>

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

#include "axr_internal.h"

namespace axr {

namespace {
thread_local std::string g_last_error;
}

int fail(int status, const std::string& message) {
  g_last_error = message;
  return status;
}

int fail_nothrow(int status, const char* message) noexcept {
  try {
    g_last_error = message;
  } catch (...) {
    g_last_error.clear();
  }
  return status;
}

int check_hip(int hip_error, const char* what) {
  if (hip_error == hipSuccess) return AXR_OK;
  const hipError_t e = static_cast<hipError_t>(hip_error);
  std::string msg = std::string(what) + ": " + hipGetErrorName(e) + " (" +
                    hipGetErrorString(e) + ")";
  if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) return fail(AXR_ERR_NO_DEVICE, msg);
  if (e == hipErrorOutOfMemory) return fail(AXR_ERR_NOMEM, msg);
  return fail(AXR_ERR_HIP, msg);
}

Tunables& tunables() {
  static Tunables t;
  return t;
}

int device_compute_units(int* cus) {
  static std::mutex mu;
  static std::map<int, int> cache;
  int dev = 0;
  int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(dev);
  if (it == cache.end()) {
    int n = 0;
    rc = check_hip(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev),
                   "hipDeviceGetAttribute");
    if (rc) return rc;
    it = cache.emplace(dev, n).first;
  }
  *cus = it->second;
  return AXR_OK;
}

// ------------------------------------------------------------ table blocks
//
// Plan tables are staged in pinned host memory and copied to a device block
// with one async copy.  Both halves are recycled through a size-bucketed
// free list so that steady-state planning performs no driver allocation.  The
// list keeps at most kTableCacheBytes per half; what is released beyond that
// goes back to the driver, so a burst of thousands of live plans does not pin
// its peak forever.

namespace {
constexpr size_t kTableCacheBytes = 256u << 20;
struct TableCache {
  std::mutex mu;
  std::multimap<std::pair<int, size_t>, TableBlock> free_blocks;
  size_t cached_bytes = 0;
};
TableCache& table_cache() {
  static TableCache* c = new TableCache();   // leaked on purpose: outlives static dtors
  return *c;
}
size_t bucket_bytes(size_t bytes) {
  size_t b = 4096;
  while (b < bytes) b <<= 1;
  return b;
}
}  // namespace

namespace {
std::mutex g_event_mutex;
std::unordered_map<int, std::vector<hipEvent_t>> g_idle_events;   // per device
constexpr size_t kMaxIdleEvents = 64;
}  // namespace

int event_acquire(void** event, int* device) {
  int dev = -1;
  int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc) return rc;
  {
    std::lock_guard<std::mutex> lock(g_event_mutex);
    std::vector<hipEvent_t>& idle = g_idle_events[dev];
    if (!idle.empty()) {
      *event = idle.back();
      *device = dev;
      idle.pop_back();
      return AXR_OK;
    }
  }
  hipEvent_t e = nullptr;
  rc = check_hip(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
  if (rc) return rc;
  *event = e;
  *device = dev;
  return AXR_OK;
}

void event_release(void* event, int device) {
  if (!event) return;
  {
    std::lock_guard<std::mutex> lock(g_event_mutex);
    std::vector<hipEvent_t>& idle = g_idle_events[device];
    if (idle.size() < kMaxIdleEvents) {
      idle.push_back(static_cast<hipEvent_t>(event));
      return;
    }
  }
  (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}

int table_block_acquire(size_t bytes, TableBlock* block) {
  int dev = 0;
  int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc) return rc;
  const size_t want = bucket_bytes(bytes);
  TableCache& c = table_cache();
  {
    std::lock_guard<std::mutex> lock(c.mu);
    auto it = c.free_blocks.find({dev, want});
    if (it != c.free_blocks.end()) {
      *block = it->second;
      c.free_blocks.erase(it);
      c.cached_bytes -= want;
      return AXR_OK;
    }
  }
  TableBlock b;
  b.bytes = want;
  b.device_id = dev;
  rc = check_hip(hipHostMalloc(&b.host, want, hipHostMallocDefault), "hipHostMalloc(table)");
  if (rc) return rc;
  rc = check_hip(hipMalloc(&b.device, want), "hipMalloc(table)");
  if (rc) {
    (void)hipHostFree(b.host);
    return rc;
  }
  *block = b;
  return AXR_OK;
}

void table_block_release(TableBlock* block) {
  if (!block->host) return;
  TableCache& c = table_cache();
  {
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.cached_bytes + block->bytes <= kTableCacheBytes) {
      c.free_blocks.emplace(std::make_pair(block->device_id, block->bytes), *block);
      c.cached_bytes += block->bytes;
      *block = TableBlock();
      return;
    }
  }
  // callers release a block only when nothing on the device reads it any more
  (void)hipHostFree(block->host);
  (void)hipFree(block->device);
  *block = TableBlock();
}

}  // namespace axr

namespace axr {
namespace {
// Bytes [begin, end) of the concatenation of all jobs.
void copy_share(const HostCopyJob* jobs, size_t count, size_t begin, size_t end) {
  size_t at = 0;
  for (size_t i = 0; i < count && at < end; ++i) {
    const size_t n = jobs[i].bytes;
    if (at + n > begin) {
      const size_t lo = begin > at ? begin - at : 0;
      const size_t hi = end - at < n ? end - at : n;
      std::memcpy(static_cast<uint8_t*>(jobs[i].dst) + lo,
                  static_cast<const uint8_t*>(jobs[i].src) + lo, hi - lo);
    }
    at += n;
  }
}
}  // namespace

void host_copy(const HostCopyJob* jobs, size_t count) {
  size_t total = 0;
  for (size_t i = 0; i < count; ++i) total += jobs[i].bytes;
  size_t shares = static_cast<size_t>(tunables().host_threads);
  if (shares > total / (1u << 20)) shares = total / (1u << 20);   // a MiB per thread at least
  if (shares < 2) {
    copy_share(jobs, count, 0, total);
    return;
  }
  const size_t share = (total / shares + 63) & ~static_cast<size_t>(63);
  std::vector<std::thread> helpers;
  size_t begin = share;   // the caller takes the first share
  try {
    helpers.reserve(shares - 1);
    for (; begin < total; begin += share) {
      const size_t end = begin + share < total ? begin + share : total;
      helpers.emplace_back(copy_share, jobs, count, begin, end);
    }
  } catch (...) {
    // no more threads to be had: whatever was not handed out is copied here
  }
  copy_share(jobs, count, 0, share < total ? share : total);
  if (begin < total) copy_share(jobs, count, begin, total);
  for (std::thread& t : helpers) t.join();
}
}  // namespace axr

// Streams made by axr_stream_create, and the handles of those destroyed since.
// A plan remembers the streams it ran on and drains them before its tables go
// away; a handle whose stream is gone must not reach HIP again.
namespace {
std::mutex g_stream_mutex;
std::unordered_set<void*> g_retired_streams;
}  // namespace

namespace axr {
namespace {
std::atomic<uint64_t> g_launch_mark{0};
std::mutex g_drained_mutex;
std::unordered_map<void*, uint64_t> g_drained;   // stream -> highest mark seen drained
std::unordered_set<void*> g_host_writes;         // streams whose queued kernels write host memory
}  // namespace
uint64_t stream_mark_launch() { return g_launch_mark.fetch_add(1, std::memory_order_seq_cst) + 1; }
uint64_t stream_launch_mark() { return g_launch_mark.load(std::memory_order_seq_cst); }
void stream_note_drained(void* stream, uint64_t mark) {
  std::lock_guard<std::mutex> lock(g_drained_mutex);
  uint64_t& seen = g_drained[stream];
  if (mark > seen) seen = mark;
}
bool stream_drained(void* stream, uint64_t mark) {
  std::lock_guard<std::mutex> lock(g_drained_mutex);
  auto it = g_drained.find(stream);
  return it != g_drained.end() && it->second >= mark;
}
void stream_forget(void* stream) {
  std::lock_guard<std::mutex> lock(g_drained_mutex);
  g_drained.erase(stream);
  g_host_writes.erase(stream);
}
void stream_note_host_writes(void* stream) {
  std::lock_guard<std::mutex> lock(g_drained_mutex);
  g_host_writes.insert(stream);
}
bool stream_take_host_writes(void* stream) {
  std::lock_guard<std::mutex> lock(g_drained_mutex);
  return g_host_writes.erase(stream) != 0;
}
}  // namespace axr

namespace axr {
bool stream_retired(void* stream) {
  std::lock_guard<std::mutex> lock(g_stream_mutex);
  return g_retired_streams.count(stream) != 0;
}
}  // namespace axr

using namespace axr;

// ================================================================ slab pool

struct axr_pool {
  struct Slab {
    char* base = nullptr;
    size_t bytes = 0;
    void* mem_h = nullptr;
    size_t live = 0;   // blocks handed out from this slab
  };
  int device = 0;
  size_t slab_bytes = 0;
  std::mutex mu;
  std::map<char*, Slab> slabs;                 // by base address
  std::map<char*, size_t> free_by_addr;        // free block -> size
  std::set<std::pair<size_t, char*>> free_by_size;
  std::unordered_map<void*, std::pair<char*, size_t>> live;   // user ptr -> (block, size)
  axr_register_fn reg = nullptr;
  axr_unregister_fn unreg = nullptr;
  void* user = nullptr;
  uint64_t allocated = 0, peak = 0;

  static constexpr size_t kGranule = 256;

  void add_free(char* p, size_t n) {
    // coalesce with the neighbours that lie in the same slab
    auto next = free_by_addr.lower_bound(p);
    if (next != free_by_addr.end() && p + n == next->first && same_slab(p, next->first)) {
      n += next->second;
      free_by_size.erase({next->second, next->first});
      next = free_by_addr.erase(next);
    }
    if (next != free_by_addr.begin()) {
      auto prev = std::prev(next);
      if (prev->first + prev->second == p && same_slab(prev->first, p)) {
        p = prev->first;
        n += prev->second;
        free_by_size.erase({prev->second, prev->first});
        free_by_addr.erase(prev);
      }
    }
    free_by_addr[p] = n;
    free_by_size.insert({n, p});
  }
  Slab* slab_of(char* p) {
    auto it = slabs.upper_bound(p);
    if (it == slabs.begin()) return nullptr;
    --it;
    return (p < it->second.base + it->second.bytes) ? &it->second : nullptr;
  }
  bool same_slab(char* a, char* b) { return slab_of(a) == slab_of(b); }
};

namespace {

struct DeviceGuard {
  int prev = -1;
  bool switched = false;
  int enter(int device) {
    int rc = check_hip(hipGetDevice(&prev), "hipGetDevice");
    if (rc) return rc;
    if (prev != device) {
      rc = check_hip(hipSetDevice(device), "hipSetDevice");
      if (rc) return rc;
      switched = true;
    }
    return AXR_OK;
  }
  ~DeviceGuard() {
    if (switched) (void)hipSetDevice(prev);
  }
};

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int pool_grow(axr_pool* pool, size_t need) {
  size_t bytes = pool->slab_bytes > need ? pool->slab_bytes : round_up(need, 2u << 20);
  DeviceGuard guard;
  int rc = guard.enter(pool->device);
  if (rc) return rc;
  void* base = nullptr;
  rc = check_hip(hipMalloc(&base, bytes), "hipMalloc(slab)");
  if (rc) return rc;
  axr_pool::Slab slab;
  slab.base = static_cast<char*>(base);
  slab.bytes = bytes;
  if (pool->reg) {
    const int rr = pool->reg(pool->user, base, bytes, &slab.mem_h);
    if (rr != 0) {
      (void)hipFree(base);
      return fail(AXR_ERR_HIP, "slab registration callback failed with " + std::to_string(rr));
    }
  }
  pool->slabs[slab.base] = slab;
  pool->add_free(slab.base, bytes);
  return AXR_OK;
}

void pool_release_slab(axr_pool* pool, axr_pool::Slab& slab) {
  if (slab.mem_h && pool->unreg) pool->unreg(pool->user, slab.mem_h);
  (void)hipFree(slab.base);
}

std::mutex g_default_pool_mu;
std::map<int, axr_pool*> g_default_pools;

}  // namespace

extern "C" {

// ---------------------------------------------------------------- status

const char* axr_status_string(int status) {
  switch (status) {
    case AXR_OK: return "AXR_OK";
    case AXR_ERR_INVALID: return "AXR_ERR_INVALID";
    case AXR_ERR_NOMEM: return "AXR_ERR_NOMEM";
    case AXR_ERR_HIP: return "AXR_ERR_HIP";
    case AXR_ERR_LENGTH: return "AXR_ERR_LENGTH";
    case AXR_ERR_UNSUPPORTED: return "AXR_ERR_UNSUPPORTED";
    case AXR_ERR_NO_MESSAGE: return "AXR_ERR_NO_MESSAGE";
    case AXR_ERR_NOT_IMPLEMENTED: return "AXR_ERR_NOT_IMPLEMENTED";
    case AXR_ERR_HEADER: return "AXR_ERR_HEADER";
    case AXR_ERR_MISMATCH: return "AXR_ERR_MISMATCH";
    case AXR_ERR_NO_DEVICE: return "AXR_ERR_NO_DEVICE";
    case AXR_ERR_BUSY: return "AXR_ERR_BUSY";
    case AXR_ERR_CANCELED: return "AXR_ERR_CANCELED";
    default: return "AXR_ERR_?";
  }
}

const char* axr_last_error(void) { return g_last_error.c_str(); }

const char* axr_version(void) { return "0.1.0"; }

static int dl_device_to_memory_type_body(int32_t t) {
  switch (t) {
    case 2: return AXR_MEM_CUDA;
    case 13: return AXR_MEM_CUDA_MANAGED;
    case 10: return AXR_MEM_ROCM;
    case 11: return AXR_MEM_ROCM_MANAGED;
    case 1: return AXR_MEM_HOST;
    default: return AXR_MEM_UNKNOWN;
  }
}
int axr_dl_device_to_memory_type(int32_t t) {
  return guarded([&] { return dl_device_to_memory_type_body(t); });
}

int32_t axr_memory_type_to_dl_device(int m) {
  switch (m) {
    case AXR_MEM_CUDA: return 2;
    case AXR_MEM_CUDA_MANAGED: return 13;
    case AXR_MEM_ROCM: return 10;
    case AXR_MEM_ROCM_MANAGED: return 11;
    case AXR_MEM_ZE_HOST:
    case AXR_MEM_ZE_DEVICE:
    case AXR_MEM_ZE_MANAGED: return 14;
    default: return 1;   // HOST, RDMA, UNKNOWN
  }
}

static int tune_set_body(const char* key, int64_t value) {
  if (!key) return fail(AXR_ERR_INVALID, "axr_tune_set: null key");
  Tunables& t = tunables();
  const std::string k(key);
  if (k == "tile_rows") {
    if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8 && value != 16)
      return fail(AXR_ERR_INVALID, "tile_rows must be 0 (auto), 1, 2, 4, 8 or 16");
    t.tile_rows = value;
  } else if (k == "max_tiles") {
    if (value < 1) return fail(AXR_ERR_INVALID, "max_tiles must be positive");
    t.max_tiles = value;
  } else if (k == "max_waves") {
    if (value < 1 || value > (1ll << 30)) return fail(AXR_ERR_INVALID, "max_waves must be in [1, 2^30]");
    t.max_waves = value;
  } else if (k == "nontemporal") {
    if (value < -1 || value > 3) return fail(AXR_ERR_INVALID, "nontemporal must be -1 (auto) or 0..3");
    t.nontemporal = value;
  } else if (k == "payload_cache_bytes") {
    if (value < 0) return fail(AXR_ERR_INVALID, "payload_cache_bytes must not be negative");
    t.payload_cache_bytes = value;
  } else if (k == "gather_run_bytes") {
    if (value < 1 || value > (1 << 20))
      return fail(AXR_ERR_INVALID, "gather_run_bytes must be in [1, 2^20]");
    t.gather_run_bytes = value;
  } else if (k == "threads") {
    if (value != 0 && (value < 64 || value > 1024 || value % 64))
      return fail(AXR_ERR_INVALID, "threads must be 0 (auto) or a multiple of 64 in [64, 1024]");
    t.threads = value;
  } else if (k == "xcd_remap") {
    t.xcd_remap = value < 0 ? -1 : (value ? 1 : 0);
  } else if (k == "ragged_runs") {
    t.ragged_runs = value ? 1 : 0;
  } else if (k == "spin_wait_us") {
    if (value < 0 || value > 1000000) return fail(AXR_ERR_INVALID, "spin_wait_us must be in [0, 1000000]");
    t.spin_wait_us = value;
  } else if (k == "host_threads") {
    if (value < 1 || value > 64) return fail(AXR_ERR_INVALID, "host_threads must be in [1, 64]");
    t.host_threads = value;
  } else if (k == "inline_tables") {
    if (value < 0 || value > (1 << 30)) return fail(AXR_ERR_INVALID, "inline_tables must be in [0, 2^30]");
    t.inline_tables = value;
  } else if (k == "transpose") {
    t.transpose = value ? 1 : 0;
  } else if (k == "group_bytes") {
    if (value < 0 || value > static_cast<int64_t>(kGroupMaxMemberBytes))
      return fail(AXR_ERR_INVALID, "group_bytes must be in [0, 1023]");
    t.group_bytes = value;
  } else if (k == "transfer_fail_after_send") {
    if (value < 0) return fail(AXR_ERR_INVALID, "transfer_fail_after_send must not be negative");
    t.transfer_fail_after_send = value;
  } else if (k == "submit_interleave") {
    t.submit_interleave = value;
  } else if (k == "group_slots") {
    if (value != 64 && value != 128) return fail(AXR_ERR_INVALID, "group_slots must be 64 or 128");
    t.group_slots = value;
  } else if (k == "device_tables") {
    if (value < 0) return fail(AXR_ERR_INVALID, "device_tables must not be negative");
    t.device_tables = value;
  } else if (k == "loopback_copy_kernel") {
    t.loopback_copy_kernel = value ? 1 : 0;
  } else if (k == "head_align") {
    if (value < 0 || value > 128 || (value & (value - 1)))
      return fail(AXR_ERR_INVALID, "head_align must be 0 or a power of two up to 128");
    t.head_align = value;
  } else {
    return fail(AXR_ERR_INVALID, "unknown tunable: " + k);
  }
  return AXR_OK;
}
int axr_tune_set(const char* key, int64_t value) {
  return guarded([&] { return tune_set_body(key, value); });
}

static int tune_get_body(const char* key, int64_t* value) {
  if (!key || !value) return fail(AXR_ERR_INVALID, "axr_tune_get: null argument");
  const Tunables& t = tunables();
  const std::string k(key);
  if (k == "tile_rows") *value = t.tile_rows;
  else if (k == "max_tiles") *value = t.max_tiles;
  else if (k == "max_waves") *value = t.max_waves;
  else if (k == "nontemporal") *value = t.nontemporal;
  else if (k == "payload_cache_bytes") *value = t.payload_cache_bytes;
  else if (k == "gather_run_bytes") *value = t.gather_run_bytes;
  else if (k == "threads") *value = t.threads;
  else if (k == "xcd_remap") *value = t.xcd_remap;
  else if (k == "transpose") *value = t.transpose;
  else if (k == "ragged_runs") *value = t.ragged_runs;
  else if (k == "inline_tables") *value = t.inline_tables;
  else if (k == "host_threads") *value = t.host_threads;
  else if (k == "spin_wait_us") *value = t.spin_wait_us;
  else if (k == "head_align") *value = t.head_align;
  else if (k == "loopback_copy_kernel") *value = t.loopback_copy_kernel;
  else if (k == "device_tables") *value = t.device_tables;
  else if (k == "group_bytes") *value = t.group_bytes;
  else if (k == "group_slots") *value = t.group_slots;
  else if (k == "submit_interleave") *value = t.submit_interleave;
  else if (k == "transfer_fail_after_send") *value = t.transfer_fail_after_send;
  else return fail(AXR_ERR_INVALID, "unknown tunable: " + k);
  return AXR_OK;
}
int axr_tune_get(const char* key, int64_t* value) {
  return guarded([&] { return tune_get_body(key, value); });
}

// ---------------------------------------------------------------- device

static int device_count_body(int* count) {
  if (!count) return fail(AXR_ERR_INVALID, "axr_device_count: null result");
  *count = 0;
  const hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) {
    *count = 0;
    return AXR_OK;
  }
  return check_hip(e, "hipGetDeviceCount");
}
int axr_device_count(int* count) {
  return guarded([&] { return device_count_body(count); });
}

static int device_get_body(int* device) {
  if (!device) return fail(AXR_ERR_INVALID, "axr_device_get: null result");
  return check_hip(hipGetDevice(device), "hipGetDevice");
}
int axr_device_get(int* device) {
  return guarded([&] { return device_get_body(device); });
}

static int device_set_body(int device) {
  return check_hip(hipSetDevice(device), "hipSetDevice");
}
int axr_device_set(int device) {
  return guarded([&] { return device_set_body(device); });
}

static int device_push_body(int device, int* token) {
  if (!token) return fail(AXR_ERR_INVALID, "axr_device_push: null token");
  int prev = 0;
  int rc = check_hip(hipGetDevice(&prev), "hipGetDevice");
  if (rc) return rc;
  rc = check_hip(hipSetDevice(device), "hipSetDevice");
  if (rc) return rc;
  *token = prev;
  return AXR_OK;
}
int axr_device_push(int device, int* token) {
  return guarded([&] { return device_push_body(device, token); });
}

static int device_pop_body(int token) {
  return check_hip(hipSetDevice(token), "hipSetDevice");
}
int axr_device_pop(int token) {
  return guarded([&] { return device_pop_body(token); });
}

static int device_synchronize_body() {
  return check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
}
int axr_device_synchronize(void) {
  return guarded([&] { return device_synchronize_body(); });
}

static int device_info_body(int* compute_units, uint64_t* total_mem, uint64_t* free_mem) {
  if (compute_units) {
    int rc = device_compute_units(compute_units);
    if (rc) return rc;
  }
  if (total_mem || free_mem) {
    size_t f = 0, t = 0;
    int rc = check_hip(hipMemGetInfo(&f, &t), "hipMemGetInfo");
    if (rc) return rc;
    if (total_mem) *total_mem = t;
    if (free_mem) *free_mem = f;
  }
  return AXR_OK;
}
int axr_device_info(int* compute_units, uint64_t* total_mem, uint64_t* free_mem) {
  return guarded([&] { return device_info_body(compute_units, total_mem, free_mem); });
}

static int stream_create_body(void** stream) {
  if (!stream) return fail(AXR_ERR_INVALID, "axr_stream_create: null result");
  hipStream_t s = nullptr;
  // Default priority on purpose; non-blocking so it does not serialise with the null stream.
  int rc = check_hip(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
  if (rc) return rc;
  {
    std::lock_guard<std::mutex> lock(g_stream_mutex);
    g_retired_streams.erase(s);   // the runtime hands addresses out again
  }
  *stream = s;
  return AXR_OK;
}
int axr_stream_create(void** stream) {
  return guarded([&] { return stream_create_body(stream); });
}

static int stream_destroy_body(void* stream) {
  if (!stream) return AXR_OK;
  {
    std::lock_guard<std::mutex> lock(g_stream_mutex);
    g_retired_streams.insert(stream);
  }
  stream_forget(stream);
  return check_hip(hipStreamDestroy(static_cast<hipStream_t>(stream)), "hipStreamDestroy");
}
int axr_stream_destroy(void* stream) {
  return guarded([&] { return stream_destroy_body(stream); });
}


namespace {
// Words of pinned host memory, per device, that notify kernels write and waiting threads
// poll ("spin_wait_us").  Each wait takes the next word in turn and a value of its own;
// should two waits ever share a word (more than kNotifySlots under way at once), the loser
// merely runs out of time and falls back to the runtime's wait.
constexpr int kNotifyDevices = 64;
constexpr uint32_t kNotifySlots = 256;
constexpr uint32_t kNotifyStride = 16;   // words: one 64-byte line per slot
std::atomic<uint32_t*> g_notify_words[kNotifyDevices];
std::atomic<uint32_t> g_notify_ticket{0};

uint32_t* notify_words(int device) {
  if (device < 0 || device >= kNotifyDevices) return nullptr;
  uint32_t* words = g_notify_words[device].load(std::memory_order_acquire);
  if (words) return words;
  void* fresh = nullptr;
  if (hipHostMalloc(&fresh, kNotifySlots * kNotifyStride * sizeof(uint32_t), hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::memset(fresh, 0, kNotifySlots * kNotifyStride * sizeof(uint32_t));
  uint32_t* expected = nullptr;
  if (!g_notify_words[device].compare_exchange_strong(expected, static_cast<uint32_t*>(fresh),
                                                      std::memory_order_acq_rel)) {
    (void)hipHostFree(fresh);   // another thread was first
    return expected;
  }
  return static_cast<uint32_t*>(fresh);   // kept until the process ends
}

// True when the stream was seen to reach its end by polling; false: the caller waits through
// the runtime (capturing stream, no pinned memory, launch refused, time budget spent).
bool spin_until_stream_end(hipStream_t stream, int64_t budget_us) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (status != hipStreamCaptureStatusNone) return false;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  uint32_t* words = notify_words(device);
  if (!words) return false;
  const uint32_t ticket = g_notify_ticket.fetch_add(1, std::memory_order_relaxed) + 1;
  volatile uint32_t* word = words + (ticket % kNotifySlots) * kNotifyStride;
  const uint32_t value = ticket | 0x80000000u;   // never the zero the words start with
  if (launch_notify(const_cast<uint32_t*>(word), value, stream) != AXR_OK) return false;
  const auto deadline = std::chrono::steady_clock::now() + std::chrono::microseconds(budget_us);
  for (;;) {
    for (int i = 0; i < 64; ++i) {
      if (*word == value) {
        std::atomic_thread_fence(std::memory_order_acquire);
        return true;
      }
      __builtin_ia32_pause();
    }
    if (std::chrono::steady_clock::now() >= deadline) return false;
  }
}
}  // namespace

static int stream_synchronize_body(void* stream) {
  const uint64_t reached = stream_launch_mark();
  // A kernel's writes to host memory become visible to the CPU with the completion the runtime
  // waits for, which the polled wait returns ahead of: a stream that has scattered into
  // device-visible host tensors since its last wait takes the runtime's wait.
  const bool host_writes = stream_take_host_writes(stream);
  const int64_t budget = host_writes ? 0 : tunables().spin_wait_us.load();
  if (!(budget > 0 && spin_until_stream_end(static_cast<hipStream_t>(stream), budget))) {
    int rc = check_hip(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
    if (rc) return rc;
  }
  stream_note_drained(stream, reached);   // plans released next need not wait for this stream again
  return AXR_OK;
}
int axr_stream_synchronize(void* stream) {
  return guarded([&] { return stream_synchronize_body(stream); });
}

static int stream_wait_event_body(void* stream, void* event) {
  if (!event) return fail(AXR_ERR_INVALID, "axr_stream_wait_event: null event");
  return check_hip(hipStreamWaitEvent(static_cast<hipStream_t>(stream),
                                      static_cast<hipEvent_t>(event), 0),
                   "hipStreamWaitEvent");
}
int axr_stream_wait_event(void* stream, void* event) {
  return guarded([&] { return stream_wait_event_body(stream, event); });
}

static int event_create_body(void** event) {
  if (!event) return fail(AXR_ERR_INVALID, "axr_event_create: null result");
  hipEvent_t e = nullptr;
  int rc = check_hip(hipEventCreate(&e), "hipEventCreate");
  if (rc) return rc;
  *event = e;
  return AXR_OK;
}
int axr_event_create(void** event) {
  return guarded([&] { return event_create_body(event); });
}

static int event_destroy_body(void* event) {
  if (!event) return AXR_OK;
  return check_hip(hipEventDestroy(static_cast<hipEvent_t>(event)), "hipEventDestroy");
}
int axr_event_destroy(void* event) {
  return guarded([&] { return event_destroy_body(event); });
}

static int event_record_body(void* event, void* stream) {
  if (!event) return fail(AXR_ERR_INVALID, "axr_event_record: null event");
  return check_hip(hipEventRecord(static_cast<hipEvent_t>(event),
                                  static_cast<hipStream_t>(stream)),
                   "hipEventRecord");
}
int axr_event_record(void* event, void* stream) {
  return guarded([&] { return event_record_body(event, stream); });
}

static int event_synchronize_body(void* event) {
  if (!event) return fail(AXR_ERR_INVALID, "axr_event_synchronize: null event");
  return check_hip(hipEventSynchronize(static_cast<hipEvent_t>(event)), "hipEventSynchronize");
}
int axr_event_synchronize(void* event) {
  return guarded([&] { return event_synchronize_body(event); });
}

static int event_query_body(void* event, int* done) {
  if (!event || !done) return fail(AXR_ERR_INVALID, "axr_event_query: null argument");
  const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipSuccess) {
    *done = 1;
    return AXR_OK;
  }
  if (e == hipErrorNotReady) {
    *done = 0;
    return AXR_OK;
  }
  return check_hip(e, "hipEventQuery");
}
int axr_event_query(void* event, int* done) {
  return guarded([&] { return event_query_body(event, done); });
}

static int event_elapsed_ms_body(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return fail(AXR_ERR_INVALID, "axr_event_elapsed_ms: null argument");
  return check_hip(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start),
                                       static_cast<hipEvent_t>(stop)),
                   "hipEventElapsedTime");
}
int axr_event_elapsed_ms(void* start, void* stop, float* ms) {
  return guarded([&] { return event_elapsed_ms_body(start, stop, ms); });
}

// ---------------------------------------------------------------- memory

static int mem_alloc_body(int memory_type, size_t bytes, size_t alignment, void** ptr) {
  if (!ptr) return fail(AXR_ERR_INVALID, "axr_mem_alloc: null result");
  *ptr = nullptr;
  switch (memory_type) {
    case AXR_MEM_HOST: {
      // std::malloc like the reference's device manager (ucx_cuda_memory_manager.hpp:93);
      // over-aligned requests go through aligned_alloc.
      void* p = nullptr;
      if (alignment > alignof(max_align_t)) {
        if (alignment & (alignment - 1)) return fail(AXR_ERR_INVALID, "alignment not a power of two");
        p = std::aligned_alloc(alignment, round_up(bytes ? bytes : 1, alignment));
      } else {
        p = std::malloc(bytes ? bytes : 1);
      }
      if (!p) return fail(AXR_ERR_NOMEM, "host allocation failed");
      *ptr = p;
      return AXR_OK;
    }
    case AXR_MEM_ROCM: {
      axr_pool_t* pool = nullptr;
      int rc = axr_pool_default(&pool);
      if (rc) return rc;
      return axr_pool_alloc(pool, bytes, alignment, ptr, nullptr);
    }
    case AXR_MEM_ROCM_MANAGED: {
      void* p = nullptr;
      int rc = check_hip(hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault),
                         "hipHostMalloc");
      if (rc) return rc;
      *ptr = p;
      return AXR_OK;
    }
    default:
      return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory type");
  }
}
int axr_mem_alloc(int memory_type, size_t bytes, size_t alignment, void** ptr) {
  return guarded([&] { return mem_alloc_body(memory_type, bytes, alignment, ptr); });
}

static int mem_free_body(int memory_type, void* ptr, size_t bytes) {
  if (!ptr) return AXR_OK;
  switch (memory_type) {
    case AXR_MEM_HOST:
      std::free(ptr);
      return AXR_OK;
    case AXR_MEM_ROCM: {
      // the block may come from any device's default pool
      std::lock_guard<std::mutex> lock(g_default_pool_mu);
      for (auto& kv : g_default_pools) {
        if (axr_pool_free(kv.second, ptr) == AXR_OK) return AXR_OK;
      }
      return fail(AXR_ERR_INVALID, "axr_mem_free: pointer not owned by a default pool");
    }
    case AXR_MEM_ROCM_MANAGED:
      return check_hip(hipHostFree(ptr), "hipHostFree");
    default:
      return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory type");
  }
}
int axr_mem_free(int memory_type, void* ptr, size_t bytes) {
  return guarded([&] { return mem_free_body(memory_type, ptr, bytes); });
}

static int copy_kind(int dst_type, int src_type, hipMemcpyKind* kind) {
  auto is_host = [](int t) { return t == AXR_MEM_HOST || t == AXR_MEM_ROCM_MANAGED; };
  auto is_dev = [](int t) { return t == AXR_MEM_ROCM; };
  if (is_host(dst_type) && is_host(src_type)) *kind = hipMemcpyHostToHost;
  else if (is_host(dst_type) && is_dev(src_type)) *kind = hipMemcpyDeviceToHost;
  else if (is_dev(dst_type) && is_host(src_type)) *kind = hipMemcpyHostToDevice;
  else if (is_dev(dst_type) && is_dev(src_type)) *kind = hipMemcpyDeviceToDevice;
  else return fail(AXR_ERR_UNSUPPORTED, "Unsupported memory copy combination");
  return AXR_OK;
}

// Device memory to pageable host memory through two alternating pinned blocks:
// while one block is filled by the copy engine, the other is emptied (host_copy:
// up to host_threads threads).  The runtime's own pageable path reached 18 GB/s on
// MI355X hosts where this reaches 28 GB/s with one thread and the rate of the
// link with four.
static int staged_to_host(void* dst, const void* src, size_t bytes) {
  constexpr size_t kChunk = 8u << 20;
  TableBlock block[2];
  hipEvent_t done[2] = {nullptr, nullptr};
  size_t pending_at[2] = {0, 0}, pending_len[2] = {0, 0};
  int rc = AXR_OK;
  for (int i = 0; i < 2 && !rc; ++i) {
    rc = table_block_acquire(kChunk, &block[i]);
    if (!rc) rc = check_hip(hipEventCreateWithFlags(&done[i], hipEventDisableTiming), "hipEventCreate");
  }
  uint8_t* out = static_cast<uint8_t*>(dst);
  const uint8_t* in = static_cast<const uint8_t*>(src);
  size_t k = 0;
  for (size_t at = 0; at < bytes && !rc; at += kChunk, ++k) {
    const int slot = static_cast<int>(k & 1);
    if (pending_len[slot]) {
      rc = check_hip(hipEventSynchronize(done[slot]), "hipEventSynchronize");
      if (rc) break;
      const HostCopyJob job{out + pending_at[slot], block[slot].host, pending_len[slot]};
      host_copy(&job, 1);
      pending_len[slot] = 0;
    }
    const size_t len = bytes - at < kChunk ? bytes - at : kChunk;
    rc = check_hip(hipMemcpyAsync(block[slot].host, in + at, len, hipMemcpyDeviceToHost, nullptr),
                   "hipMemcpyAsync(staged)");
    if (!rc) rc = check_hip(hipEventRecord(done[slot], nullptr), "hipEventRecord");
    if (!rc) {
      pending_at[slot] = at;
      pending_len[slot] = len;
    }
  }
  for (size_t j = 0; j < 2; ++j) {   // the two blocks still in flight, oldest first
    const int slot = static_cast<int>((k + j) & 1);
    if (!pending_len[slot]) continue;
    const int wait = check_hip(hipEventSynchronize(done[slot]), "hipEventSynchronize");
    if (!wait && !rc) {
      const HostCopyJob job{out + pending_at[slot], block[slot].host, pending_len[slot]};
      host_copy(&job, 1);
    }
    if (wait && !rc) rc = wait;
  }
  for (int i = 0; i < 2; ++i) {
    if (done[i]) (void)hipEventDestroy(done[i]);
    table_block_release(&block[i]);
  }
  return rc;
}

// Pageable host memory to device memory, the other way round: the threads of
// host_copy fill one pinned block while the copy engine drains the other (57 GB/s
// from pinned memory, 32 GB/s for the runtime's own pageable path).
static int staged_from_host(void* dst, const void* src, size_t bytes) {
  constexpr size_t kChunk = 8u << 20;
  TableBlock block[2];
  hipEvent_t done[2] = {nullptr, nullptr};
  bool pending[2] = {false, false};
  int rc = AXR_OK;
  for (int i = 0; i < 2 && !rc; ++i) {
    rc = table_block_acquire(kChunk, &block[i]);
    if (!rc) rc = check_hip(hipEventCreateWithFlags(&done[i], hipEventDisableTiming), "hipEventCreate");
  }
  uint8_t* out = static_cast<uint8_t*>(dst);
  const uint8_t* in = static_cast<const uint8_t*>(src);
  size_t k = 0;
  for (size_t at = 0; at < bytes && !rc; at += kChunk, ++k) {
    const int slot = static_cast<int>(k & 1);
    if (pending[slot]) {   // the block's previous device copy must have read it
      rc = check_hip(hipEventSynchronize(done[slot]), "hipEventSynchronize");
      pending[slot] = false;
      if (rc) break;
    }
    const size_t len = bytes - at < kChunk ? bytes - at : kChunk;
    const HostCopyJob job{block[slot].host, in + at, len};
    host_copy(&job, 1);
    rc = check_hip(hipMemcpyAsync(out + at, block[slot].host, len, hipMemcpyHostToDevice, nullptr),
                   "hipMemcpyAsync(staged)");
    if (!rc) rc = check_hip(hipEventRecord(done[slot], nullptr), "hipEventRecord");
    if (!rc) pending[slot] = true;
  }
  for (int i = 0; i < 2; ++i) {
    if (pending[i]) {
      const int wait = check_hip(hipEventSynchronize(done[i]), "hipEventSynchronize");
      if (wait && !rc) rc = wait;
    }
    if (done[i]) (void)hipEventDestroy(done[i]);
    table_block_release(&block[i]);
  }
  return rc;
}

static int memcpy_body(int dst_type, void* dst, int src_type, const void* src, size_t bytes) {
  if (bytes == 0) return AXR_OK;
  if (!dst || !src) return fail(AXR_ERR_INVALID, "axr_memcpy: null pointer");
  hipMemcpyKind kind;
  int rc = copy_kind(dst_type, src_type, &kind);
  if (rc) return rc;
  if (dst_type == AXR_MEM_HOST && src_type == AXR_MEM_HOST) {
    std::memcpy(dst, src, bytes);
    return AXR_OK;
  }
  if (dst_type == AXR_MEM_HOST && kind == hipMemcpyDeviceToHost && bytes >= (16u << 20)) {
    // everything queued before this copy must have finished, as with hipMemcpy
    rc = check_hip(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
    if (rc) return rc;
    return staged_to_host(dst, src, bytes);
  }
  if (src_type == AXR_MEM_HOST && kind == hipMemcpyHostToDevice && bytes >= (16u << 20))
    return staged_from_host(dst, src, bytes);
  return check_hip(hipMemcpy(dst, src, bytes, kind), "hipMemcpy");
}
int axr_memcpy(int dst_type, void* dst, int src_type, const void* src, size_t bytes) {
  return guarded([&] { return memcpy_body(dst_type, dst, src_type, src, bytes); });
}

static int memcpy_async_body(int dst_type, void* dst, int src_type, const void* src, size_t bytes,
                             void* stream) {
  if (bytes == 0) return AXR_OK;
  if (!dst || !src) return fail(AXR_ERR_INVALID, "axr_memcpy_async: null pointer");
  hipMemcpyKind kind;
  int rc = copy_kind(dst_type, src_type, &kind);
  if (rc) return rc;
  return check_hip(hipMemcpyAsync(dst, src, bytes, kind, static_cast<hipStream_t>(stream)),
                   "hipMemcpyAsync");
}
int axr_memcpy_async(int dst_type,
                     void* dst,
                     int src_type,
                     const void* src,
                     size_t bytes,
                     void* stream) {
  return guarded([&] { return memcpy_async_body(dst_type, dst, src_type, src, bytes, stream); });
}

static int memset_async_body(void* dst, int value, size_t bytes, void* stream) {
  if (bytes == 0) return AXR_OK;
  if (!dst) return fail(AXR_ERR_INVALID, "axr_memset_async: null pointer");
  return launch_fill(dst, value, bytes, stream);
}
int axr_memset_async(void* dst, int value, size_t bytes, void* stream) {
  return guarded([&] { return memset_async_body(dst, value, bytes, stream); });
}

// ---------------------------------------------------------------- pool

static int pool_create_body(int device, size_t slab_bytes, axr_pool_t** pool) {
  if (!pool) return fail(AXR_ERR_INVALID, "axr_pool_create: null result");
  int count = 0;
  int rc = axr_device_count(&count);
  if (rc) return rc;
  if (device < 0 || device >= count)
    return fail(AXR_ERR_NO_DEVICE, "axr_pool_create: no such device " + std::to_string(device));
  axr_pool* p = new (std::nothrow) axr_pool();
  if (!p) return fail(AXR_ERR_NOMEM, "axr_pool_create: out of host memory");
  p->device = device;
  p->slab_bytes = slab_bytes ? round_up(slab_bytes, 2u << 20) : (256u << 20);
  *pool = p;
  return AXR_OK;
}
int axr_pool_create(int device, size_t slab_bytes, axr_pool_t** pool) {
  return guarded([&] { return pool_create_body(device, slab_bytes, pool); });
}

static int pool_destroy_body(axr_pool_t* pool) {
  if (!pool) return AXR_OK;
  {
    std::lock_guard<std::mutex> lock(pool->mu);
    if (!pool->live.empty()) return fail(AXR_ERR_BUSY, "axr_pool_destroy: blocks still allocated");
    DeviceGuard guard;
    (void)guard.enter(pool->device);
    for (auto& kv : pool->slabs) pool_release_slab(pool, kv.second);
    pool->slabs.clear();
  }
  delete pool;
  return AXR_OK;
}
int axr_pool_destroy(axr_pool_t* pool) {
  return guarded([&] { return pool_destroy_body(pool); });
}

static int pool_default_body(axr_pool_t** pool) {
  if (!pool) return fail(AXR_ERR_INVALID, "axr_pool_default: null result");
  int dev = 0;
  int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(g_default_pool_mu);
  auto it = g_default_pools.find(dev);
  if (it == g_default_pools.end()) {
    axr_pool_t* p = nullptr;
    rc = axr_pool_create(dev, 0, &p);
    if (rc) return rc;
    it = g_default_pools.emplace(dev, p).first;
  }
  *pool = it->second;
  return AXR_OK;
}
int axr_pool_default(axr_pool_t** pool) {
  return guarded([&] { return pool_default_body(pool); });
}

static int pool_set_registrar_body(axr_pool_t* pool, axr_register_fn reg, axr_unregister_fn unreg,
                                   void* user) {
  if (!pool) return fail(AXR_ERR_INVALID, "axr_pool_set_registrar: null pool");
  std::lock_guard<std::mutex> lock(pool->mu);
  if (!pool->slabs.empty())
    return fail(AXR_ERR_BUSY, "axr_pool_set_registrar: pool already holds slabs");
  pool->reg = reg;
  pool->unreg = unreg;
  pool->user = user;
  return AXR_OK;
}
int axr_pool_set_registrar(axr_pool_t* pool,
                           axr_register_fn reg,
                           axr_unregister_fn unreg,
                           void* user) {
  return guarded([&] { return pool_set_registrar_body(pool, reg, unreg, user); });
}

static int pool_alloc_body(axr_pool_t* pool, size_t bytes, size_t alignment, void** ptr,
                           void** mem_h) {
  if (!pool || !ptr) return fail(AXR_ERR_INVALID, "axr_pool_alloc: null argument");
  *ptr = nullptr;
  if (mem_h) *mem_h = nullptr;
  if (alignment == 0) alignment = 1;
  if (alignment & (alignment - 1)) return fail(AXR_ERR_INVALID, "alignment not a power of two");
  const size_t g = axr_pool::kGranule;
  const size_t need = round_up(bytes ? bytes : 1, g);
  // Blocks start on 256-byte boundaries; larger alignments over-allocate and shift.
  const size_t slack = alignment > g ? alignment : 0;
  std::lock_guard<std::mutex> lock(pool->mu);
  for (int attempt = 0; attempt < 2; ++attempt) {
    auto it = pool->free_by_size.lower_bound({need + slack, nullptr});
    if (it != pool->free_by_size.end()) {
      char* block = it->second;
      const size_t have = it->first;
      pool->free_by_size.erase(it);
      pool->free_by_addr.erase(block);
      char* user_ptr = block;
      if (slack) {
        user_ptr = reinterpret_cast<char*>(
            round_up(reinterpret_cast<uintptr_t>(block), alignment));
      }
      const size_t used = static_cast<size_t>(user_ptr - block) + need;
      if (have > used) pool->add_free(block + used, have - used);
      pool->live[user_ptr] = {block, used};
      axr_pool::Slab* slab = pool->slab_of(block);
      slab->live++;
      pool->allocated += used;
      if (pool->allocated > pool->peak) pool->peak = pool->allocated;
      *ptr = user_ptr;
      if (mem_h) *mem_h = slab->mem_h;
      return AXR_OK;
    }
    int rc = pool_grow(pool, need + slack);
    if (rc) return rc;
  }
  return fail(AXR_ERR_NOMEM, "axr_pool_alloc: no block after growing the pool");
}
int axr_pool_alloc(axr_pool_t* pool, size_t bytes, size_t alignment, void** ptr, void** mem_h) {
  return guarded([&] { return pool_alloc_body(pool, bytes, alignment, ptr, mem_h); });
}

static int pool_free_body(axr_pool_t* pool, void* ptr) {
  if (!pool) return fail(AXR_ERR_INVALID, "axr_pool_free: null pool");
  if (!ptr) return AXR_OK;
  std::lock_guard<std::mutex> lock(pool->mu);
  auto it = pool->live.find(ptr);
  if (it == pool->live.end()) return fail(AXR_ERR_INVALID, "axr_pool_free: unknown pointer");
  char* block = it->second.first;
  const size_t used = it->second.second;
  pool->live.erase(it);
  pool->slab_of(block)->live--;
  pool->allocated -= used;
  pool->add_free(block, used);
  return AXR_OK;
}
int axr_pool_free(axr_pool_t* pool, void* ptr) {
  return guarded([&] { return pool_free_body(pool, ptr); });
}

static int pool_trim_body(axr_pool_t* pool) {
  if (!pool) return fail(AXR_ERR_INVALID, "axr_pool_trim: null pool");
  std::lock_guard<std::mutex> lock(pool->mu);
  DeviceGuard guard;
  int rc = guard.enter(pool->device);
  if (rc) return rc;
  for (auto it = pool->slabs.begin(); it != pool->slabs.end();) {
    axr_pool::Slab& slab = it->second;
    if (slab.live == 0) {
      // the slab is one coalesced free block
      auto fb = pool->free_by_addr.find(slab.base);
      if (fb != pool->free_by_addr.end() && fb->second == slab.bytes) {
        pool->free_by_size.erase({fb->second, fb->first});
        pool->free_by_addr.erase(fb);
        pool_release_slab(pool, slab);
        it = pool->slabs.erase(it);
        continue;
      }
    }
    ++it;
  }
  return AXR_OK;
}
int axr_pool_trim(axr_pool_t* pool) {
  return guarded([&] { return pool_trim_body(pool); });
}

static int pool_get_stats_body(axr_pool_t* pool, axr_pool_stats_t* stats) {
  if (!pool || !stats) return fail(AXR_ERR_INVALID, "axr_pool_get_stats: null argument");
  std::lock_guard<std::mutex> lock(pool->mu);
  stats->slabs = pool->slabs.size();
  stats->slab_bytes = 0;
  for (auto& kv : pool->slabs) stats->slab_bytes += kv.second.bytes;
  stats->allocated_bytes = pool->allocated;
  stats->live_blocks = pool->live.size();
  stats->peak_bytes = pool->peak;
  return AXR_OK;
}
int axr_pool_get_stats(axr_pool_t* pool, axr_pool_stats_t* stats) {
  return guarded([&] { return pool_get_stats_body(pool, stats); });
}

}  // extern "C"
