// HIP kernels of the tensor-bundle path, written for gfx950 (64-lane
// wavefronts, no matrix cores involved: this is pure data movement bound by
// HBM bandwidth).
//
// One launch moves a whole bundle.  Every wavefront owns a contiguous range of
// tile ids, finds its first segment in a host-built per-wave index (one scalar
// load instead of a search), and walks forward through the segment table.  A
// tile is at most ROWS x 1 KiB; a wave moves it with ROWS independent 16-byte
// loads per lane issued back to back, then ROWS 16-byte stores, so each wave
// keeps ROWS KiB in flight and every access is a fully coalesced 1 KiB row.
#include <hip/hip_runtime.h>

#include "axr_internal.h"

namespace axr {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Tensor and payload bytes are addressed through explicit global-address-space
// pointers (addresses arrive as integers in the segment table, which would
// otherwise make every access a flat one); the tables themselves are read
// through the constant address space so wave-uniform reads become scalar loads.
#define AXR_GLOBAL __attribute__((address_space(1)))
#define AXR_CONST __attribute__((address_space(4)))
typedef AXR_GLOBAL uint8_t* gbytes;
typedef const AXR_GLOBAL uint8_t* gcbytes;
typedef AXR_GLOBAL u32x4* gvec;
typedef const AXR_GLOBAL u32x4* gcvec;

// 16-byte accesses carry no alignment promise: gfx950 serves unaligned global
// loads and stores in hardware, at full speed when the address happens to be
// aligned (the 256-byte aligned layout with 16-byte aligned tensors) and with
// straddling accesses otherwise (tight layouts with odd sizes).
typedef u32x4 __attribute__((aligned(1))) u32x4_loose;

template <bool NT>
__device__ __forceinline__ u32x4 load16(gcbytes p) {
  const AXR_GLOBAL u32x4_loose* q = reinterpret_cast<const AXR_GLOBAL u32x4_loose*>(p);
  if constexpr (NT) {
    return __builtin_nontemporal_load(q);
  } else {
    return *q;
  }
}

template <bool NT>
__device__ __forceinline__ void store16(gbytes p, u32x4 v) {
  AXR_GLOBAL u32x4_loose* q = reinterpret_cast<AXR_GLOBAL u32x4_loose*>(p);
  if constexpr (NT) {
    __builtin_nontemporal_store(v, q);
  } else {
    *q = v;
  }
}

__device__ __forceinline__ uint32_t uniform(uint32_t v) {
  return __builtin_amdgcn_readfirstlane(v);
}

__device__ __forceinline__ gbytes as_global(uint64_t address) {
  return reinterpret_cast<gbytes>(address);
}

// Wave-cooperative copy of one tile.  src, dst and the length are
// wave-uniform, lane_off is lane * 16.  A full tile is ROWS loads then ROWS
// stores per lane.
template <uint32_t ROWS, bool NTL, bool NTS>
__device__ __forceinline__ void wave_copy_full(gcbytes src, gbytes dst, uint32_t lane_off) {
  u32x4 v[ROWS];
#pragma unroll
  for (uint32_t k = 0; k < ROWS; ++k) v[k] = load16<NTL>(src + lane_off + k * kRowBytes);
#pragma unroll
  for (uint32_t k = 0; k < ROWS; ++k) store16<NTS>(dst + lane_off + k * kRowBytes, v[k]);
}

// A partial tile (n < ROWS KiB) keeps the same shape: slot j (= lane + 64 k)
// moves bytes [16 j, 16 j + 16) while that lies inside the range, and the first
// slot past the last whole vector moves the final 16 bytes [n - 16, n), which
// overlap the previous slot with identical data.  No byte loops, no second
// memory round trip; only ranges under 16 bytes are moved bytewise.
template <uint32_t ROWS, bool NTL, bool NTS>
__device__ __forceinline__ void wave_copy_partial(gcbytes src, gbytes dst, uint32_t n,
                                                  uint32_t lane, uint32_t lane_off) {
  if (n < kVecBytes) {
    if (lane < n) dst[lane] = src[lane];
    return;
  }
  u32x4 v[ROWS];
  const uint32_t body = n & ~15u;            // bytes covered by whole vectors
  const uint32_t last = n - kVecBytes;       // start of the final (possibly overlapping) vector
  const uint32_t limit = body + ((n & 15u) ? kVecBytes : 0u);   // slots at offsets < limit store
#pragma unroll
  for (uint32_t k = 0; k < ROWS; ++k) {
    const uint32_t o = lane_off + k * kRowBytes;
    v[k] = load16<NTL>(src + (o < body ? o : last));   // unconditional: all loads in flight together
  }
  // Pin every loaded value here: it keeps the compiler from sinking a load into
  // the masked store that uses it (load -> wait -> store per slot), and it puts
  // the single wait for the loads ahead of the first store, so no masked store
  // is followed by a wait that would also cover that store's own completion.
#pragma unroll
  for (uint32_t k = 0; k < ROWS; ++k) asm volatile("" : "+v"(v[k])::"memory");
#pragma unroll
  for (uint32_t k = 0; k < ROWS; ++k) {
    const uint32_t o = lane_off + k * kRowBytes;
    if (o < limit) store16<NTS>(dst + (o < body ? o : last), v[k]);
  }
}

// `left` bytes remain in the run from this tile's start; the tile takes at
// most ROWS KiB of them.
template <uint32_t ROWS, bool NTL, bool NTS>
__device__ __forceinline__ void wave_copy(gcbytes src, gbytes dst, uint64_t left, uint32_t lane,
                                          uint32_t lane_off) {
  if (left >= ROWS * kRowBytes) {
    wave_copy_full<ROWS, NTL, NTS>(src, dst, lane_off);
  } else {
    wave_copy_partial<ROWS, NTL, NTS>(src, dst, static_cast<uint32_t>(left), lane, lane_off);
  }
}

__device__ __forceinline__ void wave_zero(gbytes dst, uint32_t n, uint32_t lane) {
  for (uint32_t i = lane; i < n; i += kWaveLanes) dst[i] = 0;
}

template <typename T>
__device__ __forceinline__ void move_as(gcbytes src, gbytes dst) {
  typedef T __attribute__((aligned(1))) loose;   // no alignment promise on either side
  *reinterpret_cast<AXR_GLOBAL loose*>(dst) = *reinterpret_cast<const AXR_GLOBAL loose*>(src);
}

__device__ __forceinline__ void move_granule_dyn(uint32_t g, gcbytes src, gbytes dst) {
  switch (g) {
    case 16: move_as<u32x4>(src, dst); break;
    case 8: move_as<uint64_t>(src, dst); break;
    case 4: move_as<uint32_t>(src, dst); break;
    case 2: move_as<uint16_t>(src, dst); break;
    default: move_as<uint8_t>(src, dst); break;
  }
}

typedef const AXR_CONST Seg* seg_table;
typedef const AXR_CONST Dims* dims_table;

// Byte offset of run `run` inside a strided tensor; dims are right-aligned in
// the table (unused leading entries have extent 1, stride 0).
__device__ __forceinline__ int64_t run_offset(dims_table dm, uint32_t run) {
  int64_t off = 0;
  const uint32_t nd = dm->ndim;
  if (nd == 1)   // one strided dimension (pitched rows, cache blocks): no division
    return static_cast<int64_t>(run) * dm->stride[kMaxOuterDims - 1];
#pragma unroll
  for (int d = static_cast<int>(kMaxOuterDims) - 1; d >= 0; --d) {
    if (static_cast<uint32_t>(d) + nd >= kMaxOuterDims) {
      const uint32_t extent = dm->shape[d];
      const uint32_t next = run / extent;
      const uint32_t idx = run - next * extent;
      off += static_cast<int64_t>(idx) * dm->stride[d];
      run = next;
    }
  }
  return off;
}

// Element mode: the tile covers kTile packed bytes of a strided segment whose
// contiguous runs are short; each lane decodes the tensor address of its own
// granules.  Only kernels instantiated with ELEMENTS carry this code, so the
// streaming kernels keep a small register footprint.
template <bool PACK, uint32_t ROWS>
__device__ __forceinline__ void element_tile(uint64_t seg_ptr, uint64_t run_bytes, dims_table dm,
                                          gbytes pay, uint32_t q, uint32_t lane) {
  constexpr uint32_t kTile = ROWS * kRowBytes;
  const uint32_t g = dm->granule;
  const uint32_t gpr = static_cast<uint32_t>(run_bytes / g);
  const uint64_t b0 = static_cast<uint64_t>(q) * kTile;
  const uint64_t left = dm->nbytes - b0;
  const uint32_t n = left < kTile ? static_cast<uint32_t>(left) : kTile;
  const uint64_t e0 = b0 / g;
  const uint64_t run0 = e0 / gpr;
  const uint32_t w0 = static_cast<uint32_t>(e0 - run0 * gpr);
  uint32_t idx0[kMaxOuterDims];
  {
    uint64_t r = run0;
#pragma unroll
    for (int d = static_cast<int>(kMaxOuterDims) - 1; d >= 0; --d) {
      const uint32_t extent = dm->shape[d];
      const uint64_t next = r / extent;
      idx0[d] = static_cast<uint32_t>(r - next * extent);
      r = next;
    }
  }
  const uint32_t ng = n / g;
  gbytes tbase = as_global(seg_ptr);
  gbytes pbase = pay + b0;
  for (uint32_t e = lane; e < ng; e += kWaveLanes) {
    uint32_t w = w0 + e;
    uint32_t carry = w / gpr;
    w -= carry * gpr;
    int64_t toff = static_cast<int64_t>(w) * g;
#pragma unroll
    for (int d = static_cast<int>(kMaxOuterDims) - 1; d >= 0; --d) {
      const uint32_t extent = dm->shape[d];
      const uint64_t v = static_cast<uint64_t>(idx0[d]) + carry;
      const uint32_t c = static_cast<uint32_t>(v / extent);
      const uint32_t i = static_cast<uint32_t>(v - static_cast<uint64_t>(c) * extent);
      toff += static_cast<int64_t>(i) * dm->stride[d];
      carry = c;
    }
    gbytes pp = pbase + static_cast<uint64_t>(e) * g;
    if constexpr (PACK) {
      move_granule_dyn(g, tbase + toff, pp);
    } else {
      move_granule_dyn(g, pp, tbase + toff);
    }
  }
}

template <bool PACK, uint32_t ROWS, bool NTT, bool NTP, bool ELEMENTS>
__global__ __launch_bounds__(kMaxThreadsPerWorkgroup) void bundle_kernel(
    const Seg* segs_arg, const Dims* dims_arg, const uint32_t* wave_seg_arg, uint8_t* payload_arg,
    uint32_t ntiles, uint32_t tiles_per_wave, uint32_t xcd_remap, uint32_t seg_shift) {
  // Scalar arguments (not one struct) so that the compiler can preload them
  // into SGPRs at dispatch instead of fetching the kernarg segment first.
  KernelArgs a;
  a.segs = segs_arg;
  a.dims = dims_arg;
  a.wave_seg = wave_seg_arg;
  a.payload = payload_arg;
  a.ntiles = ntiles;
  a.tiles_per_wave = tiles_per_wave;
  a.xcd_remap = xcd_remap;
  a.seg_shift = seg_shift;
  constexpr uint32_t kTile = ROWS * kRowBytes;
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint32_t lane_off = lane * kVecBytes;
  uint32_t wg = blockIdx.x;
  if (a.xcd_remap) {
    // consecutive workgroup ids land on consecutive dies; hand die d the d-th
    // contiguous share of the index space so neighbouring tiles share an L2
    wg = (wg % kXcds) * a.xcd_remap + wg / kXcds;
  }
  const uint32_t wave = uniform(wg * (blockDim.x >> 6) + (threadIdx.x >> 6));
  uint32_t t = wave * a.tiles_per_wave;
  if (t >= a.ntiles) return;
  const uint32_t t_end =
      (a.ntiles - t > a.tiles_per_wave) ? t + a.tiles_per_wave : a.ntiles;
  seg_table segs = reinterpret_cast<seg_table>(reinterpret_cast<uintptr_t>(a.segs));
  dims_table dims = reinterpret_cast<dims_table>(reinterpret_cast<uintptr_t>(a.dims));
  const AXR_CONST uint32_t* wave_seg =
      reinterpret_cast<const AXR_CONST uint32_t*>(reinterpret_cast<uintptr_t>(a.wave_seg));
  gbytes payload = reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(a.payload));
  // The index has one entry per block of 2^seg_shift tiles (the planner sizes
  // blocks so that they rarely hold more than one segment); the loop below
  // walks forward from there to the segment of this wave's first tile.
  uint32_t s = wave_seg[t >> a.seg_shift];
  uint64_t seg_ptr = segs[s].ptr, seg_off = segs[s].off, seg_run = segs[s].run_bytes;
  uint32_t seg_begin = segs[s].tile_begin, seg_meta = segs[s].meta;
  uint32_t seg_end = segs[s + 1].tile_begin;

  while (t < t_end) {
    if (t >= seg_end) {   // wave-uniform: step to the next segment
      ++s;
      seg_ptr = segs[s].ptr;
      seg_off = segs[s].off;
      seg_run = segs[s].run_bytes;
      seg_begin = segs[s].tile_begin;
      seg_meta = segs[s].meta;
      seg_end = segs[s + 1].tile_begin;
      continue;
    }
    const uint32_t q = t - seg_begin;
    const uint32_t pad = seg_meta & kSegPadMask;
    const uint32_t dsel = seg_meta >> kSegDimsShift;
    const bool last = (t + 1 == seg_end);
    gbytes pay = payload + seg_off;
    if (dsel == 0) {
      // one contiguous run
      const uint64_t boff = static_cast<uint64_t>(q) * kTile;
      const uint64_t left = seg_run - boff;
      gbytes ten = as_global(seg_ptr) + boff;
      if constexpr (PACK) {
        wave_copy<ROWS, NTT, NTP>(ten, pay + boff, left, lane, lane_off);
        if (last && pad) wave_zero(pay + seg_run, pad, lane);
      } else {
        wave_copy<ROWS, NTP, NTT>(pay + boff, ten, left, lane, lane_off);
      }
    } else if (dsel == kSegFillOnly) {
      if constexpr (PACK) wave_zero(pay, pad, lane);
    } else {
      dims_table dm = dims + (dsel - 1);
      if (dm->mode == kModeRunTiles) {
        const uint32_t tpr = dm->tiles_per_run;
        const uint32_t tpr_log2 = dm->granule;   // run-tile mode: 1 + log2(tpr) when a power of two
        const uint32_t run = tpr_log2 ? q >> (tpr_log2 - 1) : q / tpr;
        const uint32_t piece = q - run * tpr;
        const uint64_t boff = static_cast<uint64_t>(piece) * kTile;
        const uint64_t left = seg_run - boff;
        gbytes ten = as_global(seg_ptr) + run_offset(dm, run) + boff;
        gbytes p = pay + static_cast<uint64_t>(run) * seg_run + boff;
        if constexpr (PACK) {
          wave_copy<ROWS, NTT, NTP>(ten, p, left, lane, lane_off);
        } else {
          wave_copy<ROWS, NTP, NTT>(p, ten, left, lane, lane_off);
        }
      } else if constexpr (ELEMENTS) {
        element_tile<PACK, ROWS>(seg_ptr, seg_run, dm, pay, q, lane);
      }
      if constexpr (PACK) {
        if (last && pad) wave_zero(pay + dm->nbytes, pad, lane);
      }
    }
    ++t;
  }
}

__global__ __launch_bounds__(256) void fill_kernel(uint8_t* dst, uint8_t value, size_t bytes) {
  // 16-byte stores on the aligned body, bytes at both ends.
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t head = (16u - (reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  const size_t h = head < bytes ? head : bytes;
  for (size_t i = tid; i < h; i += nthreads) dst[i] = value;
  const size_t body = (bytes - h) >> 4;
  const uint32_t w = value * 0x01010101u;
  const u32x4 v = {w, w, w, w};
  u32x4* d = reinterpret_cast<u32x4*>(dst + h);
  for (size_t i = tid; i < body; i += nthreads) d[i] = v;
  const size_t done = h + (body << 4);
  for (size_t i = done + tid; i < bytes; i += nthreads) dst[i] = value;
}

__global__ __launch_bounds__(256) void divide_by_two_kernel(float* data, size_t count) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) data[i] /= 2.0f;
}

__global__ __launch_bounds__(256) void compare_kernel(const uint8_t* a, const uint8_t* b,
                                                      size_t bytes,
                                                      unsigned long long* mismatches) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  unsigned long long local = 0;
  for (size_t i = tid; i < bytes; i += nthreads) local += (a[i] != b[i]) ? 1u : 0u;
  if (local) atomicAdd(mismatches, local);
}

__global__ __launch_bounds__(256) void checksum_kernel(const uint8_t* data, size_t bytes,
                                                       uint64_t start,
                                                       unsigned long long* sum) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  unsigned long long local = 0;
  for (size_t i = tid; i < bytes; i += nthreads) {
    const uint64_t wgt = 1u + ((start + i) % 65521u);
    local += static_cast<unsigned long long>(data[i]) * wgt;
  }
  atomicAdd(sum, local);
}

__global__ __launch_bounds__(256) void copy_reference_kernel(u32x4* __restrict__ dst,
                                                             const u32x4* __restrict__ src,
                                                             size_t nvec) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = tid; i < nvec; i += nthreads) dst[i] = src[i];
}

template <bool PACK, uint32_t ROWS>
int launch_rows(const KernelArgs& args, const LaunchConfig& cfg, hipStream_t stream) {
  const dim3 grid(cfg.workgroups), block(cfg.threads);
#define AXR_ARGS args.segs, args.dims, args.wave_seg, args.payload, args.ntiles, args.tiles_per_wave, args.xcd_remap, args.seg_shift
#define AXR_LAUNCH(NTT, NTP, EL) \
  hipLaunchKernelGGL((bundle_kernel<PACK, ROWS, NTT, NTP, EL>), grid, block, 0, stream, AXR_ARGS)
  if (cfg.elements) {
    // strided tensors with short runs are present: the general kernel
    AXR_LAUNCH(false, false, true);
  } else {
    switch (cfg.nontemporal) {   // bit 0: tensor side, bit 1: payload side
      case 0: AXR_LAUNCH(false, false, false); break;
      case 1: AXR_LAUNCH(true, false, false); break;
      case 2: AXR_LAUNCH(false, true, false); break;
      default: AXR_LAUNCH(true, true, false); break;
    }
  }
#undef AXR_LAUNCH
#undef AXR_ARGS
  return check_hip(hipGetLastError(), "bundle kernel launch");
}

template <bool PACK>
int launch_dir(const KernelArgs& args, const LaunchConfig& cfg, hipStream_t stream) {
  switch (cfg.tile_rows) {
    case 1: return launch_rows<PACK, 1>(args, cfg, stream);
    case 2: return launch_rows<PACK, 2>(args, cfg, stream);
    case 4: return launch_rows<PACK, 4>(args, cfg, stream);
    case 8: return launch_rows<PACK, 8>(args, cfg, stream);
    case 16: return launch_rows<PACK, 16>(args, cfg, stream);
    default: return fail(AXR_ERR_INVALID, "tile_rows must be 1, 2, 4, 8 or 16");
  }
}

uint32_t blocks_for(size_t items, uint32_t cap) {
  size_t b = (items + 255) / 256;
  if (b == 0) b = 1;
  return static_cast<uint32_t>(b < cap ? b : cap);
}

}  // namespace

int launch_bundle_kernel(bool pack, const KernelArgs& args, const LaunchConfig& cfg,
                         void* stream) {
  if (args.ntiles == 0 || cfg.workgroups == 0) return AXR_OK;
  // The grid must cover every tile: waves * tiles_per_wave >= ntiles.
  if (cfg.threads == 0 || cfg.threads % kWaveLanes || cfg.threads > kMaxThreadsPerWorkgroup)
    return fail(AXR_ERR_INVALID, "workgroup size must be a multiple of 64 up to 1024");
  if (args.xcd_remap && (cfg.workgroups % kXcds || args.xcd_remap != cfg.workgroups / kXcds))
    return fail(AXR_ERR_INVALID, "die remapping needs a grid that is a multiple of 8");
  const uint64_t covered = static_cast<uint64_t>(cfg.workgroups) * (cfg.threads / kWaveLanes) *
                           cfg.tiles_per_wave;
  if (covered < args.ntiles || args.tiles_per_wave != cfg.tiles_per_wave) {
    return fail(AXR_ERR_INVALID, "launch geometry does not cover the tile range");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return pack ? launch_dir<true>(args, cfg, s) : launch_dir<false>(args, cfg, s);
}

int launch_fill(void* dst, int value, size_t bytes, void* stream) {
  if (bytes == 0) return AXR_OK;
  hipLaunchKernelGGL(fill_kernel, dim3(blocks_for(bytes / 16 + 1, 4096)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint8_t*>(dst),
                     static_cast<uint8_t>(value), bytes);
  return check_hip(hipGetLastError(), "fill kernel launch");
}

}  // namespace axr

using namespace axr;

extern "C" {

int axr_divide_by_two(float* data, size_t count, void* stream) {
  if (count == 0) return AXR_OK;
  if (!data) return fail(AXR_ERR_INVALID, "axr_divide_by_two: null data");
  const size_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffu) return fail(AXR_ERR_INVALID, "axr_divide_by_two: count too large");
  hipLaunchKernelGGL(divide_by_two_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), data, count);
  return check_hip(hipGetLastError(), "divide_by_two launch");
}

int axr_compare(const void* a, const void* b, size_t bytes, uint64_t* mismatches) {
  if (!mismatches) return fail(AXR_ERR_INVALID, "axr_compare: null result");
  *mismatches = 0;
  if (bytes == 0) return AXR_OK;
  if (!a || !b) return fail(AXR_ERR_INVALID, "axr_compare: null range");
  unsigned long long* dev = nullptr;
  int rc = check_hip(hipMalloc(reinterpret_cast<void**>(&dev), sizeof(*dev)), "hipMalloc");
  if (rc) return rc;
  rc = check_hip(hipMemset(dev, 0, sizeof(*dev)), "hipMemset");
  if (!rc) {
    hipLaunchKernelGGL(compare_kernel, dim3(blocks_for(bytes, 8192)), dim3(256), 0, nullptr,
                       static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), bytes, dev);
    rc = check_hip(hipGetLastError(), "compare launch");
  }
  unsigned long long host = 0;
  if (!rc) rc = check_hip(hipMemcpy(&host, dev, sizeof(host), hipMemcpyDeviceToHost), "hipMemcpy");
  (void)hipFree(dev);
  if (!rc) *mismatches = host;
  return rc;
}

int axr_checksum(const void* data, size_t bytes, uint64_t start, uint64_t* sum) {
  if (!sum) return fail(AXR_ERR_INVALID, "axr_checksum: null result");
  *sum = 0;
  if (bytes == 0) return AXR_OK;
  if (!data) return fail(AXR_ERR_INVALID, "axr_checksum: null range");
  unsigned long long* dev = nullptr;
  int rc = check_hip(hipMalloc(reinterpret_cast<void**>(&dev), sizeof(*dev)), "hipMalloc");
  if (rc) return rc;
  rc = check_hip(hipMemset(dev, 0, sizeof(*dev)), "hipMemset");
  if (!rc) {
    hipLaunchKernelGGL(checksum_kernel, dim3(blocks_for(bytes, 8192)), dim3(256), 0, nullptr,
                       static_cast<const uint8_t*>(data), bytes, start, dev);
    rc = check_hip(hipGetLastError(), "checksum launch");
  }
  unsigned long long host = 0;
  if (!rc) rc = check_hip(hipMemcpy(&host, dev, sizeof(host), hipMemcpyDeviceToHost), "hipMemcpy");
  (void)hipFree(dev);
  if (!rc) *sum = host;
  return rc;
}

int axr_copy_reference(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return AXR_OK;
  if (!dst || !src) return fail(AXR_ERR_INVALID, "axr_copy_reference: null range");
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes) & 15u) {
    return fail(AXR_ERR_INVALID, "axr_copy_reference: pointers and size must be multiples of 16");
  }
  const size_t nvec = bytes / 16;
  hipLaunchKernelGGL(copy_reference_kernel, dim3(blocks_for(nvec, 256 * 32)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<u32x4*>(dst),
                     static_cast<const u32x4*>(src), nvec);
  return check_hip(hipGetLastError(), "copy_reference launch");
}

}  // extern "C"
