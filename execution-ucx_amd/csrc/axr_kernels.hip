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
//
// Strided views with long runs use the same tile copy per run.  Views with
// short runs (element mode) and transpositions (square or rectangular blocks
// staged through LDS) live in separate instantiations of the kernel, so that
// bundles without them run the small streaming kernels.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

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

// Zero bytes of an alignment gap: 16-byte stores, the last one covering the gap's final 16
// bytes (one store instruction for a gap of up to 1 KiB); gaps under 16 bytes bytewise.
__device__ __forceinline__ void wave_zero(gbytes dst, uint32_t n, uint32_t lane) {
  if (n < kVecBytes) {
    if (lane < n) dst[lane] = 0;
    return;
  }
  const uint32_t slots = (n + kVecBytes - 1) / kVecBytes;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (uint32_t j = lane; j < slots; j += kWaveLanes) {
    const uint32_t o = j * kVecBytes;
    store16<false>(dst + (o + kVecBytes <= n ? o : n - kVecBytes), zero);
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

// Moves the ng granules (type T) of one element-mode tile, U per lane at a
// time: addresses first, then all loads, then all stores, so a lane keeps U
// accesses in flight instead of a load-wait-store chain per granule.
// decode(e, &packed) gives granule e's tensor-side offset from tbase and its
// payload offset from pbase.
template <bool PACK, typename T, uint32_t U, typename DECODE>
__device__ __forceinline__ void element_moves(gbytes tbase, gbytes pbase, uint32_t ng,
                                              uint32_t lane, uint32_t nt_bits, DECODE decode) {
  typedef T __attribute__((aligned(1))) loose;   // no alignment promise on either side
  // cache hints of the side that is read and of the side that is written (wave-uniform; the
  // empty asm statements keep the arms apart, or the optimizer merges them and drops the hint)
  const bool nt_rd = (nt_bits & (PACK ? 1u : 2u)) != 0, nt_wr = (nt_bits & (PACK ? 2u : 1u)) != 0;
  for (uint32_t e0 = lane; e0 < ng; e0 += U * kWaveLanes) {
    gbytes tp[U], pp[U];
    T val[U];
    bool moves[U];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t e = e0 + u * kWaveLanes;
      const uint32_t ec = e < ng ? e : ng - 1u;   // slots past the end repeat the last slot's load
      uint64_t packed;
      bool live;                                  // false for a slot that pads a run to whole quads
      tp[u] = tbase + decode(ec, &packed, &live);
      pp[u] = pbase + packed;
      moves[u] = live && e < ng;
    }
    if (nt_rd) {
      asm volatile("");
#pragma unroll
      for (uint32_t u = 0; u < U; ++u)
        val[u] = __builtin_nontemporal_load(reinterpret_cast<const AXR_GLOBAL loose*>(PACK ? tp[u] : pp[u]));
      asm volatile("");
    } else {
#pragma unroll
      for (uint32_t u = 0; u < U; ++u)
        val[u] = *reinterpret_cast<const AXR_GLOBAL loose*>(PACK ? tp[u] : pp[u]);
    }
    if constexpr (sizeof(T) == 16) {
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) asm volatile("" : "+v"(val[u])::"memory");
    }
    if (nt_wr) {
      asm volatile("");
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (moves[u]) __builtin_nontemporal_store(val[u], reinterpret_cast<AXR_GLOBAL loose*>(PACK ? pp[u] : tp[u]));
      }
      asm volatile("");
    } else {
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (moves[u]) *reinterpret_cast<AXR_GLOBAL loose*>(PACK ? pp[u] : tp[u]) = val[u];
      }
    }
  }
}

// Element mode: the tile covers kTile packed bytes of a strided segment whose
// contiguous runs are short; each lane decodes the tensor address of its own
// granules.  Only kernels instantiated with ELEMENTS carry this code, so the
// streaming kernels keep a small register footprint.  The planner keeps every
// extent and the run count below 2^31, so the per-granule arithmetic is 32-bit;
// the tile's first run is decoded once (wave-uniform) and each lane only
// propagates the carry of its own distance from it, stopping at the first
// dimension where no lane carries further.
template <bool PACK, uint32_t ROWS>
__device__ __forceinline__ void element_tile(uint64_t seg_ptr, uint64_t run_bytes, dims_table dm,
                                          gbytes pay, uint32_t q, uint32_t lane, uint32_t nt_bits) {
  nt_bits &= PACK ? dm->nt_allowed : dm->nt_allowed >> 2;
  // element-mode tiles are at least 8 KiB: the per-tile decode is amortised over more bytes
  constexpr uint32_t kTile = ROWS * kRowBytes < kMinElementTileBytes ? kMinElementTileBytes : ROWS * kRowBytes;
  const uint32_t g = dm->granule;
  const uint32_t gs = static_cast<uint32_t>(__builtin_ctz(g));
  // Runs of 16 bytes or more that are no whole number of 64-byte quads (ragged runs):
  // a run is ceil(run / 16) granules of 16 bytes, its last granule covers the run's
  // final 16 bytes (overlapping the one before it with identical data when the length
  // is no multiple of 16), and the run occupies `lanes_per_run` lane slots, the granule
  // count rounded up to a multiple of four: the memory pipeline takes a wave's
  // 16-byte accesses four lanes at a time, and a group of four that lies in one run
  // is one 64-byte request where a group that straddles two runs is two.  Slots past a
  // run's last granule move nothing.  Tiles then count slots, not packed bytes.
  const uint32_t lpr = dm->lanes_per_run;
  const bool ragged = lpr != 0;
  const uint32_t run32 = static_cast<uint32_t>(run_bytes);
  const uint32_t granules = ragged ? (run32 + 15u) >> 4 : static_cast<uint32_t>(run_bytes >> gs);
  const uint32_t gpr = ragged ? lpr : granules;   // slots per run
  const uint32_t nd = dm->ndim;
  const uint64_t b0 = static_cast<uint64_t>(q) * kTile;   // exact runs: packed byte of the tile
  uint64_t e0;
  uint32_t ng;
  if (ragged) {
    e0 = static_cast<uint64_t>(q) * (kTile / kVecBytes);
    const uint64_t left = dm->pstride[0] - e0;            // slots of the whole segment
    ng = left < kTile / kVecBytes ? static_cast<uint32_t>(left) : kTile / kVecBytes;
  } else {
    const uint64_t left = dm->nbytes - b0;
    const uint32_t n = left < kTile ? static_cast<uint32_t>(left) : kTile;
    e0 = b0 >> gs;
    ng = n >> gs;
  }
  uint32_t run0, w0;
  if ((e0 >> 32) == 0) {
    const uint32_t e32 = static_cast<uint32_t>(e0);
    run0 = e32 / gpr;
    w0 = e32 - run0 * gpr;
  } else {
    run0 = static_cast<uint32_t>(e0 / gpr);
    w0 = static_cast<uint32_t>(e0 - static_cast<uint64_t>(run0) * gpr);
  }
  uint32_t idx0[kMaxOuterDims];
  int64_t base = 0;
  {
    uint32_t r = run0;
#pragma unroll
    for (int d = static_cast<int>(kMaxOuterDims) - 1; d >= 0; --d) {
      idx0[d] = 0;
      if (static_cast<uint32_t>(d) + nd >= kMaxOuterDims) {
        const uint32_t extent = dm->shape[d];
        const uint32_t next = r / extent;
        idx0[d] = r - next * extent;
        base += static_cast<int64_t>(idx0[d]) * dm->stride[d];
        r = next;
      }
    }
  }
  const uint32_t gpr_magic = 0xffffffffu / gpr + 1u;
  const int64_t stride_last = dm->stride[kMaxOuterDims - 1];
  const int64_t stride_prev = dm->stride[kMaxOuterDims - 2];
  const uint32_t extent_last = dm->shape[kMaxOuterDims - 1];
  const uint32_t magic_last = 0xffffffffu / extent_last + 1u;
  gbytes tbase = as_global(seg_ptr) + base;
  gbytes pbase = ragged ? pay + static_cast<uint64_t>(run0) * run32 : pay + b0;
  // tensor-side byte offset (relative to the tile's first run) of granule e of the
  // tile, and its payload offset (relative to pbase)
  auto decode = [&](uint32_t e, uint64_t* packed, bool* live) -> int64_t {
    uint32_t w = w0 + e;
    // w < gpr + tile / g: for gpr <= 2^15, w * gpr < 2^32 and the multiply-high quotient is exact
    uint32_t carry = gpr == 1 ? w : (gpr <= 32768u ? __umulhi(w, gpr_magic) : w / gpr);
    w -= carry * gpr;
    uint32_t in_run = w << gs;
    if (ragged) {
      *live = w < granules;
      in_run = w + 1u >= granules ? run32 - kVecBytes : in_run;
      *packed = static_cast<uint64_t>(carry) * run32 + in_run;
    } else {
      *live = true;
      *packed = static_cast<uint64_t>(e) << gs;
    }
    int64_t toff = static_cast<int64_t>(in_run);
    if (nd == 1) {   // one strided dimension (rows of a matrix): the run index is the only coordinate
      return toff + static_cast<int64_t>(carry) * stride_last;
    }
    if (nd == 2) {
      // two strided dimensions (every k-th element of the rows of a matrix, a slice of a
      // 3-d tensor): one quotient, no carry beyond the outer one, nothing to vote on.
      // v < extent + 2^14, so the multiply-high quotient is exact for extents below 2^15.
      uint32_t v = idx0[kMaxOuterDims - 1] + carry;
      uint32_t c = extent_last < 32768u ? __umulhi(v, magic_last) : v / extent_last;
      c = extent_last == 1 ? v : c;
      v -= c * extent_last;
      return toff + static_cast<int64_t>(static_cast<int32_t>(v - idx0[kMaxOuterDims - 1])) * stride_last +
             static_cast<int64_t>(c) * stride_prev;
    }
#pragma unroll
    for (int d = static_cast<int>(kMaxOuterDims) - 1; d >= 0; --d) {
      if (static_cast<uint32_t>(d) + nd >= kMaxOuterDims) {
        if (__builtin_amdgcn_ballot_w64(carry != 0) == 0) break;   // wave-uniform
        const uint32_t extent = dm->shape[d];
        uint32_t v = idx0[d] + carry;
        uint32_t c = 0;
        if (__builtin_amdgcn_ballot_w64(v >= extent) != 0) {
          // v < extent + 2^14: for extents below 2^15 the multiply-high quotient is
          // exact (v * extent < 2^32)
          c = extent < 32768u ? __umulhi(v, 0xffffffffu / extent + 1u) : v / extent;
          c = extent == 1 ? v : c;
          v -= c * extent;
        }
        toff += static_cast<int64_t>(static_cast<int32_t>(v - idx0[d])) * dm->stride[d];
        carry = c;
      }
    }
    return toff;
  };
  // Accesses per lane and round: four in flight.
  switch (g) {
    case 16: element_moves<PACK, u32x4, 4>(tbase, pbase, ng, lane, nt_bits, decode); break;
    case 8: element_moves<PACK, uint64_t, 2>(tbase, pbase, ng, lane, nt_bits, decode); break;
    case 4: element_moves<PACK, uint32_t, 4>(tbase, pbase, ng, lane, nt_bits, decode); break;
    case 2: element_moves<PACK, uint16_t, 4>(tbase, pbase, ng, lane, nt_bits, decode); break;
    default: element_moves<PACK, uint8_t, 4>(tbase, pbase, ng, lane, nt_bits, decode); break;
  }
}

// ---------------------------------------------------------------- transposed tiles
//
// A view whose innermost packed dimension (A) is strided in the tensor while
// another dimension (B) is contiguous there is a transposition: rows that are
// contiguous on one side are columns on the other.  A wavefront moves one
// T x T block (T = 128 bytes / element size) through its own slice of LDS:
// rows are read from global memory as eight 16-byte vectors each (eight rows per
// instruction), parked in LDS in the same orientation with a one-dword pad per
// row, gathered back column-wise, and written as 16-byte vectors along the
// other side's contiguous direction.  Both global sides therefore see whole
// 128-byte lines.  LDS traffic of one wavefront is processed in issue order,
// so no workgroup barrier is involved (waves never share a slice).
#define AXR_LDS __attribute__((address_space(3)))
typedef AXR_LDS uint8_t* lbytes;

template <uint32_t E> struct unit_of;
template <> struct unit_of<1> { typedef uint8_t type; };
template <> struct unit_of<2> { typedef uint16_t type; };
template <> struct unit_of<4> { typedef uint32_t type; };
template <> struct unit_of<8> { typedef uint64_t type; };
template <> struct unit_of<16> { typedef u32x4 type; };

template <uint32_t E>
__device__ __forceinline__ void transpose_full(gcbytes rd, int64_t rd_pitch, gbytes wr,
                                               int64_t wr_pitch, lbytes lds, uint32_t lane,
                                               bool nt_rd, bool nt_wr) {
  constexpr uint32_t T = transpose_edge(E), PITCH = transpose_lds_pitch(E), EV = kVecBytes / E;
  constexpr uint32_t NC = T * E / kVecBytes;   // vectors per block row: 8 or 16
  constexpr uint32_t RPI = kWaveLanes / NC;    // block rows one wave-wide access covers
  constexpr uint32_t NK = T / RPI;
  typedef typename unit_of<E>::type U;
  typedef U __attribute__((aligned(E < 4 ? E : 4))) lds_unit;
  // at most eight vectors per lane in flight: a block of bytes (128 rows) moves in two halves
  constexpr uint32_t B = NK < 8 ? NK : 8;
  const uint32_t r8 = lane / NC, v = lane % NC;
  // The cache hints are wave-uniform: one branch around each batch, not per access.
  // The empty asm statements keep the two arms distinct: without them the optimizer
  // merges the arms' identical accesses and the hint is lost.
#pragma unroll
  for (uint32_t kb = 0; kb < NK; kb += B) {
    u32x4 x[B];
    if (nt_rd) {
      asm volatile("");
#pragma unroll
      for (uint32_t k = 0; k < B; ++k)
        x[k] = load16<true>(rd + static_cast<int64_t>((kb + k) * RPI + r8) * rd_pitch + v * kVecBytes);
      asm volatile("");
    } else {
#pragma unroll
      for (uint32_t k = 0; k < B; ++k)
        x[k] = load16<false>(rd + static_cast<int64_t>((kb + k) * RPI + r8) * rd_pitch + v * kVecBytes);
    }
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) {
      const uint32_t row = (kb + k) * RPI + r8;
      // byte blocks: the 16-byte chunks of a row are permuted by the row's group of
      // 16, which spreads the dword column reads below over the banks
      const uint32_t chunk = E == 1 ? v ^ ((row >> 4) & 7u) : v;
      AXR_LDS uint32_t* w = reinterpret_cast<AXR_LDS uint32_t*>(lds + row * PITCH + chunk * kVecBytes);
      w[0] = x[k].x;
      w[1] = x[k].y;
      w[2] = x[k].z;
      w[3] = x[k].w;
    }
  }
  __builtin_amdgcn_wave_barrier();
  if constexpr (E == 1) {
    // Bytes: a lane produces four output rows at once.  It reads the dword
    // (4 columns) of 16 consecutive block rows and transposes each 4 x 4 byte
    // square in registers (v_perm_b32), a quarter of the LDS reads of a
    // byte-by-byte gather.  256 units of (4 output rows) x (one 16-byte vector).
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k) {
      const uint32_t cg = (lane >> 3) + 8u * k;   // output rows 4 cg .. 4 cg + 3
      const AXR_LDS uint8_t* col = lds + (((cg >> 2) ^ v) * kVecBytes) + (cg & 3u) * 4u;
      u32x4 out[4];
#pragma unroll
      for (uint32_t m = 0; m < 4; ++m) {
        uint32_t d[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
          d[j] = *reinterpret_cast<const AXR_LDS uint32_t*>(col + (v * 16u + m * 4u + j) * PITCH);
        // perm(hi, lo, sel): selector values 0-3 take bytes of lo, 4-7 bytes of hi
        const uint32_t ab_lo = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u);
        const uint32_t ab_hi = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
        const uint32_t cd_lo = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
        const uint32_t cd_hi = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
        out[0][m] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
        out[1][m] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
        out[2][m] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
        out[3][m] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
      }
      if (nt_wr) {
        asm volatile("");
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i)
          store16<true>(wr + static_cast<int64_t>(4u * cg + i) * wr_pitch + v * kVecBytes, out[i]);
        asm volatile("");
      } else {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i)
          store16<false>(wr + static_cast<int64_t>(4u * cg + i) * wr_pitch + v * kVecBytes, out[i]);
      }
    }
    __builtin_amdgcn_wave_barrier();
    return;
  }
#pragma unroll
  for (uint32_t kb = 0; kb < NK; kb += B) {
    u32x4 out[B];
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) {
      const uint32_t c = (kb + k) * RPI + r8;
      U e[EV];
#pragma unroll
      for (uint32_t i = 0; i < EV; ++i)
        e[i] = *reinterpret_cast<const AXR_LDS lds_unit*>(lds + (v * EV + i) * PITCH + c * E);
      __builtin_memcpy(&out[k], e, kVecBytes);
    }
    if (nt_wr) {
      asm volatile("");
#pragma unroll
      for (uint32_t k = 0; k < B; ++k)
        store16<true>(wr + static_cast<int64_t>((kb + k) * RPI + r8) * wr_pitch + v * kVecBytes, out[k]);
      asm volatile("");
    } else {
#pragma unroll
      for (uint32_t k = 0; k < B; ++k)
        store16<false>(wr + static_cast<int64_t>((kb + k) * RPI + r8) * wr_pitch + v * kVecBytes, out[k]);
    }
  }
  __builtin_amdgcn_wave_barrier();
}

// Quotient idx / d by multiplication, exact while idx * d < 2^32 (blocks hold at
// most 2^14 elements with edges up to 2^10).
__device__ __forceinline__ uint32_t small_div(uint32_t idx, uint32_t d, uint32_t magic) {
  return d == 1 ? idx : __umulhi(idx, magic);
}

// Partial or rectangular block: the same two phases one element per lane, eight
// elements per lane in flight.  Both global sides still see consecutive lanes on
// consecutive elements.  Rows in LDS are nc elements plus one dword apart.
template <uint32_t E>
__device__ __forceinline__ void transpose_partial(gcbytes rd, int64_t rd_pitch, gbytes wr,
                                                  int64_t wr_pitch, uint32_t nr, uint32_t nc,
                                                  lbytes lds, uint32_t lane) {
  typedef typename unit_of<E>::type U;
  typedef U __attribute__((aligned(1))) global_unit;
  typedef U __attribute__((aligned(E < 4 ? E : 4))) lds_unit;
  constexpr uint32_t B = E == 16 ? 4 : 8;   // elements per lane and round
  const uint32_t lds_pitch = nc * E + 4u;
  const uint32_t total = nr * nc;
  const uint32_t mc = 0xffffffffu / nc + 1u, mr = 0xffffffffu / nr + 1u;
  for (uint32_t i0 = lane; i0 < total; i0 += B * kWaveLanes) {
    U x[B];
    uint32_t at[B];
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) {
      const uint32_t i = i0 + k * kWaveLanes;
      const uint32_t ic = i < total ? i : total - 1u;   // slots past the end repeat the last element
      const uint32_t r = small_div(ic, nc, mc);
      const uint32_t c = ic - r * nc;
      at[k] = r * lds_pitch + c * E;
      x[k] = *reinterpret_cast<const AXR_GLOBAL global_unit*>(rd + static_cast<int64_t>(r) * rd_pitch + c * E);
    }
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) *reinterpret_cast<AXR_LDS lds_unit*>(lds + at[k]) = x[k];
  }
  __builtin_amdgcn_wave_barrier();
  for (uint32_t i0 = lane; i0 < total; i0 += B * kWaveLanes) {
    U x[B];
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) {
      const uint32_t i = i0 + k * kWaveLanes;
      const uint32_t ic = i < total ? i : total - 1u;
      const uint32_t c = small_div(ic, nr, mr);
      const uint32_t r = ic - c * nr;
      x[k] = *reinterpret_cast<const AXR_LDS lds_unit*>(lds + r * lds_pitch + c * E);
    }
#pragma unroll
    for (uint32_t k = 0; k < B; ++k) {
      const uint32_t i = i0 + k * kWaveLanes;
      if (i < total) {
        const uint32_t c = small_div(i, nr, mr);
        const uint32_t r = i - c * nr;
        *reinterpret_cast<AXR_GLOBAL global_unit*>(wr + static_cast<int64_t>(c) * wr_pitch + r * E) = x[k];
      }
    }
  }
  __builtin_amdgcn_wave_barrier();
}

// Rectangular blocks of 1-, 2- and 4-byte elements with 16-byte accesses on both
// global sides.  One side of
// such a block is a few long rows ("planes"), the other one is contiguous and
// holds the same elements interleaved (nr planes of nc elements <-> nc groups of
// nr elements).  Only the LDS side works element by element.

// nr rows of nc elements (row bytes a multiple of 16) -> one contiguous range.
template <uint32_t E>
__device__ __forceinline__ void rows_to_interleaved(gcbytes rd, int64_t rd_pitch, gbytes wr,
                                                    uint32_t nr, uint32_t nc, lbytes lds,
                                                    uint32_t lane) {
  typedef typename unit_of<E>::type U;
  constexpr uint32_t EV = kVecBytes / E;
  constexpr uint32_t IN = E == 1 ? 2 : 4, OUT = E == 1 ? 1 : 2;   // vectors per lane and round
  const uint32_t pitch = nc * E + 4u, vpr = nc * E / kVecBytes, nvec = nr * vpr;
  const uint32_t mv = 0xffffffffu / vpr + 1u, mr = 0xffffffffu / nr + 1u;
  for (uint32_t v0 = lane; v0 < nvec; v0 += IN * kWaveLanes) {
    u32x4 x[IN];
    uint32_t at[IN];
#pragma unroll
    for (uint32_t k = 0; k < IN; ++k) {
      const uint32_t v = v0 + k * kWaveLanes < nvec ? v0 + k * kWaveLanes : nvec - 1u;
      const uint32_t r = small_div(v, vpr, mv);
      const uint32_t cv = v - r * vpr;
      at[k] = r * pitch + cv * kVecBytes;
      x[k] = load16<false>(rd + static_cast<int64_t>(r) * rd_pitch + cv * kVecBytes);
    }
#pragma unroll
    for (uint32_t k = 0; k < IN; ++k) {   // slots past the end repeat the last vector: same bytes
      AXR_LDS uint32_t* w = reinterpret_cast<AXR_LDS uint32_t*>(lds + at[k]);
      w[0] = x[k].x;
      w[1] = x[k].y;
      w[2] = x[k].z;
      w[3] = x[k].w;
    }
  }
  __builtin_amdgcn_wave_barrier();
  for (uint32_t j0 = lane; j0 < nvec; j0 += OUT * kWaveLanes) {
    u32x4 out[OUT];
#pragma unroll
    for (uint32_t k = 0; k < OUT; ++k) {
      const uint32_t j = j0 + k * kWaveLanes < nvec ? j0 + k * kWaveLanes : nvec - 1u;
      U e[EV];
#pragma unroll
      for (uint32_t i = 0; i < EV; ++i) {
        const uint32_t p = j * EV + i;           // packed element: group b, member a
        const uint32_t b = small_div(p, nr, mr);
        const uint32_t a = p - b * nr;
        e[i] = *reinterpret_cast<const AXR_LDS U*>(lds + a * pitch + b * E);
      }
      __builtin_memcpy(&out[k], e, kVecBytes);
    }
#pragma unroll
    for (uint32_t k = 0; k < OUT; ++k) {
      const uint32_t j = j0 + k * kWaveLanes;
      if (j < nvec) store16<false>(wr + static_cast<uint64_t>(j) * kVecBytes, out[k]);
    }
  }
  __builtin_amdgcn_wave_barrier();
}

// One contiguous range of nr groups of nc elements -> nc rows of nr elements
// (row bytes a multiple of 16).  In LDS every 128 bytes are followed by a pad
// dword, which spreads the strided element reads over the banks.
template <uint32_t E>
__device__ __forceinline__ void interleaved_to_rows(gcbytes rd, gbytes wr, int64_t wr_pitch,
                                                    uint32_t nr, uint32_t nc, lbytes lds,
                                                    uint32_t lane) {
  typedef typename unit_of<E>::type U;
  constexpr uint32_t EV = kVecBytes / E;
  constexpr uint32_t IN = E == 1 ? 2 : 4, OUT = E == 1 ? 1 : 2;   // vectors per lane and round
  const uint32_t vpr = nr * E / kVecBytes, nvec = nc * vpr;
  const uint32_t mv = 0xffffffffu / vpr + 1u;
  for (uint32_t j0 = lane; j0 < nvec; j0 += IN * kWaveLanes) {
    u32x4 x[IN];
    uint32_t at[IN];
#pragma unroll
    for (uint32_t k = 0; k < IN; ++k) {
      const uint32_t j = j0 + k * kWaveLanes < nvec ? j0 + k * kWaveLanes : nvec - 1u;
      at[k] = j * kVecBytes + (j >> 3) * 4u;
      x[k] = load16<false>(rd + static_cast<uint64_t>(j) * kVecBytes);
    }
#pragma unroll
    for (uint32_t k = 0; k < IN; ++k) {
      AXR_LDS uint32_t* w = reinterpret_cast<AXR_LDS uint32_t*>(lds + at[k]);
      w[0] = x[k].x;
      w[1] = x[k].y;
      w[2] = x[k].z;
      w[3] = x[k].w;
    }
  }
  __builtin_amdgcn_wave_barrier();
  for (uint32_t v0 = lane; v0 < nvec; v0 += OUT * kWaveLanes) {
    u32x4 out[OUT];
    uint32_t c[OUT], cv[OUT];
#pragma unroll
    for (uint32_t k = 0; k < OUT; ++k) {
      const uint32_t v = v0 + k * kWaveLanes < nvec ? v0 + k * kWaveLanes : nvec - 1u;
      c[k] = small_div(v, vpr, mv);
      cv[k] = v - c[k] * vpr;
      U e[EV];
#pragma unroll
      for (uint32_t i = 0; i < EV; ++i) {
        const uint32_t q = ((cv[k] * EV + i) * nc + c[k]) * E;   // byte of element (group r, member c)
        e[i] = *reinterpret_cast<const AXR_LDS U*>(lds + q + (q >> 7) * 4u);
      }
      __builtin_memcpy(&out[k], e, kVecBytes);
    }
#pragma unroll
    for (uint32_t k = 0; k < OUT; ++k) {
      if (v0 + k * kWaveLanes < nvec)
        store16<false>(wr + static_cast<int64_t>(c[k]) * wr_pitch + cv[k] * kVecBytes, out[k]);
    }
  }
  __builtin_amdgcn_wave_barrier();
}

// Reads nr rows of nc elements (rows rd_pitch bytes apart) and writes nc rows of
// nr elements (rows wr_pitch bytes apart).
__device__ __forceinline__ void transpose_block(uint32_t E, gcbytes rd, int64_t rd_pitch, gbytes wr,
                                                int64_t wr_pitch, uint32_t nr, uint32_t nc,
                                                bool square, lbytes lds, uint32_t lane, bool nt_rd,
                                                bool nt_wr) {
  // Whole blocks take the vector path whatever the alignment of the two sides
  // (global 16-byte accesses need none; the LDS side is always aligned).
  if (square) {
    switch (E) {
      case 1: transpose_full<1>(rd, rd_pitch, wr, wr_pitch, lds, lane, nt_rd, nt_wr); break;
      case 2: transpose_full<2>(rd, rd_pitch, wr, wr_pitch, lds, lane, nt_rd, nt_wr); break;
      case 4: transpose_full<4>(rd, rd_pitch, wr, wr_pitch, lds, lane, nt_rd, nt_wr); break;
      case 8: transpose_full<8>(rd, rd_pitch, wr, wr_pitch, lds, lane, nt_rd, nt_wr); break;
      default: transpose_full<16>(rd, rd_pitch, wr, wr_pitch, lds, lane, nt_rd, nt_wr); break;
    }
  } else if (E <= 4 && wr_pitch == static_cast<int64_t>(nr * E) && ((nc * E) & 15u) == 0) {
    // the written side is contiguous: a few long rows become interleaved groups
    if (E == 1) rows_to_interleaved<1>(rd, rd_pitch, wr, nr, nc, lds, lane);
    else if (E == 2) rows_to_interleaved<2>(rd, rd_pitch, wr, nr, nc, lds, lane);
    else rows_to_interleaved<4>(rd, rd_pitch, wr, nr, nc, lds, lane);
  } else if (E <= 4 && rd_pitch == static_cast<int64_t>(nc * E) && ((nr * E) & 15u) == 0) {
    // the read side is contiguous: interleaved groups become a few long rows
    if (E == 1) interleaved_to_rows<1>(rd, wr, wr_pitch, nr, nc, lds, lane);
    else if (E == 2) interleaved_to_rows<2>(rd, wr, wr_pitch, nr, nc, lds, lane);
    else interleaved_to_rows<4>(rd, wr, wr_pitch, nr, nc, lds, lane);
  } else {
    switch (E) {
      case 1: transpose_partial<1>(rd, rd_pitch, wr, wr_pitch, nr, nc, lds, lane); break;
      case 2: transpose_partial<2>(rd, rd_pitch, wr, wr_pitch, nr, nc, lds, lane); break;
      case 4: transpose_partial<4>(rd, rd_pitch, wr, wr_pitch, nr, nc, lds, lane); break;
      case 8: transpose_partial<8>(rd, rd_pitch, wr, wr_pitch, nr, nc, lds, lane); break;
      default: transpose_partial<16>(rd, rd_pitch, wr, wr_pitch, nr, nc, lds, lane); break;
    }
  }
}

// Tile q of a transposed segment: batch index (outer dims), then block (ia, ib).
// Deliberately not inlined: the block routines get a register allocation of
// their own (inlined into the kernel's segment walk they spilled and cost the
// other modes registers too), and forty kernel instantiations share two copies.
template <bool PACK>
__device__ __attribute__((noinline)) void transpose_tile(uint64_t seg_ptr, dims_table dm, gbytes pay,
                                               uint32_t q, lbytes lds, uint32_t lane,
                                               uint32_t nt_bits) {
  const uint32_t E = dm->granule;
  const uint32_t es = static_cast<uint32_t>(__builtin_ctz(E));
  const uint32_t T = transpose_edge(E);
  // rows that straddle lines share them with the neighbouring blocks
  nt_bits &= PACK ? dm->nt_allowed : dm->nt_allowed >> 2;
  const uint32_t edge_a = dm->edge_a, edge_b = dm->edge_b;
  const uint32_t ta = dm->tiles_a, tb = dm->tiles_b;
  const uint32_t per_batch = ta * tb;
  uint32_t o = q / per_batch;
  const uint32_t rem = q - o * per_batch;
  const uint32_t ia = rem / tb;
  const uint32_t ib = rem - ia * tb;
  int64_t toff = 0;
  uint64_t poff = 0;
  const uint32_t nbatch = dm->ndim;
#pragma unroll
  for (int d = static_cast<int>(kMaxBatchDims) - 1; d >= 0; --d) {
    if (static_cast<uint32_t>(d) + nbatch >= kMaxBatchDims) {
      const uint32_t extent = dm->shape[kMaxOuterDims - kMaxBatchDims + d];
      const uint32_t next = o / extent;
      const uint32_t idx = o - next * extent;
      toff += static_cast<int64_t>(idx) * dm->stride[kMaxOuterDims - kMaxBatchDims + d];
      poff += static_cast<uint64_t>(idx) * dm->pstride[d];
      o = next;
    }
  }
  uint32_t a0 = ia * edge_a, b0 = ib * edge_b;
  if (edge_a == T && edge_b == T) {
    // Square blocks: the ragged last block of a dimension that holds at least one whole
    // block is moved back so that it ends at the extent.  It overlaps its neighbour and
    // moves those elements a second time with the same values, and stays on the vector
    // path, where the element-per-lane routine would take many times longer than a whole
    // block (8191 x 8193 bytes: 2.3 -> 5 TB/s).
    if (a0 + T > dm->ext_a && dm->ext_a >= T) a0 = dm->ext_a - T;
    if (b0 + T > dm->ext_b && dm->ext_b >= T) b0 = dm->ext_b - T;
  }
  const uint32_t ra = dm->ext_a - a0, rb = dm->ext_b - b0;
  const uint32_t na = ra < edge_a ? ra : edge_a, nb = rb < edge_b ? rb : edge_b;
  const bool square = na == T && nb == T;   // a whole square block: the vector path
  const int64_t stride_a = dm->stride_a;
  const uint64_t pstride_b = dm->pstride_b;
  gbytes ten = as_global(seg_ptr) + toff + static_cast<int64_t>(a0) * stride_a +
               (static_cast<uint64_t>(b0) << es);
  gbytes pp = pay + poff + static_cast<uint64_t>(b0) * pstride_b + (static_cast<uint64_t>(a0) << es);
  if constexpr (PACK) {
    transpose_block(E, ten, stride_a, pp, static_cast<int64_t>(pstride_b), na, nb, square, lds, lane,
                    (nt_bits & 1u) != 0, (nt_bits & 2u) != 0);
  } else {
    transpose_block(E, pp, static_cast<int64_t>(pstride_b), ten, stride_a, nb, na, square, lds, lane,
                    (nt_bits & 2u) != 0, (nt_bits & 1u) != 0);
  }
}

// ---------------------------------------------------------------- group tiles
//
// Several whole short tensors moved by one wavefront.  A group's block in the table holds
// one 64-bit mask per round of 64 lane slots (bit j: slot j is the first slot of a member),
// the group's payload offset and counts, and then the member records.  Lane l loads member
// l's record while the head arrives by scalar load; slot s finds its member by counting the mask bits up to s (two ALU
// instructions), fetches that member's record from the lane that holds it through the
// cross-lane permute, and moves its 16 bytes: the last data slot of a member covers the
// member's final 16 bytes, the zero slots behind it clear the gap to the next aligned
// offset.  Members and gaps shorter than 16 bytes move in pieces of 8, 4, 2 and 1 bytes.
// Both rounds of 64 slots are in flight together: record fetches, then loads, then stores.
__device__ __forceinline__ uint32_t lane_value(uint32_t from_lane, uint32_t value) {
  return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>(from_lane << 2), static_cast<int>(value)));
}

template <bool PACK>
__device__ __attribute__((noinline)) void group_tile(const AXR_CONST GroupHead* head, gbytes payload,
                                                     uint64_t delta, uint32_t lane) {
  typedef uint64_t __attribute__((aligned(1))) loose64;
  typedef uint32_t __attribute__((aligned(1))) loose32;
  typedef uint16_t __attribute__((aligned(1))) loose16;
  constexpr uint32_t R = kGroupMaxSlots / kWaveLanes;
  static_assert(R == 2, "two masks per group head");
  {
    // the block's address is the same in every lane: say so, and the head arrives by scalar load
    const uint64_t a = reinterpret_cast<uint64_t>(head);
    head = reinterpret_cast<const AXR_CONST GroupHead*>(
        static_cast<uint64_t>(uniform(static_cast<uint32_t>(a))) |
        static_cast<uint64_t>(uniform(static_cast<uint32_t>(a >> 32))) << 32);
  }
  // Lane l holds member l % 16's record (only lanes 0..15 are ever asked for theirs).  Every lane
  // loads, so that no branch stands between this load and the loads of the head: a load under a
  // lane mask is waited for inside its branch, which put two memory round trips in a row here.
  const AXR_CONST Member* recs = reinterpret_cast<const AXR_CONST Member*>(head + 1);
  const u32x4 rec = *reinterpret_cast<const AXR_CONST u32x4*>(recs + (lane & (kGroupMaxMembers - 1u)));
  asm volatile("" ::: "memory");   // the record load is issued before the head's loads are waited for
  const uint32_t my_lo = rec.x, my_hi = rec.y, my_off_pad = rec.z, my_nb = rec.w;
  // member of slot s: the number of members that begin at or before s, minus one
  const uint64_t mask0 = head->starts[0], mask1 = head->starts[1];
  gbytes pay = payload + head->off;
  uint32_t m[R];
  {
    const uint32_t lo0 = static_cast<uint32_t>(mask0), hi0 = static_cast<uint32_t>(mask0 >> 32);
    const uint32_t lo1 = static_cast<uint32_t>(mask1), hi1 = static_cast<uint32_t>(mask1 >> 32);
    // mbcnt counts the mask bits below this lane; the lane's own bit is added
    m[0] = __builtin_amdgcn_mbcnt_hi(hi0, __builtin_amdgcn_mbcnt_lo(lo0, 0)) +
           static_cast<uint32_t>((mask0 >> lane) & 1u) - 1u;
    m[1] = static_cast<uint32_t>(__builtin_popcountll(mask0)) +
           __builtin_amdgcn_mbcnt_hi(hi1, __builtin_amdgcn_mbcnt_lo(lo1, 0)) +
           static_cast<uint32_t>((mask1 >> lane) & 1u) - 1u;
  }
  uint32_t f_lo[R], f_hi[R], f_off_pad[R], f_nb[R];
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    const uint32_t from = m[r] & (kGroupMaxMembers - 1u);
    f_lo[r] = lane_value(from, my_lo);
    f_hi[r] = lane_value(from, my_hi);
    f_off_pad[r] = lane_value(from, my_off_pad);
    f_nb[r] = lane_value(from, my_nb);
  }
  // What slot s of a member does, without branches.  With k16 = 16 * (s - first slot of the
  // member) and nd = the bytes its data slots span (n rounded up to 16, at least 16):
  //   k16 < nd           a data slot: bytes [min(k16, n - 16), +16) of a member of 16 bytes or
  //                      more (the last slot overlaps its neighbour), the pieces of a shorter one;
  //   nd <= k16 < nd + pad, pad >= 16   (pack) a zero slot: gap bytes [min(k16 - nd, pad - 16), +16);
  //   anything else      nothing - which covers the slots past the group's last one: they map to
  //                      the last member with k16 beyond its data and zero slots.
  gbytes ten[R], pp[R];
  bool data16[R], zero16[R];
  uint32_t small_n[R];   // a member shorter than 16 bytes: its length, in the lane of its only data slot
  uint32_t small_pad[R]; // a gap shorter than 16 bytes, in the lane of the member's last data slot
  gbytes gap_at[R], small_pp[R];
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    const uint32_t s = r * kWaveLanes + lane;
    const uint64_t ptr = (static_cast<uint64_t>(f_hi[r]) << 32 | f_lo[r]) + delta;
    const uint32_t off_pad = f_off_pad[r], nb = f_nb[r];
    const uint32_t n = nb & 0xffffu, k16 = (s - (nb >> 16)) << 4;
    const uint32_t rel = off_pad & ((1u << kMemberOffBits) - 1u), pad = off_pad >> kMemberOffBits;
    const bool big = n >= kVecBytes;
    const uint32_t nd = big ? (n + kVecBytes - 1u) & ~(kVecBytes - 1u) : kVecBytes;
    const bool is_data = k16 < nd;
    const uint32_t zb = k16 - nd;
    data16[r] = is_data && big;
    zero16[r] = PACK && pad >= kVecBytes && zb < pad;
    small_n[r] = (is_data && !big) ? n : 0u;
    small_pad[r] = (PACK && k16 + kVecBytes == nd && pad < kVecBytes) ? pad : 0u;
    const uint32_t o = data16[r] ? (k16 < n - kVecBytes ? k16 : n - kVecBytes) : 0u;
    const uint32_t oz = zero16[r] ? n + (zb < pad - kVecBytes ? zb : pad - kVecBytes) : o;
    gbytes t0 = as_global(ptr), p0 = pay + rel;
    ten[r] = t0 + o;
    pp[r] = p0 + oz;
    small_pp[r] = p0;
    gap_at[r] = p0 + n;   // where a short gap begins (payload side)
  }
  // Ordinary (cacheable) accesses on both sides whatever the launch's hints: short tensors
  // share their 128-byte lines with their neighbours, and a line marked as streaming is fetched
  // again for the next member (measured: 5 to 15 % slower with either hint).
  // Every load of the tile, the pieces of members shorter than 16 bytes included, is issued
  // before the first store: one memory round trip for the whole tile.
  bool any_small = false;
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) any_small = any_small || small_n[r] != 0;
  const bool wave_has_small = __builtin_amdgcn_ballot_w64(any_small) != 0;   // wave-uniform: most groups have none
  u32x4 v[R];
  uint64_t a8[R];
  uint32_t b4[R];
  uint16_t c2[R];
  uint8_t d1[R];
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    v[r] = u32x4{0u, 0u, 0u, 0u};
    if (data16[r]) v[r] = load16<false>(PACK ? ten[r] : pp[r]);
  }
  if (wave_has_small) {
#pragma unroll
    for (uint32_t r = 0; r < R; ++r) {
      const uint32_t n = small_n[r];
      gcbytes src = PACK ? ten[r] : small_pp[r];
      a8[r] = 0;
      b4[r] = 0;
      c2[r] = 0;
      d1[r] = 0;
      if (n & 8u) a8[r] = *reinterpret_cast<const AXR_GLOBAL loose64*>(src);
      if (n & 4u) b4[r] = *reinterpret_cast<const AXR_GLOBAL loose32*>(src + (n & 8u));
      if (n & 2u) c2[r] = *reinterpret_cast<const AXR_GLOBAL loose16*>(src + (n & 12u));
      if (n & 1u) d1[r] = src[n & 14u];
    }
  }
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) asm volatile("" : "+v"(v[r])::"memory");
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    if (data16[r]) store16<false>(PACK ? pp[r] : ten[r], v[r]);
    else if (PACK && zero16[r]) store16<false>(pp[r], v[r]);
  }
  if (wave_has_small) {
#pragma unroll
    for (uint32_t r = 0; r < R; ++r) {
      const uint32_t n = small_n[r];
      gbytes dst = PACK ? small_pp[r] : ten[r];
      if (n & 8u) *reinterpret_cast<AXR_GLOBAL loose64*>(dst) = a8[r];
      if (n & 4u) *reinterpret_cast<AXR_GLOBAL loose32*>(dst + (n & 8u)) = b4[r];
      if (n & 2u) *reinterpret_cast<AXR_GLOBAL loose16*>(dst + (n & 12u)) = c2[r];
      if (n & 1u) dst[n & 14u] = d1[r];
    }
  }
  if constexpr (PACK) {
    // gaps shorter than 16 bytes (tight layouts have none)
    bool any_gap = false;
#pragma unroll
    for (uint32_t r = 0; r < R; ++r) any_gap = any_gap || small_pad[r] != 0;
    if (__builtin_amdgcn_ballot_w64(any_gap) != 0) {
#pragma unroll
      for (uint32_t r = 0; r < R; ++r) {
        const uint32_t z = small_pad[r];
        gbytes dst = gap_at[r];
        if (z & 8u) *reinterpret_cast<AXR_GLOBAL loose64*>(dst) = 0;
        if (z & 4u) *reinterpret_cast<AXR_GLOBAL loose32*>(dst + (z & 8u)) = 0;
        if (z & 2u) *reinterpret_cast<AXR_GLOBAL loose16*>(dst + (z & 12u)) = 0;
        if (z & 1u) dst[z & 14u] = 0;
      }
    }
  }
}

// The whole pack or unpack of a bundle: every wavefront finds the segment of its
// first tile through the tile-block index and walks forward from there.  `wg` is the
// workgroup's index within this bundle's share of the grid; `a.tensor_delta` is added to
// every tensor-side address (one plan serves tensors of the same geometry elsewhere).
template <bool PACK, uint32_t ROWS, bool NTT, bool NTP, bool ELEMENTS>
__device__ __forceinline__ void bundle_body(seg_table segs, dims_table dims,
                                            const AXR_CONST uint32_t* wave_seg, gbytes payload,
                                            const KernelArgs& a, uint32_t wg, uint32_t lds_per_wave,
                                            uint32_t nt_bits) {
  constexpr uint32_t kTile = ROWS * kRowBytes;
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint32_t lane_off = lane * kVecBytes;
  if (a.xcd_remap) {
    // consecutive workgroup ids land on consecutive dies; hand die d the d-th
    // contiguous share of the index space so neighbouring tiles share an L2
    wg = (wg % kXcds) * a.xcd_remap + wg / kXcds;
  }
  // wavefronts per workgroup travel in bits 8-15 of the hint argument, which is preloaded into
  // a scalar register: blockDim would be a load from the hidden kernel arguments in front of
  // everything else
  const uint32_t waves_per_wg = nt_bits >> 8;
  nt_bits &= 3u;
  const uint32_t wave = uniform(wg * waves_per_wg + (threadIdx.x >> 6));
  uint32_t t = wave * a.tiles_per_wave;
  if (t >= a.ntiles) return;
  const uint32_t t_end =
      (a.ntiles - t > a.tiles_per_wave) ? t + a.tiles_per_wave : a.ntiles;
  const uint64_t delta = static_cast<uint64_t>(a.tensor_delta);
  if (a.seg_shift == kGroupBlocksShift) {
    // a bundle of group tiles only: tile t's block lies at a fixed stride behind `dims`
    const AXR_CONST uint8_t* blocks = reinterpret_cast<const AXR_CONST uint8_t*>(dims);
    for (; t < t_end; ++t)
      group_tile<PACK>(reinterpret_cast<const AXR_CONST GroupHead*>(blocks + static_cast<uint64_t>(t) * kGroupBlockBytes),
                       payload, delta, lane);
    return;
  }
  // The index has one entry per block of 2^seg_shift tiles (the planner sizes
  // blocks so that they rarely hold more than one segment); the loop below
  // walks forward from there to the segment of this wave's first tile.
  // (a bundle whose segments are one tile each needs no index: tile t is segment t)
  uint32_t s = a.seg_shift == kDirectSegShift ? t : wave_seg[t >> a.seg_shift];
  uint64_t seg_ptr = segs[s].ptr + delta, seg_off = segs[s].off, seg_run = segs[s].run_bytes;
  uint32_t seg_begin = segs[s].tile_begin, seg_meta = segs[s].meta;
  uint32_t seg_end = segs[s + 1].tile_begin;

  while (t < t_end) {
    if (t >= seg_end) {   // wave-uniform: step to the next segment
      ++s;
      seg_ptr = segs[s].ptr + delta;
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
      // One contiguous run.  Its first `head` bytes (fewer than 128) are peeled off and
      // moved by tile 0 on top of its own range, so that every tile starts on a 128-byte
      // line of the side that is written.
      const uint32_t head = static_cast<uint32_t>(seg_run >> kSegHeadShift);
      const uint64_t run = seg_run & kSegRunMask;
      const uint64_t boff = head + static_cast<uint64_t>(q) * kTile;
      const uint64_t left = run > boff ? run - boff : 0;
      gbytes ten = as_global(seg_ptr);
      if constexpr (PACK) {
        if (head && q == 0) wave_copy_partial<1, NTT, NTP>(ten, pay, head, lane, lane_off);
        wave_copy<ROWS, NTT, NTP>(ten + boff, pay + boff, left, lane, lane_off);
        if (last && pad) wave_zero(pay + run, pad, lane);
      } else {
        if (head && q == 0) wave_copy_partial<1, NTP, NTT>(pay, ten, head, lane, lane_off);
        wave_copy<ROWS, NTP, NTT>(pay + boff, ten + boff, left, lane, lane_off);
      }
    } else if (dsel == kSegFillOnly) {
      if constexpr (PACK) wave_zero(pay, pad, lane);
    } else if (dsel == kSegGroup) {
      // seg_ptr is an offset into the table block here, not a tensor address
      const AXR_CONST GroupHead* head = reinterpret_cast<const AXR_CONST GroupHead*>(
          reinterpret_cast<const AXR_CONST uint8_t*>(segs) + (seg_ptr - delta));
      group_tile<PACK>(head, payload, delta, lane);
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
        if (dm->mode == kModeTranspose) {
          extern __shared__ uint8_t lds_slices[];   // lds_per_wave bytes for each wavefront
          lbytes lds = (lbytes)lds_slices + (threadIdx.x >> 6) * lds_per_wave;
          transpose_tile<PACK>(seg_ptr, dm, pay, q, lds, lane, nt_bits);
        } else {
          element_tile<PACK, ROWS>(seg_ptr, seg_run, dm, pay, q, lane, nt_bits);
        }
      }
      if constexpr (PACK) {
        if (last && pad) wave_zero(pay + dm->nbytes, pad, lane);
      }
    }
    ++t;
  }
}

// Tables in device memory (uploaded once per plan).
// At least four waves per SIMD (at most 128 VGPRs): the streaming instantiations
// use far fewer, and the general ones sit just around that limit, where one
// register too many would cost a quarter of the occupancy.
template <bool PACK, uint32_t ROWS, bool NTT, bool NTP, bool ELEMENTS>
__global__ __attribute__((amdgpu_waves_per_eu(4))) __launch_bounds__(ELEMENTS ? kMaxElementThreads : kMaxThreadsPerWorkgroup) void bundle_kernel(
    const Seg* segs_arg, const Dims* dims_arg, const uint32_t* wave_seg_arg, uint8_t* payload_arg,
    uint32_t ntiles, uint32_t tiles_per_wave, uint32_t xcd_remap, uint32_t geometry, int64_t tensor_delta) {
  // Scalar arguments (not one struct) so that the compiler can preload them into SGPRs at
  // dispatch instead of fetching the kernarg segment first.  Fourteen dwords are preloaded,
  // which is why the LDS bytes per wavefront (bits 0-16), the hints with the wavefronts per
  // workgroup (bits 17-23, the argument bundle_body takes) and the tile-block shift (bits
  // 24-31) share one of them: the address delta then fits in as well, and no wavefront waits
  // for a kernel-argument load before it can form its first tensor address.
  const uint32_t lds_per_wave = geometry & 0x1ffffu;
  const uint32_t nt_bits = (geometry >> 17 & 3u) | (geometry >> 19 & 0x1fu) << 8;
  KernelArgs a;
  a.ntiles = ntiles;
  a.tiles_per_wave = tiles_per_wave;
  a.xcd_remap = xcd_remap;
  a.seg_shift = geometry >> 24;
  a.tensor_delta = tensor_delta;
  bundle_body<PACK, ROWS, NTT, NTP, ELEMENTS>(
      reinterpret_cast<seg_table>(reinterpret_cast<uintptr_t>(segs_arg)),
      reinterpret_cast<dims_table>(reinterpret_cast<uintptr_t>(dims_arg)),
      reinterpret_cast<const AXR_CONST uint32_t*>(reinterpret_cast<uintptr_t>(wave_seg_arg)),
      reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(payload_arg)), a, blockIdx.x, lds_per_wave,
      nt_bits);
}

// Several bundles in ONE launch: the grid is cut into consecutive workgroup ranges, one per
// job, and every workgroup walks the tables of its own job in that job's direction (a
// sender packing bundle k + 1 while the receiver unpacks bundle k; a batch of small
// bundles).  Halves the per-launch cost of short kernels.  The job table arrives by value
// and is read in place in the kernarg segment (scalar loads, no private copy).
// 1 when `wg` lies at or beyond `begin`, by the sign of the difference (both are below 2^31):
// scalar arithmetic, where a comparison turned into a lane mask and back.
__device__ __forceinline__ uint32_t at_or_beyond(uint32_t wg, uint32_t begin) {
  return ((wg - begin) >> 31) ^ 1u;
}

// What a wavefront needs for its first two table reads arrives as scalar arguments in front of
// the job table: leading scalar arguments are preloaded into scalar registers when a wavefront
// starts, a struct passed by value is not (and the kernel-argument segment is slow memory).
// `head` = job count (bits 0-7), the in-turn flag (bit 8), the directions of jobs 0 and 1 (bits
// 9, 10: 1 = unpack), "jobs 0 and 1 give every wavefront one tile" (bit 11) and their tile-block
// shifts (bits 16-23, 24-31); then the hints, the first workgroup of job 1 and, for jobs 0 and 1,
// the tile count and the addresses of the tile-block index and of the segment records.  A
// workgroup of a launch of one or two jobs (a pack and an unpack handed over together) finds its
// job, reads its index entry and its segment record without a kernel-argument load in front of
// them; the rest of its job's descriptor (payload address, address delta, strided-view table) is
// read from the table meanwhile.  Launches of more jobs, or of jobs whose wavefronts take several
// tiles, read the descriptor first (first workgroups of jobs that do not exist are kNoJobBegin).
template <uint32_t ROWS, bool NTT, bool NTP, bool ELEMENTS>
__global__ __attribute__((amdgpu_waves_per_eu(4))) __launch_bounds__(ELEMENTS ? kMaxElementThreads : kMaxThreadsPerWorkgroup) void bundle_jobs_kernel(
    uint32_t head, uint32_t nt_bits, uint32_t b1, uint32_t ntiles0, uint64_t index0, uint64_t segs0,
    uint64_t index1, uint64_t segs1, uint32_t ntiles1, uint32_t lds_per_wave, JobTable jobs_arg) {
  (void)jobs_arg;
  static_assert(kJobTableKernargOffset % alignof(JobTable) == 0 && kJobTableKernargOffset >= 14 * 4, "kernarg layout");
  const AXR_CONST JobTable* jt = (const AXR_CONST JobTable*)((const AXR_CONST uint8_t*)
      __builtin_amdgcn_kernarg_segment_ptr() + kJobTableKernargOffset);
  const uint32_t wg = blockIdx.x;
  const uint32_t count = head & 0xffu;
  // the job whose workgroup range holds this workgroup: the ranges ascend, so it is the number of
  // ranges that begin at or below this workgroup
  uint32_t j = at_or_beyond(wg, b1);
  if (count > 2) {
#pragma unroll
    for (uint32_t k = 2; k < kMaxJobs; ++k) j += at_or_beyond(wg, jt->begins[k]);
  }
  bool in_turn = false;
  if constexpr (NTP) {
    // Streaming payloads only (these instantiations): two jobs of equal grids take the
    // workgroups in turn.  Kept out of the other instantiations, where the extra test cost the
    // 48 MB bundle 0.7 % per launch.
    in_turn = (head & 0x100u) != 0;
    if (in_turn) j = wg & 1u;
  }
  const AXR_CONST JobDesc* d = &jt->job[j];
  KernelArgs a;
  a.xcd_remap = 0;
  const AXR_CONST uint32_t* wave_seg;
  seg_table segs;
  uint32_t begin, unpack;
  if (j < 2 && (head & 0x800u) != 0) {   // from the preloaded arguments (uniform)
    wave_seg = reinterpret_cast<const AXR_CONST uint32_t*>(j ? index1 : index0);
    segs = reinterpret_cast<seg_table>(j ? segs1 : segs0);
    a.ntiles = j ? ntiles1 : ntiles0;
    a.tiles_per_wave = 1;
    a.seg_shift = (head >> (16u + 8u * j)) & 0xffu;
    unpack = (head >> (9u + j)) & 1u;
    begin = j ? b1 : 0u;
  } else {
    wave_seg = reinterpret_cast<const AXR_CONST uint32_t*>(d->wave_seg);
    uint64_t segs_at = d->segs;
    a.ntiles = d->ntiles;
    a.tiles_per_wave = d->tiles_per_wave;
    a.seg_shift = d->seg_shift;
    unpack = d->unpack;
    begin = d->wg_begin;
    // consumed here, so that these loads are waited for inside this arm and not where the arms
    // meet (scalar loads return out of order: a wait there would cover the loads issued below)
    asm volatile("" : "+s"(begin), "+s"(unpack), "+s"(a.ntiles), "+s"(a.tiles_per_wave), "+s"(a.seg_shift));
    asm volatile("" : "+s"(wave_seg), "+s"(segs_at));
    segs = reinterpret_cast<seg_table>(segs_at);
  }
  // The rest of the descriptor is asked for here, behind the branch: loads issued in front of it
  // would be waited for where the two arms meet, ahead of the first table read.
  asm volatile("" ::: "memory");
  a.tensor_delta = d->tensor_delta;
  dims_table dims = reinterpret_cast<dims_table>(d->dims);
  gbytes payload = reinterpret_cast<gbytes>(d->payload);
  const uint32_t local = in_turn ? wg >> 1 : wg - begin;
  if (unpack) {   // workgroup-uniform
    bundle_body<false, ROWS, NTT, NTP, ELEMENTS>(segs, dims, wave_seg, payload, a, local, lds_per_wave, nt_bits);
  } else {
    bundle_body<true, ROWS, NTT, NTP, ELEMENTS>(segs, dims, wave_seg, payload, a, local, lds_per_wave, nt_bits);
  }
}

// Tables of a small bundle travelling in the kernel arguments themselves: no
// device block, no upload and nothing to keep alive after the launch.  The
// kernarg segment holds the explicit arguments in order at their natural
// alignment, so `tables` sits at kInlineTablesOffset; the kernel addresses it
// there through the constant address space like the uploaded tables, and does
// nothing unless the first word carries the mark the host wrote.
struct InlineScalars {   // mirrors the argument list of bundle_kernel_inline
  uint8_t* payload;
  uint32_t ntiles, tiles_per_wave, xcd_remap, seg_shift, lds_per_wave, nt_bits, dims_at, wave_at;
  InlineTables tables;
};
constexpr uint32_t kInlineTablesOffset = __builtin_offsetof(InlineScalars, tables);
static_assert(kInlineTablesOffset == 48 && alignof(InlineTables) == 16, "kernarg layout");

template <bool PACK, bool ELEMENTS>
__global__ __attribute__((amdgpu_waves_per_eu(4))) __launch_bounds__(ELEMENTS ? kMaxElementThreads : kMaxThreadsPerWorkgroup) void bundle_kernel_inline(
    uint8_t* payload_arg, uint32_t ntiles, uint32_t tiles_per_wave, uint32_t xcd_remap,
    uint32_t seg_shift, uint32_t lds_per_wave, uint32_t nt_bits, uint32_t dims_at, uint32_t wave_at,
    InlineTables tables) {
  (void)tables;
  const AXR_CONST uint8_t* base =
      (const AXR_CONST uint8_t*)__builtin_amdgcn_kernarg_segment_ptr() + kInlineTablesOffset;
  if (*reinterpret_cast<const AXR_CONST uint64_t*>(base) != kInlineTablesMark) return;
  KernelArgs a;
  a.ntiles = ntiles;
  a.tiles_per_wave = tiles_per_wave;
  a.xcd_remap = xcd_remap;
  a.seg_shift = seg_shift;
  a.tensor_delta = 0;
  // tensor side streaming, payload side cacheable: what small bundles use
  bundle_body<PACK, 2, true, false, ELEMENTS>(
      reinterpret_cast<seg_table>(base + kInlineTablesHead),
      reinterpret_cast<dims_table>(base + kInlineTablesHead + dims_at),
      reinterpret_cast<const AXR_CONST uint32_t*>(base + kInlineTablesHead + wave_at),
      reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(payload_arg)), a, blockIdx.x, lds_per_wave,
      nt_bits);
}

__global__ __launch_bounds__(256) void fill_kernel(uint8_t* dst, uint8_t value, size_t bytes) {
  // 16-byte streaming stores on the aligned body, bytes at both ends.
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t head = (16u - (reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  const size_t h = head < bytes ? head : bytes;
  for (size_t i = tid; i < h; i += nthreads) dst[i] = value;
  const size_t body = (bytes - h) >> 4;
  const uint32_t w = value * 0x01010101u;
  const u32x4 v = {w, w, w, w};
  u32x4* d = reinterpret_cast<u32x4*>(dst + h);
  for (size_t i = tid; i < body; i += nthreads) __builtin_nontemporal_store(v, d + i);
  const size_t done = h + (body << 4);
  for (size_t i = done + tid; i < bytes; i += nthreads) dst[i] = value;
}

// The reference's device-side test step (x /= 2 per element), four floats per
// access where the array allows it.
__global__ __launch_bounds__(256) void divide_by_two_kernel(float* data, size_t count) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t head_all = ((16u - (reinterpret_cast<uintptr_t>(data) & 15u)) & 15u) / sizeof(float);
  const size_t head = head_all < count ? head_all : count;
  for (size_t i = tid; i < head; i += nthreads) data[i] /= 2.0f;
  const size_t body = (count - head) / 4;
  f32x4* d = reinterpret_cast<f32x4*>(data + head);
  for (size_t i = tid; i < body; i += nthreads) {
    f32x4 x = d[i];
    x.x /= 2.0f;
    x.y /= 2.0f;
    x.z /= 2.0f;
    x.w /= 2.0f;
    d[i] = x;
  }
  for (size_t i = head + body * 4 + tid; i < count; i += nthreads) data[i] /= 2.0f;
}

// One atomic per workgroup instead of one per thread, spread over kSumSlots
// counters that the host adds up: atomics on one address are served one after
// the other (about 12 ns each on MI355X), which dominated these kernels whenever
// every thread had something to add.
constexpr uint32_t kSumSlots = 64;
__device__ __forceinline__ void block_atomic_add(unsigned long long* slots, unsigned long long local) {
  __shared__ unsigned long long partial[4];   // launched with 256 threads
#pragma unroll
  for (int step = 32; step >= 1; step >>= 1) local += __shfl_xor(local, step, 64);
  if ((threadIdx.x & (kWaveLanes - 1)) == 0) partial[threadIdx.x >> 6] = local;
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned long long total = partial[0] + partial[1] + partial[2] + partial[3];
    if (total) atomicAdd(slots + blockIdx.x % kSumSlots, total);
  }
}

// Number of bytes that differ, 16 bytes per access (no alignment needed).
__global__ __launch_bounds__(256) void compare_kernel(const uint8_t* a, const uint8_t* b,
                                                      size_t bytes,
                                                      unsigned long long* mismatches) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t nvec = bytes >> 4;
  unsigned long long local = 0;
  for (size_t i = tid; i < nvec; i += nthreads) {
    const u32x4 x = *reinterpret_cast<const u32x4_loose*>(a + (i << 4));
    const u32x4 y = *reinterpret_cast<const u32x4_loose*>(b + (i << 4));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t d = x[k] ^ y[k];
      // bit 7 of every byte that is not zero
      const uint32_t nz = (((d & 0x7f7f7f7fu) + 0x7f7f7f7fu) | d) & 0x80808080u;
      local += __builtin_popcount(nz);
    }
  }
  for (size_t i = (nvec << 4) + tid; i < bytes; i += nthreads) local += (a[i] != b[i]) ? 1u : 0u;
  block_atomic_add(mismatches, local);
}

// sum of byte[i] * (1 + (start + i) mod 65521): the modulus is taken once per
// 16 bytes and stepped from there.
__global__ __launch_bounds__(256) void checksum_kernel(const uint8_t* data, size_t bytes,
                                                       uint64_t start,
                                                       unsigned long long* sum) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t nvec = bytes >> 4;
  unsigned long long local = 0;
  for (size_t i = tid; i < nvec; i += nthreads) {
    const u32x4 x = *reinterpret_cast<const u32x4_loose*>(data + (i << 4));
    uint32_t m = static_cast<uint32_t>((start + (i << 4)) % 65521u);
    uint32_t part = 0;   // 16 * 255 * 65521 fits 32 bits
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        part += ((x[k] >> (8 * j)) & 0xffu) * (m + 1u);
        m = m + 1u == 65521u ? 0u : m + 1u;
      }
    }
    local += part;
  }
  for (size_t i = (nvec << 4) + tid; i < bytes; i += nthreads) {
    const uint64_t wgt = 1u + ((start + i) % 65521u);
    local += static_cast<unsigned long long>(data[i]) * wgt;
  }
  block_atomic_add(sum, local);
}

// Plain copy in the shape of the bundle kernels' wavefronts: every wavefront moves KIB KiB (KIB
// 16-byte loads per lane, all issued before the stores), with or without the streaming hint,
// in workgroups of the launch's choosing.  No tables, no segments: what this kernel reaches is
// what a wavefront shape allows on the device.
template <bool NT, uint32_t KIB>
__global__ __launch_bounds__(1024) void copy_shaped_kernel(uint8_t* dst_arg, const uint8_t* src_arg,
                                                           uint64_t waves, uint32_t waves_per_group) {
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * waves_per_group + (threadIdx.x >> 6);
  if (wave >= waves) return;
  const uint64_t off = wave * (1024ull * KIB) + lane * kVecBytes;
  gcbytes src = reinterpret_cast<gcbytes>(reinterpret_cast<uintptr_t>(src_arg)) + off;
  gbytes dst = reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(dst_arg)) + off;
  u32x4 v[KIB];
#pragma unroll
  for (uint32_t u = 0; u < KIB; ++u) v[u] = load16<NT>(src + u * 1024u);
#pragma unroll
  for (uint32_t u = 0; u < KIB; ++u) store16<NT>(dst + u * 1024u, v[u]);
}

__global__ __launch_bounds__(256) void copy_reference_kernel(u32x4* __restrict__ dst,
                                                             const u32x4* __restrict__ src,
                                                             size_t nvec) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t nthreads = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = tid; i < nvec; i += nthreads) dst[i] = src[i];
}

// Plain gather or scatter of equally long rows at a constant pitch: one 16-byte access per
// lane, a row's last access covering its final 16 bytes, every row in a whole number of
// four-lane groups, four accesses per lane in flight, nothing looked up in a table.  What
// this kernel reaches is what the access pattern of such a strided view allows.
template <bool SCATTER, bool NTS, bool NTP>
__global__ __launch_bounds__(256) void rows_reference_kernel(uint8_t* strided_arg, uint64_t pitch, uint8_t* packed_arg,
                                                             uint32_t run, uint32_t lanes_per_row,
                                                             uint32_t rows_per_wave, uint64_t rows) {
  constexpr uint32_t U = 4;
  gbytes strided = reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(strided_arg));
  gbytes packed = reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(packed_arg));
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const uint64_t row0 = wave * rows_per_wave;
  if (row0 >= rows) return;
  const uint32_t granules = (run + kVecBytes - 1) / kVecBytes;
  const uint32_t magic = 0xffffffffu / lanes_per_row + 1u;   // slots < 2^15: the quotient is exact
  const uint32_t slots = rows_per_wave * lanes_per_row;
  for (uint32_t s0 = lane; s0 < slots; s0 += U * kWaveLanes) {
    gbytes sp[U], pp[U];
    bool live[U];
    u32x4 v[U];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t s = s0 + u * kWaveLanes;
      const uint32_t r = lanes_per_row == 1 ? s : __umulhi(s, magic);
      const uint32_t w = s - r * lanes_per_row;
      const uint64_t row = row0 + r;
      live[u] = s < slots && w < granules && row < rows;
      const uint32_t o = (w + 1u >= granules) ? run - kVecBytes : w * kVecBytes;
      const uint64_t safe_row = live[u] ? row : row0;
      sp[u] = strided + safe_row * pitch + o;
      pp[u] = packed + safe_row * run + o;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) v[u] = SCATTER ? load16<NTP>(pp[u]) : load16<NTS>(sp[u]);
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) asm volatile("" : "+v"(v[u])::"memory");
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      if (live[u]) {
        if constexpr (SCATTER) store16<NTS>(sp[u], v[u]); else store16<NTP>(pp[u], v[u]);
      }
    }
  }
}

// Tables of a bundle of contiguous device tensors.  The host writes the n + 1 segment
// records (one pass over the tensors, straight into pinned memory); this kernel, one thread
// per segment, brings them into device memory and writes the entries of the tile-block index
// that fall into each segment, so that the host neither builds the index nor waits for a copy
// engine.  Tensors without bytes are segments without tiles, which the bundle kernel's walk
// steps over.
constexpr uint32_t kUtilityThreads = 256;   // workgroup size of the table expansion and stream copy launches

__global__ __launch_bounds__(256) void expand_tables_kernel(const Seg* staged, uint32_t n, Seg* segs,
                                                            uint32_t* wave_seg, uint32_t seg_shift) {
  // (the launch below always uses workgroups of kUtilityThreads: blockDim would be a load from
  // the hidden kernel arguments in front of the first read)
  const uint32_t i = blockIdx.x * kUtilityThreads + threadIdx.x;
  if (i > n) return;
  const Seg sg = staged[i];
  segs[i] = sg;
  if (i == n) return;   // the sentinel
  const uint64_t first = sg.tile_begin, last = staged[i + 1].tile_begin;
  // index entries k with first <= (k << seg_shift) < last
  const uint64_t step = 1ull << seg_shift;
  for (uint64_t k = (first + step - 1) >> seg_shift; (k << seg_shift) < last; ++k) wave_seg[k] = i;
}

// One contiguous range, 2 KiB per wavefront with the same tile copy as the bundle
// kernels (two 16-byte loads per lane in flight, an overlapped final vector instead of a
// byte tail).  The loopback transport moves same-device payloads with it.
template <bool NT>
__global__ __launch_bounds__(256) void stream_copy_kernel(const uint8_t* src_arg, uint8_t* dst_arg,
                                                          uint64_t bytes) {
  constexpr uint32_t kTile = 2 * kRowBytes;
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint64_t wave = uniform(blockIdx.x * (kUtilityThreads >> 6) + (threadIdx.x >> 6));
  const uint64_t off = wave * kTile;
  if (off >= bytes) return;
  gcbytes src = reinterpret_cast<gcbytes>(reinterpret_cast<uintptr_t>(src_arg)) + off;
  gbytes dst = reinterpret_cast<gbytes>(reinterpret_cast<uintptr_t>(dst_arg)) + off;
  wave_copy<2, NT, NT>(src, dst, bytes - off, lane, lane * kVecBytes);
}

// The cache hints (bits 0-1) and the wavefronts per workgroup (bits 8-15) in one argument.
uint32_t hint_argument(const LaunchConfig& cfg) {
  return (cfg.nontemporal & 3u) | (cfg.threads / kWaveLanes) << 8;
}

template <bool PACK, uint32_t ROWS>
int launch_rows(const KernelArgs& args, const LaunchConfig& cfg, hipStream_t stream) {
  const dim3 grid(cfg.workgroups), block(cfg.threads);
  const uint32_t lds_bytes = cfg.elements ? cfg.lds_per_wave * (cfg.threads / kWaveLanes) : 0u;
  if (cfg.lds_per_wave > 0x1ffffu || args.seg_shift > 0xffu || cfg.threads / kWaveLanes > 0x1fu)
    return fail(AXR_ERR_INVALID, "launch geometry does not fit the kernel's geometry argument");
  // LDS bytes per wavefront | hints << 17 | wavefronts per workgroup << 19 | tile-block shift << 24
  const uint32_t geometry = cfg.lds_per_wave | (cfg.nontemporal & 3u) << 17 |
                            (cfg.threads / kWaveLanes) << 19 | args.seg_shift << 24;
#define AXR_ARGS args.segs, args.dims, args.wave_seg, args.payload, args.ntiles, args.tiles_per_wave, args.xcd_remap, geometry, args.tensor_delta
#define AXR_LAUNCH(NTT, NTP, EL) \
  hipLaunchKernelGGL((bundle_kernel<PACK, ROWS, NTT, NTP, EL>), grid, block, lds_bytes, stream, AXR_ARGS)
  // cfg.elements: strided tensors with short runs or transpositions are present
  switch ((cfg.elements ? 4u : 0u) | (cfg.nontemporal & 3u)) {   // bit 0: tensor side, bit 1: payload side
    case 0: AXR_LAUNCH(false, false, false); break;
    case 1: AXR_LAUNCH(true, false, false); break;
    case 2: AXR_LAUNCH(false, true, false); break;
    case 3: AXR_LAUNCH(true, true, false); break;
    case 4: AXR_LAUNCH(false, false, true); break;
    case 5: AXR_LAUNCH(true, false, true); break;
    case 6: AXR_LAUNCH(false, true, true); break;
    default: AXR_LAUNCH(true, true, true); break;
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
  if (cfg.elements && cfg.threads > kMaxElementThreads)
    return fail(AXR_ERR_INVALID, "bundles with short strided runs need workgroups of at most 256");
  if (static_cast<uint64_t>(cfg.lds_per_wave) * (cfg.threads / kWaveLanes) > 64u * 1024u)
    return fail(AXR_ERR_INVALID, "workgroup needs more than 64 KiB of LDS");
  const uint64_t covered = static_cast<uint64_t>(cfg.workgroups) * (cfg.threads / kWaveLanes) *
                           cfg.tiles_per_wave;
  if (covered < args.ntiles || args.tiles_per_wave != cfg.tiles_per_wave) {
    return fail(AXR_ERR_INVALID, "launch geometry does not cover the tile range");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return pack ? launch_dir<true>(args, cfg, s) : launch_dir<false>(args, cfg, s);
}

int launch_bundle_jobs(const JobTable& jobs, const LaunchConfig& cfg, void* stream) {
  if (jobs.count == 0 || cfg.workgroups == 0) return AXR_OK;
  if (jobs.count > kMaxJobs) return fail(AXR_ERR_INVALID, "too many jobs for one launch");
  if (cfg.threads == 0 || cfg.threads % kWaveLanes ||
      cfg.threads > (cfg.elements ? kMaxElementThreads : kMaxThreadsPerWorkgroup))
    return fail(AXR_ERR_INVALID, "workgroup size does not fit the kernel");
  if (static_cast<uint64_t>(cfg.lds_per_wave) * (cfg.threads / kWaveLanes) > 64u * 1024u)
    return fail(AXR_ERR_INVALID, "workgroup needs more than 64 KiB of LDS");
  const uint32_t waves_per_wg = cfg.threads / kWaveLanes;
  for (uint32_t k = 0; k < jobs.count; ++k) {
    const JobDesc& d = jobs.job[k];
    const uint32_t end = k + 1 < jobs.count ? jobs.job[k + 1].wg_begin : cfg.workgroups;
    if (d.wg_begin > end || (k == 0 && d.wg_begin != 0))
      return fail(AXR_ERR_INVALID, "job workgroup ranges are not consecutive");
    const uint64_t covered = static_cast<uint64_t>(end - d.wg_begin) * waves_per_wg * d.tiles_per_wave;
    if (covered < d.ntiles) return fail(AXR_ERR_INVALID, "launch geometry does not cover a job's tiles");
  }
  const dim3 grid(cfg.workgroups), block(cfg.threads);
  const uint32_t lds_bytes = cfg.elements ? cfg.lds_per_wave * waves_per_wg : 0u;
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (uint32_t k = 0; k < 2 && k < jobs.count; ++k)
    if (jobs.job[k].seg_shift > 0xffu) return fail(AXR_ERR_INVALID, "tile-block shift does not fit the job head");
  // count, in-turn flag, directions, one tile per wavefront and tile-block shifts of jobs 0 and 1
  const bool one_tile_each = jobs.job[0].tiles_per_wave == 1 && (jobs.count < 2 || jobs.job[1].tiles_per_wave == 1);
  const uint32_t head = (jobs.count & 0xffu) | (jobs.interleaved ? 0x100u : 0u) |
                        (jobs.job[0].unpack ? 0x200u : 0u) | (jobs.count > 1 && jobs.job[1].unpack ? 0x400u : 0u) |
                        (one_tile_each ? 0x800u : 0u) |
                        (jobs.job[0].seg_shift & 0xffu) << 16 | (jobs.count > 1 ? jobs.job[1].seg_shift & 0xffu : 0u) << 24;
#define AXR_JOBS(ROWS, NTT, NTP, EL) \
  hipLaunchKernelGGL((bundle_jobs_kernel<ROWS, NTT, NTP, EL>), grid, block, lds_bytes, s, head, jobs.nt_bits,   \
                     jobs.begins[1], jobs.job[0].ntiles, jobs.job[0].wave_seg, jobs.job[0].segs,               \
                     jobs.job[1].wave_seg, jobs.job[1].segs, jobs.job[1].ntiles, jobs.lds_per_wave, jobs)
#define AXR_JOBS_NT(ROWS, EL)                                    \
  switch (cfg.nontemporal & 3u) {                                \
    case 0: AXR_JOBS(ROWS, false, false, EL); break;             \
    case 1: AXR_JOBS(ROWS, true, false, EL); break;              \
    case 2: AXR_JOBS(ROWS, false, true, EL); break;              \
    default: AXR_JOBS(ROWS, true, true, EL); break;              \
  }
  if (cfg.elements) {
    // bundles with short strided runs or transpositions: the default tile only
    if (cfg.tile_rows != 2) return fail(AXR_ERR_INVALID, "element-mode jobs need 2 KiB tiles");
    AXR_JOBS_NT(2, true)
  } else {
    switch (cfg.tile_rows) {
      case 1: AXR_JOBS_NT(1, false) break;
      case 2: AXR_JOBS_NT(2, false) break;
      case 4: AXR_JOBS_NT(4, false) break;
      case 8: AXR_JOBS_NT(8, false) break;
      case 16: AXR_JOBS_NT(16, false) break;
      default: return fail(AXR_ERR_INVALID, "tile_rows must be 1, 2, 4, 8 or 16");
    }
  }
#undef AXR_JOBS_NT
#undef AXR_JOBS
  return check_hip(hipGetLastError(), "bundle jobs kernel launch");
}

int launch_bundle_kernel_inline(bool pack, const KernelArgs& args, const LaunchConfig& cfg,
                                const InlineTables& tables, uint32_t dims_at, uint32_t wave_at,
                                void* stream) {
  if (args.ntiles == 0 || cfg.workgroups == 0) return AXR_OK;
  if (cfg.tile_rows != 2 || (cfg.nontemporal & 3u) != 1u || args.xcd_remap)
    return fail(AXR_ERR_INVALID, "inline tables go with the default launch geometry only");
  if (cfg.threads == 0 || cfg.threads % kWaveLanes ||
      cfg.threads > (cfg.elements ? kMaxElementThreads : kMaxThreadsPerWorkgroup))
    return fail(AXR_ERR_INVALID, "workgroup size does not fit the kernel");
  if (static_cast<uint64_t>(cfg.lds_per_wave) * (cfg.threads / kWaveLanes) > 64u * 1024u)
    return fail(AXR_ERR_INVALID, "workgroup needs more than 64 KiB of LDS");
  const uint64_t covered = static_cast<uint64_t>(cfg.workgroups) * (cfg.threads / kWaveLanes) *
                           cfg.tiles_per_wave;
  if (covered < args.ntiles || args.tiles_per_wave != cfg.tiles_per_wave)
    return fail(AXR_ERR_INVALID, "launch geometry does not cover the tile range");
  if (std::memcmp(tables.bytes, &kInlineTablesMark, sizeof(kInlineTablesMark)) != 0)
    return fail(AXR_ERR_INVALID, "inline tables lack their mark");
  const dim3 grid(cfg.workgroups), block(cfg.threads);
  const uint32_t lds_bytes = cfg.elements ? cfg.lds_per_wave * (cfg.threads / kWaveLanes) : 0u;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define AXR_INLINE_LAUNCH(PACK, EL)                                                              \
  hipLaunchKernelGGL((bundle_kernel_inline<PACK, EL>), grid, block, lds_bytes, s, args.payload,   \
                     args.ntiles, args.tiles_per_wave, args.xcd_remap, args.seg_shift,            \
                     cfg.lds_per_wave, hint_argument(cfg), dims_at, wave_at, tables)
  if (pack) {
    if (cfg.elements) AXR_INLINE_LAUNCH(true, true); else AXR_INLINE_LAUNCH(true, false);
  } else {
    if (cfg.elements) AXR_INLINE_LAUNCH(false, true); else AXR_INLINE_LAUNCH(false, false);
  }
#undef AXR_INLINE_LAUNCH
  return check_hip(hipGetLastError(), "bundle kernel launch (inline tables)");
}

// ---------------------------------------------------------------- static table area
//
// Device memory for the tables of axr_pack_noalloc: part of the code object, so no
// call ever allocates it.  Every device the library runs on holds its own copy at its
// own address until the process ends.  `scratch` below is only the host-side handle of
// the symbol; the device address comes from hipGetSymbolAddress, once per device, and
// that address is what copies and kernel arguments use.
static __device__ __align__(256) uint8_t scratch[kStaticTableBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<uint8_t*> g_scratch_address[kMaxDevices];
}  // namespace

int static_table_area(void** ptr) {
  int device = -1;
  int rc = check_hip(hipGetDevice(&device), "hipGetDevice");
  if (rc) return rc;
  if (device < 0 || device >= kMaxDevices)
    return fail(AXR_ERR_UNSUPPORTED, "device ordinal beyond the static table area's registry");
  uint8_t* address = g_scratch_address[device].load(std::memory_order_acquire);
  if (!address) {
    // the current device is `device`: the lookup answers for that device's copy.  Two
    // threads racing here obtain the same address.
    void* found = nullptr;
    rc = check_hip(hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(static table area)");
    if (rc) return rc;
    if (!found) return fail(AXR_ERR_HIP, "hipGetSymbolAddress returned no address");
    address = static_cast<uint8_t*>(found);
    g_scratch_address[device].store(address, std::memory_order_release);
  }
  *ptr = address;
  return AXR_OK;
}

int launch_expand_tables(const Seg* staged, uint32_t n, Seg* segs, uint32_t* wave_seg, uint32_t seg_shift,
                         void* stream) {
  hipLaunchKernelGGL(expand_tables_kernel, dim3((n + kUtilityThreads) / kUtilityThreads), dim3(kUtilityThreads), 0,
                     static_cast<hipStream_t>(stream), staged, n, segs, wave_seg, seg_shift);
  return check_hip(hipGetLastError(), "table expansion launch");
}

int launch_stream_copy(void* dst, const void* src, size_t bytes, bool nontemporal, void* stream) {
  if (bytes == 0) return AXR_OK;
  const uint64_t waves = (static_cast<uint64_t>(bytes) + 2 * kRowBytes - 1) / (2 * kRowBytes);
  const uint64_t groups = (waves + kUtilityThreads / kWaveLanes - 1) / (kUtilityThreads / kWaveLanes);
  if (groups > 0x7fffffffull) return fail(AXR_ERR_UNSUPPORTED, "range too long for one copy launch");
  const dim3 grid(static_cast<uint32_t>(groups)), block(kUtilityThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (nontemporal) {
    hipLaunchKernelGGL(stream_copy_kernel<true>, grid, block, 0, s, static_cast<const uint8_t*>(src),
                       static_cast<uint8_t*>(dst), static_cast<uint64_t>(bytes));
  } else {
    hipLaunchKernelGGL(stream_copy_kernel<false>, grid, block, 0, s, static_cast<const uint8_t*>(src),
                       static_cast<uint8_t*>(dst), static_cast<uint64_t>(bytes));
  }
  return check_hip(hipGetLastError(), "stream copy launch");
}

// One lane stores `value` into a word of pinned host memory: a host thread that polls the
// word learns that the stream has reached this point without waiting for the runtime's
// completion signal.  A vector store at system scope; nothing is released with it (the
// kernels ahead of this one in the stream have ended by then).
__global__ void notify_kernel(uint32_t* flag, uint32_t value) {
  if (threadIdx.x == 0) __hip_atomic_store(flag, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

int launch_notify(uint32_t* flag, uint32_t value, void* stream) {
  hipLaunchKernelGGL(notify_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), flag, value);
  return check_hip(hipGetLastError(), "notify kernel launch");
}

int launch_fill(void* dst, int value, size_t bytes, void* stream) {
  if (bytes == 0) return AXR_OK;
  hipLaunchKernelGGL(fill_kernel, dim3(blocks_for(bytes / 16 + 1, 1u << 16)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint8_t*>(dst),
                     static_cast<uint8_t>(value), bytes);
  return check_hip(hipGetLastError(), "fill kernel launch");
}

}  // namespace axr

using namespace axr;

namespace {
// Runs `launch(slots)` with kSumSlots zeroed device counters and returns their sum.
template <typename Launch>
int sum_over_slots(Launch&& launch, const char* what, uint64_t* total) {
  unsigned long long* dev = nullptr;
  const size_t bytes = kSumSlots * sizeof(*dev);
  int rc = check_hip(hipMalloc(reinterpret_cast<void**>(&dev), bytes), "hipMalloc");
  if (rc) return rc;
  rc = check_hip(hipMemset(dev, 0, bytes), "hipMemset");
  if (!rc) {
    launch(dev);
    rc = check_hip(hipGetLastError(), what);
  }
  unsigned long long host[kSumSlots] = {};
  if (!rc) rc = check_hip(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost), "hipMemcpy");
  (void)hipFree(dev);
  if (!rc) {
    uint64_t sum = 0;
    for (unsigned long long v : host) sum += v;
    *total = sum;
  }
  return rc;
}

}  // namespace

extern "C" {

static int divide_by_two_body(float* data, size_t count, void* stream) {
  if (count == 0) return AXR_OK;
  if (!data) return fail(AXR_ERR_INVALID, "axr_divide_by_two: null data");
  hipLaunchKernelGGL(divide_by_two_kernel, dim3(blocks_for(count / 4 + 1, 1u << 18)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), data, count);
  return check_hip(hipGetLastError(), "divide_by_two launch");
}
int axr_divide_by_two(float* data, size_t count, void* stream) {
  return guarded([&] { return divide_by_two_body(data, count, stream); });
}

static int compare_body(const void* a, const void* b, size_t bytes, uint64_t* mismatches) {
  if (!mismatches) return fail(AXR_ERR_INVALID, "axr_compare: null result");
  *mismatches = 0;
  if (bytes == 0) return AXR_OK;
  if (!a || !b) return fail(AXR_ERR_INVALID, "axr_compare: null range");
  return sum_over_slots(
      [&](unsigned long long* slots) {
        hipLaunchKernelGGL(compare_kernel, dim3(blocks_for(bytes / 16 + 1, 1u << 16)), dim3(256), 0,
                           nullptr, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                           bytes, slots);
      },
      "compare launch", mismatches);
}
int axr_compare(const void* a, const void* b, size_t bytes, uint64_t* mismatches) {
  return guarded([&] { return compare_body(a, b, bytes, mismatches); });
}

static int checksum_body(const void* data, size_t bytes, uint64_t start, uint64_t* sum) {
  if (!sum) return fail(AXR_ERR_INVALID, "axr_checksum: null result");
  *sum = 0;
  if (bytes == 0) return AXR_OK;
  if (!data) return fail(AXR_ERR_INVALID, "axr_checksum: null range");
  return sum_over_slots(
      [&](unsigned long long* slots) {
        hipLaunchKernelGGL(checksum_kernel, dim3(blocks_for(bytes / 16 + 1, 1u << 16)), dim3(256), 0,
                           nullptr, static_cast<const uint8_t*>(data), bytes, start, slots);
      },
      "checksum launch", sum);
}
int axr_checksum(const void* data, size_t bytes, uint64_t start, uint64_t* sum) {
  return guarded([&] { return checksum_body(data, bytes, start, sum); });
}

static int copy_reference_body(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return AXR_OK;
  if (!dst || !src) return fail(AXR_ERR_INVALID, "axr_copy_reference: null range");
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes) & 15u) {
    return fail(AXR_ERR_INVALID, "axr_copy_reference: pointers and size must be multiples of 16");
  }
  const size_t nvec = bytes / 16;
  hipLaunchKernelGGL(copy_reference_kernel, dim3(blocks_for(nvec, 1u << 20)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<u32x4*>(dst),
                     static_cast<const u32x4*>(src), nvec);
  return check_hip(hipGetLastError(), "copy_reference launch");
}
int axr_copy_reference(void* dst, const void* src, size_t bytes, void* stream) {
  return guarded([&] { return copy_reference_body(dst, src, bytes, stream); });
}

static int copy_reference_shaped_body(void* dst, const void* src, size_t bytes, uint32_t threads,
                                      uint32_t kib_per_wave, int nontemporal, void* stream) {
  if (bytes == 0) return AXR_OK;
  if (!dst || !src) return fail(AXR_ERR_INVALID, "axr_copy_reference_shaped: null range");
  if (threads < kWaveLanes || threads > 1024 || threads % kWaveLanes)
    return fail(AXR_ERR_INVALID, "axr_copy_reference_shaped: threads must be a multiple of 64 in [64, 1024]");
  if (kib_per_wave != 1 && kib_per_wave != 2 && kib_per_wave != 4)
    return fail(AXR_ERR_INVALID, "axr_copy_reference_shaped: 1, 2 or 4 KiB per wavefront");
  if (bytes % (1024ull * kib_per_wave))
    return fail(AXR_ERR_INVALID, "axr_copy_reference_shaped: size must be a whole number of wavefront tiles");
  const uint64_t waves = bytes / (1024ull * kib_per_wave);
  const uint32_t per_group = threads / kWaveLanes;
  const uint64_t groups = (waves + per_group - 1) / per_group;
  if (groups > 0x7fffffffull) return fail(AXR_ERR_UNSUPPORTED, "axr_copy_reference_shaped: range too long for one launch");
  const dim3 grid(static_cast<uint32_t>(groups)), block(threads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* d = static_cast<uint8_t*>(dst);
  const uint8_t* s = static_cast<const uint8_t*>(src);
#define AXR_SHAPED(NT, KIB) hipLaunchKernelGGL((copy_shaped_kernel<NT, KIB>), grid, block, 0, st, d, s, waves, per_group)
  switch (kib_per_wave * 2 + (nontemporal ? 1 : 0)) {
    case 2: AXR_SHAPED(false, 1); break;
    case 3: AXR_SHAPED(true, 1); break;
    case 4: AXR_SHAPED(false, 2); break;
    case 5: AXR_SHAPED(true, 2); break;
    case 8: AXR_SHAPED(false, 4); break;
    default: AXR_SHAPED(true, 4); break;
  }
#undef AXR_SHAPED
  return check_hip(hipGetLastError(), "copy_reference_shaped launch");
}
int axr_copy_reference_shaped(void* dst, const void* src, size_t bytes, uint32_t threads, uint32_t kib_per_wave,
                              int nontemporal, void* stream) {
  return guarded([&] { return copy_reference_shaped_body(dst, src, bytes, threads, kib_per_wave, nontemporal, stream); });
}

static int rows_reference_body(void* strided, size_t pitch, void* packed, size_t run_bytes, size_t rows,
                               int scatter, uint32_t nontemporal, void* stream) {
  if (rows == 0) return AXR_OK;
  if (!strided || !packed) return fail(AXR_ERR_INVALID, "axr_rows_reference: null range");
  if (run_bytes < kVecBytes || run_bytes > 4096 || pitch < run_bytes)
    return fail(AXR_ERR_INVALID, "axr_rows_reference: rows of 16 to 4096 bytes at a pitch of at least their length");
  const uint32_t granules = static_cast<uint32_t>((run_bytes + kVecBytes - 1) / kVecBytes);
  const uint32_t lanes_per_row = (granules + 3u) & ~3u;
  const uint32_t rows_per_wave = std::max(1u, 512u / lanes_per_row);   // about 8 KiB per wavefront
  const uint64_t waves = (static_cast<uint64_t>(rows) + rows_per_wave - 1) / rows_per_wave;
  const uint64_t groups = (waves + 3) / 4;
  if (groups > 0x7fffffffull) return fail(AXR_ERR_UNSUPPORTED, "axr_rows_reference: too many rows for one launch");
  const dim3 grid(static_cast<uint32_t>(groups)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define AXR_ROWS(SC, A, B)                                                                              \
  hipLaunchKernelGGL((rows_reference_kernel<SC, A, B>), grid, block, 0, st, static_cast<uint8_t*>(strided), \
                     static_cast<uint64_t>(pitch), static_cast<uint8_t*>(packed),                        \
                     static_cast<uint32_t>(run_bytes), lanes_per_row, rows_per_wave, static_cast<uint64_t>(rows))
  switch ((scatter ? 4u : 0u) | (nontemporal & 3u)) {
    case 0: AXR_ROWS(false, false, false); break;
    case 1: AXR_ROWS(false, true, false); break;
    case 2: AXR_ROWS(false, false, true); break;
    case 3: AXR_ROWS(false, true, true); break;
    case 4: AXR_ROWS(true, false, false); break;
    case 5: AXR_ROWS(true, true, false); break;
    case 6: AXR_ROWS(true, false, true); break;
    default: AXR_ROWS(true, true, true); break;
  }
#undef AXR_ROWS
  return check_hip(hipGetLastError(), "rows_reference launch");
}
int axr_rows_reference(void* strided, size_t pitch, void* packed, size_t run_bytes, size_t rows, int scatter,
                       uint32_t nontemporal, void* stream) {
  return guarded([&] { return rows_reference_body(strided, pitch, packed, run_bytes, rows, scatter, nontemporal, stream); });
}

}  // extern "C"
