/*
 * bundle_oracle.c - CPU restatement of the reference's tensor-bundle path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (execution-ucx_amd/)
 * links, loads or calls this file; it is the checker the HIP path is compared
 * against in tests/, in __graft_entry__.smoke() and as the cpu_baseline leg of
 * bench.py.
 *
 * Each function names the reference lines it follows (paths relative to the
 * execution-ucx source tree) and how it is pinned:
 *
 *   orc_tensor_nbytes   rpc_core/utils/tensor_meta.hpp:91-104
 *       pinned by the sizes the reference's tests state (fp32[1024] -> 4096,
 *       axon/tests/axon_worker_test.cpp:1241-1250, ...).
 *   orc_layout, orc_pack, orc_unpack
 *       tight concatenation in list order: ucx_am_connection_test.cpp:1051-1108
 *       (IOV send -> contiguous receive), the memcpy loops of
 *       ucx_am_context_test.cpp:1740-1751 and axon_worker_test.cpp:1115-1131,
 *       1158-1174, dispatched as DefaultUcxMemoryResourceManager::memcpy does
 *       (ucx_context/ucx_memory_resource.cpp:106-110).  Pinned by those tests'
 *       closed-form patterns and by the compiled reference (oracle/_ref).
 *       align > 1 (zero-filled gaps) is this build's extension; align == 1 is
 *       the reference layout.
 *   orc_split           ucx_context/ucx_context_data.hpp:641-665 (to_buffer_vec)
 *       pinned by ucx_context_data_test.cpp:41-83 and by oracle/_ref.
 *   orc_gather_strided, orc_scatter_strided
 *       NOT reference behaviour: the reference ships the first nbytes of a
 *       view's storage (axon/python/src/dlpack_helpers.cpp:776-780).  The
 *       build gathers the C-order element sequence; pinned against
 *       numpy.ascontiguousarray on random shapes/strides and by brute force.
 *   orc_divide_by_two   ucx_am_context/ucx_am_context_test_cuda_helper.cu:23-28
 *       pinned by the expected values (i % 256) / 2 of
 *       ucx_am_context_test.cpp:321-333.
 *   orc_checksum        this build's verification checksum (no reference
 *       counterpart); pinned by its additivity and a brute-force numpy sum.
 */
#include <pthread.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define ORC_API __attribute__((visibility("default")))

/* prod(shape) * ceil(bits / 8); 0 for ndim == 0; lanes and strides ignored. */
ORC_API uint64_t orc_tensor_nbytes(int32_t ndim, const int64_t* shape, uint8_t bits) {
  if (ndim == 0) return 0;
  int64_t total = 1;
  for (int32_t i = 0; i < ndim; ++i) total *= shape[i];
  uint64_t per_element = ((uint64_t)bits + 7) / 8;
  return (uint64_t)total * per_element;
}

/* offsets[0] = 0; offsets[i+1] = align_up(offsets[i] + sizes[i]).
 * Returns the payload size = offsets[n-1] + sizes[n-1] (0 for n == 0). */
ORC_API uint64_t orc_layout(const uint64_t* sizes, size_t n, uint64_t align,
                            uint64_t* offsets) {
  uint64_t off = 0, end = 0;
  for (size_t i = 0; i < n; ++i) {
    off = (off + align - 1) / align * align;
    offsets[i] = off;
    off += sizes[i];
    end = off;
  }
  return n ? end : 0;
}

/* dst[offsets[i] .. +sizes[i]) = srcs[i]; every other byte of dst[0, total) = 0. */
ORC_API int orc_pack(const void* const* srcs, const uint64_t* sizes, const uint64_t* offsets,
                     size_t n, void* dst, uint64_t total) {
  unsigned char* out = (unsigned char*)dst;
  uint64_t cursor = 0;
  for (size_t i = 0; i < n; ++i) {
    if (offsets[i] < cursor || offsets[i] + sizes[i] > total) return -1;
    memset(out + cursor, 0, offsets[i] - cursor);
    if (sizes[i]) memcpy(out + offsets[i], srcs[i], sizes[i]);
    cursor = offsets[i] + sizes[i];
  }
  if (cursor > total) return -1;
  memset(out + cursor, 0, total - cursor);
  return 0;
}

ORC_API int orc_unpack(const void* src, uint64_t total, const uint64_t* sizes,
                       const uint64_t* offsets, size_t n, void* const* dsts) {
  const unsigned char* in = (const unsigned char*)src;
  for (size_t i = 0; i < n; ++i) {
    if (offsets[i] + sizes[i] > total) return -1;
    if (sizes[i]) memcpy(dsts[i], in + offsets[i], sizes[i]);
  }
  return 0;
}

/* views[i] = base + sum_{j<i} sizes[j]; -1 (std::length_error in the
 * reference) when the sizes add up to more than the buffer holds. */
ORC_API int orc_split(void* base, uint64_t size, const uint64_t* sizes, size_t n,
                      void** views) {
  uint64_t total = 0;
  for (size_t i = 0; i < n; ++i) total += sizes[i];
  if (total > size) return -1;
  char* p = (char*)base;
  for (size_t i = 0; i < n; ++i) {
    views[i] = p;
    p += sizes[i];
  }
  return 0;
}

/* C-order walk over a strided view.  strides in elements, may be negative. */
static void strided_walk(unsigned char* base, int32_t ndim, const int64_t* shape,
                         const int64_t* strides, uint64_t itemsize, unsigned char* flat,
                         int gather) {
  if (ndim == 0) return;               /* sized 0 by the nbytes rule */
  for (int32_t d = 0; d < ndim; ++d)
    if (shape[d] == 0) return;
  int64_t idx[64];
  memset(idx, 0, sizeof(idx));
  uint64_t out = 0;
  for (;;) {
    int64_t off = 0;
    for (int32_t d = 0; d < ndim; ++d) off += idx[d] * strides[d];
    unsigned char* elem = base + off * (int64_t)itemsize;
    if (gather) memcpy(flat + out, elem, itemsize);
    else memcpy(elem, flat + out, itemsize);
    out += itemsize;
    int32_t d = ndim - 1;
    while (d >= 0) {
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
      --d;
    }
    if (d < 0) break;
  }
}

ORC_API void orc_gather_strided(const void* base, int32_t ndim, const int64_t* shape,
                                const int64_t* strides, uint64_t itemsize, void* dst) {
  strided_walk((unsigned char*)base, ndim, shape, strides, itemsize, (unsigned char*)dst, 1);
}

ORC_API void orc_scatter_strided(const void* src, int32_t ndim, const int64_t* shape,
                                 const int64_t* strides, uint64_t itemsize, void* base) {
  strided_walk((unsigned char*)base, ndim, shape, strides, itemsize, (unsigned char*)src, 0);
}

ORC_API void orc_divide_by_two(float* data, size_t n) {
  for (size_t i = 0; i < n; ++i) data[i] /= 2.0f;
}

/* sum b[i] * (1 + ((start + i) mod 65521)) mod 2^64 */
ORC_API uint64_t orc_checksum(const void* data, uint64_t n, uint64_t start) {
  const unsigned char* b = (const unsigned char*)data;
  uint64_t sum = 0;
  for (uint64_t i = 0; i < n; ++i) sum += (uint64_t)b[i] * (1u + ((start + i) % 65521u));
  return sum;
}

/* ------------------------------------------------------------ CPU timing
 * pack + unpack of one bundle, `reps` times, on `threads` threads (1 = the
 * plain loop above; more = the tensor list cut into byte-balanced contiguous
 * ranges, one per thread).  Returns seconds per repetition (median). */

typedef struct {
  const void* const* srcs;
  void* const* dsts;
  const uint64_t* sizes;
  const uint64_t* offsets;
  unsigned char* packed;
  uint64_t lo, hi; /* byte range [lo, hi) of the concatenated data this thread moves */
  size_t n;
} orc_job_t;

static void copy_range(const orc_job_t* j, int unpack) {
  /* walk tensors, moving the intersection of each with [lo, hi) of the data stream */
  uint64_t cursor = 0;
  for (size_t i = 0; i < j->n && cursor < j->hi; ++i) {
    uint64_t b = cursor, e = cursor + j->sizes[i];
    cursor = e;
    if (e <= j->lo) continue;
    uint64_t s = b < j->lo ? j->lo : b;
    uint64_t t = e > j->hi ? j->hi : e;
    if (t <= s) continue;
    unsigned char* p = j->packed + j->offsets[i] + (s - b);
    if (unpack) memcpy((unsigned char*)j->dsts[i] + (s - b), p, t - s);
    else memcpy(p, (const unsigned char*)j->srcs[i] + (s - b), t - s);
  }
}

static void* pack_thread(void* arg) {
  copy_range((const orc_job_t*)arg, 0);
  return NULL;
}
static void* unpack_thread(void* arg) {
  copy_range((const orc_job_t*)arg, 1);
  return NULL;
}

static int cmp_double(const void* a, const void* b) {
  double x = *(const double*)a, y = *(const double*)b;
  return (x > y) - (x < y);
}

ORC_API double orc_time_pack_unpack(const void* const* srcs, void* const* dsts,
                                    const uint64_t* sizes, const uint64_t* offsets, size_t n,
                                    void* packed, uint64_t total, int threads, int warmup,
                                    int reps) {
  if (threads < 1) threads = 1;
  if (reps < 1) reps = 1;
  uint64_t data = 0;
  for (size_t i = 0; i < n; ++i) data += sizes[i];
  orc_job_t* jobs = (orc_job_t*)calloc((size_t)threads, sizeof(orc_job_t));
  pthread_t* tids = (pthread_t*)calloc((size_t)threads, sizeof(pthread_t));
  double* times = (double*)calloc((size_t)reps, sizeof(double));
  for (int t = 0; t < threads; ++t) {
    jobs[t].srcs = srcs;
    jobs[t].dsts = dsts;
    jobs[t].sizes = sizes;
    jobs[t].offsets = offsets;
    jobs[t].packed = (unsigned char*)packed;
    jobs[t].n = n;
    jobs[t].lo = data * (uint64_t)t / (uint64_t)threads;
    jobs[t].hi = data * (uint64_t)(t + 1) / (uint64_t)threads;
  }
  (void)total;
  for (int r = -warmup; r < reps; ++r) {
    struct timespec a, b;
    clock_gettime(CLOCK_MONOTONIC, &a);
    if (threads == 1) {
      copy_range(&jobs[0], 0);
      copy_range(&jobs[0], 1);
    } else {
      for (int t = 0; t < threads; ++t) pthread_create(&tids[t], NULL, pack_thread, &jobs[t]);
      for (int t = 0; t < threads; ++t) pthread_join(tids[t], NULL);
      for (int t = 0; t < threads; ++t) pthread_create(&tids[t], NULL, unpack_thread, &jobs[t]);
      for (int t = 0; t < threads; ++t) pthread_join(tids[t], NULL);
    }
    clock_gettime(CLOCK_MONOTONIC, &b);
    if (r >= 0) times[r] = (double)(b.tv_sec - a.tv_sec) + 1e-9 * (double)(b.tv_nsec - a.tv_nsec);
  }
  qsort(times, (size_t)reps, sizeof(double), cmp_double);
  double median = times[reps / 2];
  free(jobs);
  free(tids);
  free(times);
  return median;
}
