/*
 * axon_rocm.h - C ABI of the MI355X (gfx950) tensor-bundle path for execution-ucx.
 *
 * The library behind this header replaces, for ROCm memory, the part of the
 * reference that moves tensor payload bytes:
 *
 *   - the IOV gather done inside UCX when a tensor list is sent
 *     (ucx_context/ucx_connection.cpp:401-426, send_am_iov_data) becomes ONE
 *     pack kernel into a contiguous HBM buffer that is then sent as a plain
 *     contiguous ucx_am_data (ucx_connection.cpp:353-374);
 *   - the IOV scatter on receive (ucx_connection.cpp:428-453) becomes ONE
 *     unpack kernel out of the contiguous receive buffer;
 *   - ucx_context/cuda/ucx_cuda_memory_manager.hpp (cudaMalloc/cudaMemcpy) is
 *     replaced by a hipMalloc slab pool + copy table (axr_pool_*, axr_memcpy*);
 *   - ucx_context/cuda/ucx_cuda_context.hpp (cuCtxPushCurrent/PopCurrent) is
 *     replaced by axr_device_push / axr_device_pop.
 *
 * Conventions: every function returns 0 (AXR_OK) or a negative axr_status
 * value, never throws and never aborts.  All entry points are thread-safe
 * unless stated.  Streams and events are opaque pointers (hipStream_t /
 * hipEvent_t underneath); a NULL stream is the device's default stream.
 * No HIP, torch or UCX type appears in a signature.
 */
#ifndef AXON_ROCM_H_
#define AXON_ROCM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXR_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ status */

typedef enum axr_status {
  AXR_OK = 0,
  AXR_ERR_INVALID = -1,         /* bad argument (null pointer, bad shape ...)   */
  AXR_ERR_NOMEM = -2,           /* host or device allocation failed             */
  AXR_ERR_HIP = -3,             /* a HIP runtime call failed (see last error)   */
  AXR_ERR_LENGTH = -4,          /* sizes exceed the buffer they must fit in;
                                   the reference throws std::length_error here
                                   (ucx_context/ucx_context_data.hpp:644-646)   */
  AXR_ERR_UNSUPPORTED = -5,     /* memory type / layout this build cannot move;
                                   the reference throws std::runtime_error
                                   ("Unsupported memory type",
                                   cuda/ucx_cuda_memory_manager.hpp:103,150)    */
  AXR_ERR_NO_MESSAGE = -6,      /* unknown receive key; UCS_ERR_NO_MESSAGE in
                                   ucx_am_context.hpp:1570-1574                 */
  AXR_ERR_NOT_IMPLEMENTED = -7, /* recv_buffer on an eager message;
                                   UCS_ERR_NOT_IMPLEMENTED, :1643-1651          */
  AXR_ERR_HEADER = -8,          /* malformed bundle header                      */
  AXR_ERR_MISMATCH = -9,        /* bound tensors do not match the plan's metas  */
  AXR_ERR_NO_DEVICE = -10,      /* no usable ROCm device in this process        */
  AXR_ERR_BUSY = -11,           /* object still has work in flight              */
  AXR_ERR_CANCELED = -12        /* the peer cancelled the operation
                                   (UCS_ERR_CANCELED)                           */
} axr_status_t;

/* Human-readable name of a status code (static storage). */
AXR_API const char* axr_status_string(int status);
/* Message of the last failure on the calling thread (thread-local storage). */
AXR_API const char* axr_last_error(void);
/* Library version, "major.minor.patch". */
AXR_API const char* axr_version(void);

/* ------------------------------------------------------------ memory types */

/* Same numbering as ucx_memory_type_t (ucx_context/ucx_context_def.h:27-39),
 * so values can be passed through unchanged. */
typedef enum axr_memory_type {
  AXR_MEM_HOST = 0,
  AXR_MEM_CUDA = 1,
  AXR_MEM_CUDA_MANAGED = 2,
  AXR_MEM_ROCM = 3,
  AXR_MEM_ROCM_MANAGED = 4,
  AXR_MEM_RDMA = 5,
  AXR_MEM_ZE_HOST = 6,
  AXR_MEM_ZE_DEVICE = 7,
  AXR_MEM_ZE_MANAGED = 8,
  AXR_MEM_UNKNOWN = 9
} axr_memory_type_t;

/* DLPack device type -> memory type and back, the tables of
 * axon/python/src/dlpack_helpers.cpp:82-134 (kDLROCM=10 <-> ROCM,
 * kDLROCMHost=11 <-> ROCM_MANAGED, kDLCPU=1 <-> HOST, kDLCUDA=2 <-> CUDA,
 * kDLCUDAManaged=13 <-> CUDA_MANAGED, kDLOneAPI=14 -> UNKNOWN, else UNKNOWN). */
AXR_API int axr_dl_device_to_memory_type(int32_t dl_device_type);
AXR_API int32_t axr_memory_type_to_dl_device(int memory_type);

/* ----------------------------------------------------------------- tensors */

/* Layout-identical to DLTensor (dlpack.h, v0.8 / v1.x): a binding may pass
 * &managed->dl_tensor copied into an array of these.  `strides` (in elements)
 * may be NULL for a compact row-major tensor, as DLPack allows. */
typedef struct axr_tensor {
  void* data;
  int32_t device_type; /* DLDeviceType: 1 CPU, 10 ROCM, 11 ROCMHost ...        */
  int32_t device_id;
  int32_t ndim;
  uint8_t dtype_code; /* DLDataTypeCode: 0 int, 1 uint, 2 float, 4 bfloat ...  */
  uint8_t dtype_bits;
  uint16_t dtype_lanes;
  int64_t* shape;
  int64_t* strides;
  uint64_t byte_offset;
} axr_tensor_t;

/* Same as ucx_buffer_t (ucx_context/ucx_context_def.h:58-61). */
typedef struct axr_buffer {
  void* data;
  size_t size;
} axr_buffer_t;

/* Bytes a tensor occupies in a bundle: prod(shape) * ceil(bits/8), 0 when
 * ndim == 0, lanes and strides ignored.  Restates CalculateTensorSize
 * (rpc_core/utils/tensor_meta.hpp:91-104).  Negative extents -> AXR_ERR_INVALID. */
AXR_API int axr_tensor_nbytes(const axr_tensor_t* t, uint64_t* nbytes);

/* ------------------------------------------------------------------ device */

AXR_API int axr_device_count(int* count);
AXR_API int axr_device_get(int* device);
AXR_API int axr_device_set(int device);
/* Thread-level activation used by the ROCm UcxAutoDeviceContext: push makes
 * `device` current on the calling thread and returns the previous one in
 * *token; pop restores it.  Replaces cuCtxPushCurrent / cuCtxPopCurrent of
 * ucx_context/cuda/ucx_cuda_context.hpp:55-72. */
AXR_API int axr_device_push(int device, int* token);
AXR_API int axr_device_pop(int token);
AXR_API int axr_device_synchronize(void);
/* Compute units and bytes of device memory of the current device. */
AXR_API int axr_device_info(int* compute_units, uint64_t* total_mem, uint64_t* free_mem);

/* Non-blocking streams of default priority.  A plan drains the streams it ran on
 * before its device tables are released or rewritten (axr_plan_free,
 * axr_plan_bind and friends): a stream made here may be destroyed while such a
 * plan is alive (the plan then waits for the whole device instead); a stream made
 * with hipStreamCreate directly must outlive the plans that ran on it. */
AXR_API int axr_stream_create(void** stream);
AXR_API int axr_stream_destroy(void* stream);
AXR_API int axr_stream_synchronize(void* stream);
/* Make `stream` wait for `event` (hipStreamWaitEvent). */
AXR_API int axr_stream_wait_event(void* stream, void* event);

AXR_API int axr_event_create(void** event);
AXR_API int axr_event_destroy(void* event);
AXR_API int axr_event_record(void* event, void* stream);
AXR_API int axr_event_synchronize(void* event);
/* 1 in *done when the event has completed, 0 when still pending. */
AXR_API int axr_event_query(void* event, int* done);
AXR_API int axr_event_elapsed_ms(void* start, void* stop, float* ms);

/* ------------------------------------------------------------------ memory */

/* allocate / deallocate / memcpy of UcxMemoryResourceManager
 * (ucx_context/ucx_memory_resource.hpp:99-123) for one memory type each:
 * HOST -> malloc'ed pageable memory, ROCM -> device memory from the process
 * default pool (axr_pool_default), ROCM_MANAGED -> pinned, device-visible host
 * memory.  Other types -> AXR_ERR_UNSUPPORTED. */
AXR_API int axr_mem_alloc(int memory_type, size_t bytes, size_t alignment, void** ptr);
AXR_API int axr_mem_free(int memory_type, void* ptr, size_t bytes);
/* Blocking copy between any two of HOST / ROCM / ROCM_MANAGED; the table
 * of ucx_cuda_memory_manager.hpp:62-78 extended with the pinned type.  ROCM to
 * HOST copies of 16 MiB and more go through two pinned staging blocks that up
 * to "host_threads" threads empty (the checkpoint writer's mr.memcpy(HOST, ...),
 * avro_serialization.cpp:478-523): 51 GB/s instead of 18 GB/s for 1 GiB; HOST to
 * ROCM copies of that size are staged the same way. */
AXR_API int axr_memcpy(int dst_type, void* dst, int src_type, const void* src, size_t bytes);
/* Same, enqueued on `stream`; pageable host memory makes it synchronous. */
AXR_API int axr_memcpy_async(int dst_type, void* dst, int src_type, const void* src,
                             size_t bytes, void* stream);
/* Fill `bytes` bytes with `value` on `stream` (fill kernel, safe to capture). */
AXR_API int axr_memset_async(void* dst, int value, size_t bytes, void* stream);

/* ------------------------------------------------------------- device pool */

typedef struct axr_pool axr_pool_t;

/* Called once per slab the pool obtains from hipMalloc / before it returns
 * the slab with hipFree.  The C++ memory resource wires these to
 * ucx_am_context::register_ucx_memory / unregister_ucx_memory
 * (ucx_context/ucx_am_context/ucx_am_context.cpp:1128-1147, ucp_mem_map) so a
 * whole slab is registered once and every allocation carved from it carries
 * the slab's ucp_mem_h. */
typedef int (*axr_register_fn)(void* user, void* addr, size_t length, void** mem_h);
typedef void (*axr_unregister_fn)(void* user, void* mem_h);

/* Pool of device memory on `device`: slabs of at least `slab_bytes` (0 = 256 MiB
 * default), carved at 256-byte granularity, freed blocks coalesced. */
AXR_API int axr_pool_create(int device, size_t slab_bytes, axr_pool_t** pool);
/* Fails with AXR_ERR_BUSY while allocations are outstanding. */
AXR_API int axr_pool_destroy(axr_pool_t* pool);
/* Process-wide pool of the current device, created on first use. */
AXR_API int axr_pool_default(axr_pool_t** pool);
AXR_API int axr_pool_set_registrar(axr_pool_t* pool, axr_register_fn reg,
                                   axr_unregister_fn unreg, void* user);
/* *mem_h (may be NULL) receives the registration handle of the slab the
 * block lies in, NULL when no registrar is installed; it is what goes into
 * ucx_am_data_t::mem_h (ucx_context/ucx_context_def.h:80-93). */
AXR_API int axr_pool_alloc(axr_pool_t* pool, size_t bytes, size_t alignment,
                           void** ptr, void** mem_h);
/* The block is reusable the moment it is freed: nothing orders the free behind work
 * that is still enqueued on a stream (the reference's cudaFree synchronises
 * implicitly, cuda/ucx_cuda_memory_manager.hpp:108-131; a pool must not).  Free a
 * payload only after the launches that touch it have finished: axr_plan_free and
 * axr_plan_bind wait for a plan's launches, so "free the plan, then the payload"
 * is always safe. */
AXR_API int axr_pool_free(axr_pool_t* pool, void* ptr);
/* Return fully free slabs to the driver. */
AXR_API int axr_pool_trim(axr_pool_t* pool);

typedef struct axr_pool_stats {
  uint64_t slabs;
  uint64_t slab_bytes;      /* bytes held from the driver                     */
  uint64_t allocated_bytes; /* bytes handed out (rounded to 256)              */
  uint64_t live_blocks;
  uint64_t peak_bytes;
} axr_pool_stats_t;
AXR_API int axr_pool_get_stats(axr_pool_t* pool, axr_pool_stats_t* stats);

/* ------------------------------------------------------------ bundle plans */

typedef struct axr_plan axr_plan_t;

/* Sender side.  Lays the n tensors out in argument order (the order
 * InvokeContext::add_tensor establishes,
 * axon/python/src/bindings_runtime_helpers.hpp:351-414):
 *   offset[0] = 0, offset[i+1] = align_up(offset[i] + nbytes[i], align).
 * align == 1 is the reference layout: what a contiguous receiver sees after
 * an IOV send (ucx_am_connection_test.cpp:1051-1108) and what
 * UcxBuffer::to_buffer_vec splits (ucx_context_data.hpp:641-665).
 * align must be a power of two <= 4096.  Gap bytes are written as zero by
 * axr_pack.  Tensors may be strided views (strides != NULL, not row-major):
 * they are packed as their C-order element sequence; the reference would
 * ship the first nbytes of storage instead (dlpack_helpers.cpp:776-780).
 * Every tensor must be device-accessible (kDLROCM / kDLROCMHost) or kDLCPU;
 * kDLCPU tensors travel through pinned staging blocks of up to 8 MiB: neighbouring
 * pieces share one device copy per block; axr_pack returns once the host
 * tensors have been read, axr_unpack once they hold their data (the device
 * tensors of the same bundle still complete asynchronously on the stream).
 * The plan copies shapes and strides; `tensors` may be freed on return.
 * `flags` is reserved and must be 0 (AXR_ERR_INVALID otherwise). */
AXR_API int axr_plan_create(const axr_tensor_t* tensors, size_t n, uint32_t align,
                            uint32_t flags, axr_plan_t** plan);
/* Returns when the plan's launches have finished on the streams they were given
 * (launches recorded into a graph excepted), so the payload and the tensors may be
 * released right after it. */
AXR_API int axr_plan_free(axr_plan_t* plan);

AXR_API int axr_plan_num_tensors(const axr_plan_t* plan, size_t* n);
/* Bytes of the packed buffer, gaps included. */
AXR_API int axr_plan_payload_bytes(const axr_plan_t* plan, uint64_t* bytes);
/* Sum of tensor sizes (gaps excluded): the algorithmic payload P. */
AXR_API int axr_plan_data_bytes(const axr_plan_t* plan, uint64_t* bytes);
/* offsets[i], sizes[i] for i < n; either array may be NULL. */
AXR_API int axr_plan_layout(const axr_plan_t* plan, uint64_t* offsets, uint64_t* sizes);
/* Metadata of tensor i with data == NULL, byte_offset == 0 and shape/strides
 * pointing into the plan (valid until axr_plan_free).  On a plan made by
 * axr_plan_from_header strides is NULL: packed tensors are compact. */
AXR_API int axr_plan_tensor_meta(const axr_plan_t* plan, size_t i, axr_tensor_t* meta);

/* Serialised per-tensor header (offset, size, device, dtype, shape) that
 * travels as the AM header next to the payload; it carries the fields of
 * TensorMeta (rpc_core/utils/tensor_meta.hpp:77-82) with byte_offset fixed at
 * 0.  Little-endian, fixed layout, documented in axr_plan.cpp.  The pointer is
 * owned by the plan. */
AXR_API int axr_plan_header(const axr_plan_t* plan, const void** header, size_t* length);

/* Receiver side: rebuild the layout from a received header.  The plan has no
 * tensor addresses until axr_plan_bind. */
AXR_API int axr_plan_from_header(const void* header, size_t length, axr_plan_t** plan);
/* Attach (or replace) the tensor-side addresses: sources for axr_pack,
 * destinations for axr_unpack.  dtype bits and shape of tensors[i] must give
 * the same nbytes and element size as the plan's tensor i; strides may differ
 * (unpack into views).  Overlapping destinations (a stride of 0 on an extent
 * above 1) are refused for unpack. */
AXR_API int axr_plan_bind(axr_plan_t* plan, const axr_tensor_t* tensors, size_t n);
/* axr_plan_from_header followed by axr_plan_bind in one pass over the header's
 * records, for a receiver that has its destination tensors at hand when the
 * header arrives (a memory policy that answers from a cache of buffers,
 * axon/src/axon_worker.cpp:1150-1172).  Same checks and errors as the two calls;
 * *plan is NULL on failure. */
AXR_API int axr_plan_from_header_bind(const void* header, size_t length, const axr_tensor_t* tensors,
                                      size_t n, axr_plan_t** plan);

/* Zero-copy receive mode: views[i] = {payload + offset[i], nbytes[i]}, the
 * result of UcxBuffer::to_buffer_vec(sizes) (ucx_context_data.hpp:641-665).
 * AXR_ERR_LENGTH when the plan needs more than payload_bytes. */
AXR_API int axr_plan_split(const axr_plan_t* plan, void* payload, size_t payload_bytes,
                           axr_buffer_t* views);

/* Gather the bound tensors into payload[0, payload_bytes) / scatter payload
 * into the bound tensors, asynchronously on `stream`.  `payload` must be
 * device-accessible memory; payload_bytes must be >= axr_plan_payload_bytes
 * (AXR_ERR_LENGTH otherwise).  The first call uploads the plan's device
 * tables on the same stream.  A plan may be packed/unpacked any number of
 * times; concurrent calls on one plan from two threads are not allowed. */
AXR_API int axr_pack(axr_plan_t* plan, void* payload, size_t payload_bytes, void* stream);
AXR_API int axr_unpack(axr_plan_t* plan, const void* payload, size_t payload_bytes,
                       void* stream);

/* Builds the plan's device tables, uploads them on `stream` and waits until they
 * are resident.  Afterwards axr_pack / axr_unpack of this plan only launch one
 * kernel (no allocation, no copy, no host wait), so they may be recorded into a
 * HIP graph by stream capture; without it a capturing call fails with
 * AXR_ERR_INVALID, unless the bundle is small enough to carry its tables in the
 * kernel arguments (axr_launch_info.inline_tables; such a launch is recorded
 * whole and the plan may be freed afterwards).  While a graph that holds such a launch can still run, the
 * plan must stay alive and must not be rebound, and the tensors and the payload
 * must stay where they are.  Bundles with kDLCPU tensors cannot be captured
 * (AXR_ERR_UNSUPPORTED).  No counterpart in the reference, whose payload never
 * passes through a kernel. */
AXR_API int axr_plan_prepare(axr_plan_t* plan, void* stream);

/* Several bundles handed over at once.  A worker that has requests to send and
 * responses to receive at the same moment (ClientSendRequest_ next to
 * ProcessRndvBuffer_, axon/src/axon_worker.cpp:1424-1490 and :1098-1219, run by
 * independent coroutines in the reference) submits the gathers and scatters
 * together: neighbouring jobs of one launch geometry share ONE kernel launch
 * (up to sixteen per launch; a short kernel's fixed cost is paid once), the rest run
 * one after the other, all on `stream`.  The jobs of one call must not depend on
 * each other (no job may read what another one writes) and no plan may appear
 * twice; inside a shared launch the gathers take the first workgroups whatever
 * their place in `jobs`.  `tensor_delta` is added to every bound tensor address of that job: a
 * plan bound once serves tensors of the same shapes and strides at another base
 * (the chunks of a streamed transfer) without rebuilding or re-uploading its
 * tables; it must be 0 for bundles with kDLCPU tensors.  Results are those of
 * axr_pack / axr_unpack called job by job. */
typedef struct axr_job {
  axr_plan_t* plan;
  int unpack;            /* 0: gather the tensors into payload; 1: scatter payload */
  void* payload;
  size_t payload_bytes;
  int64_t tensor_delta;
  uint32_t flags;        /* 0, or one AXR_JOB_PAYLOAD_* value                      */
  uint32_t reserved;     /* 0                                                      */
} axr_job_t;
/* Cache treatment of the payload side for this job, overriding the plan's choice
 * (cacheable up to "payload_cache_bytes", so that a consumer that follows at once
 * finds the payload in the last-level cache): STREAMING when more payloads are in
 * flight than that cache holds (the slots of a streamed transfer), CACHED to keep
 * a larger payload cacheable. */
#define AXR_JOB_PAYLOAD_STREAMING 1u
#define AXR_JOB_PAYLOAD_CACHED 2u
AXR_API int axr_submit(const axr_job_t* jobs, size_t n, void* stream);

/* axr_pack for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference (its payload never passes through a kernel).  Same result as
 * axr_pack; the call allocates no device or pinned memory and frees none.  A small
 * bundle carries its tables inside the kernel arguments (as axr_pack's first launch
 * does); a larger one has them copied on `stream` into a table area that is part of
 * the library's device code: 1 MiB per GPU, held until the process ends (about
 * 25,000 contiguous tensors, or 50,000 short ones that share wavefronts;
 * AXR_ERR_LENGTH beyond that).  Every call on one GPU shares that GPU's area: calls
 * on ONE stream are ordered by the stream and may follow each other without a wait; a
 * call on another stream than the area's last user is made to wait, on the device, for
 * that user's launch (an event created once per GPU and recorded behind every launch
 * that reads the area), so calls on two streams are serialised, not refused.  The table
 * copies read the plan's pageable host memory with hipMemcpyAsync; the library allocates
 * nothing for them, the HIP runtime may stage them through buffers of its own.
 * Bundles with kDLCPU tensors (pinned staging) and, under stream capture, bundles whose
 * tables exceed the kernel arguments are refused with AXR_ERR_UNSUPPORTED.  The plan
 * must stay alive until the stream has run the call (axr_plan_free and axr_plan_bind
 * wait for it). */
AXR_API int axr_pack_noalloc(axr_plan_t* plan, void* payload, size_t payload_bytes, void* stream);

/* Launch geometry of a plan's kernel, for profiling reports. */
typedef struct axr_launch_info {
  uint32_t workgroups;
  uint32_t threads_per_workgroup;
  uint32_t tiles;          /* work units the kernel walks                     */
  uint32_t tile_bytes;
  uint32_t segments;       /* device segment-table entries                    */
  uint32_t table_bytes;    /* device table size                               */
  uint32_t host_copies;    /* contiguous pieces of kDLCPU tensors              */
  uint32_t host_chunks;    /* device copies that move them (pinned staging)    */
  uint32_t inline_tables;  /* 1: the next launch carries the tables inside the
                              kernel arguments (small bundle, first launch:
                              no upload, no device block)                      */
  uint32_t reserved;
} axr_launch_info_t;
AXR_API int axr_plan_launch_info(axr_plan_t* plan, axr_launch_info_t* info);

/* One entry of the device segment table, for inspection and tests. */
typedef struct axr_segment_info {
  uint32_t tensor;        /* index of the tensor the segment belongs to       */
  uint32_t mode;          /* 0 one run, 1 strided run tiles, 2 strided
                             elements, 3 zero fill only, 4 host copy,
                             5 transposed blocks (all dims in packed order;
                             the one whose stride equals `granule` is
                             contiguous in the tensor), 6 a short tensor that
                             shares one wavefront's tile with its neighbours
                             (`granule` = its first lane slot in the tile,
                             `lanes_per_run` = the slots it occupies, `tiles`
                             = 1 for the first tensor of a tile, else 0)      */
  uint64_t address;       /* tensor-side address of the first element         */
  uint64_t offset;        /* payload offset                                   */
  uint64_t run_bytes;     /* contiguous bytes per run                         */
  uint64_t nbytes;        /* bytes of the whole segment                       */
  uint32_t pad;           /* zero bytes written after the segment by pack     */
  uint32_t ndim;          /* strided outer dimensions (<= 6)                  */
  uint32_t granule;       /* mode 2: bytes per lane access; mode 5: element   */
  uint32_t tiles;
  uint32_t head;          /* mode 0: leading bytes (< 128) that the first tile
                             moves on top of its own range, so that the tiles
                             start on a 128-byte line of the written side      */
  uint32_t lanes_per_run; /* mode 2 with 16-byte granules: lane slots a run occupies
                             (its granules, the last one covering the run's final 16
                             bytes, rounded up to a multiple of four); 0: the tiles
                             count packed bytes                                  */
  uint32_t shape[6];
  int64_t stride_bytes[6];
} axr_segment_info_t;
/* Copies up to `capacity` entries into out (may be NULL) and stores the total
 * number in *count.  Works without a device (the grid is then sized for 256
 * compute units). */
AXR_API int axr_plan_segments(axr_plan_t* plan, axr_segment_info_t* out, size_t capacity,
                              size_t* count);

/* Tuning knobs (process-wide, read when a plan builds its device tables):
 * "tile_rows" (KiB per wavefront tile: 1, 2, 4, 8, 16, or 0 = automatic: 2; a whole run of up
 * to 16 KiB for bundles of strided views of one run length whose payload stays in the
 * last-level cache; 1 for payloads of compact tensors and long strided runs between
 * payload_cache_bytes and max_tiles KiB, which stream to and from memory), "max_tiles",
 * "max_waves", "threads" (workgroup size; 0 = automatic: 256 below 65,536 tiles, 128 above, 64
 * with the automatic 1 KiB tiles and for short strided rows that are no multiple of 16
 * bytes), "nontemporal" (-1 auto, or bit 0
 * tensor side / bit 1 payload side), "payload_cache_bytes", "gather_run_bytes",
 * "xcd_remap" (each accelerator die walks one contiguous share of the tiles: 1 always,
 * 0 never, -1 (default) for bundles made mostly of transposed views whose rows do not
 * start on 128-byte lines, where neighbouring blocks then meet in one L2),
 * "transpose" (1: transposed views move as square blocks through
 * LDS; 0: element by element), "ragged_runs" (1: short strided runs whose
 * length is no multiple of 16 bytes still move in 16-byte granules),
 * "head_align" (contiguous tensors longer than a tile start their tiles on a
 * multiple of this many bytes of the written side - the payload for a plan made
 * by axr_plan_create, the tensor for one made by axr_plan_from_header; a power
 * of two up to 128, default 16, 0: off),
 * "host_threads" (threads, the caller included, that share the host-side copies
 * between pageable memory and the pinned staging blocks once a copy is 2 MiB or
 * more; default 4, 1: the calling thread alone),
 * "spin_wait_us" (0, the default: axr_stream_synchronize is hipStreamSynchronize.  N > 0: it
 * first enqueues a one-wave kernel behind the stream's work that writes a word of pinned
 * memory, polls that word for up to N microseconds, and only then falls back to
 * hipStreamSynchronize.  The poll sees the end of a short kernel about 5 us before the
 * runtime's completion signal wakes the caller: a fresh bundle of four tensors makes its
 * round trip in 24 us instead of 30.  For latency-bound callers whose kernels write device
 * memory or coherent pinned memory only: what a kernel has written to NON-coherent host
 * memory is made visible to the CPU by the completion the runtime waits for, which this
 * wait returns ahead of.  Never used on a capturing stream),
 * "device_tables" (a bundle of at least this many tensors, all contiguous device
 * tensors, takes a short path to its device tables: one pass over the tensors into
 * pinned memory and a kernel that brings the records to the device and writes the
 * tile-block index, instead of the general host build plus an upload; default 512,
 * 0: never),
 * "loopback_copy_kernel" (1, default: the loopback context moves a device payload
 * to device memory with the library's copy kernel; 0: with hipMemcpyAsync),
 * "group_bytes" (contiguous device tensors of at most this many bytes that follow each
 * other in the bundle share wavefronts: up to 16 tensors or 128 sixteen-byte lane slots
 * per wavefront, so that wavefronts and table bytes scale with the payload and not with
 * the tensor count; default 512, at most 1023, 0: every tensor gets wavefronts of its own),
 * "submit_interleave" (1, the default: the two jobs of an axr_submit launch of two jobs with equal
 * grids and payloads larger than payload_cache_bytes take the workgroups in turn instead of one
 * range each; 2: also smaller payloads that stream; 0: never; read at every axr_submit),
 * "transfer_fail_after_send" (failure injection for tests: N > 0 makes the N-th chunk that
 * axr_transfer_submit is given from now on fail with AXR_ERR_MISMATCH after its send has been
 * queued, as if the message that arrived did not match the receiver's plan; 0, the default: off),
 * "inline_tables" (the first launch of a bundle of at most this many tiles
 * whose tables fit into 3.5 KiB carries the tables inside the kernel arguments:
 * no table block and no upload; a plan that is launched again uploads its
 * tables then; 0 switches that off; read at every
 * axr_pack / axr_unpack).  Unknown key -> AXR_ERR_INVALID. */
AXR_API int axr_tune_set(const char* key, int64_t value);
AXR_API int axr_tune_get(const char* key, int64_t* value);

/* ------------------------------------------------ loopback active messages */

/* In-process stand-in for the reference's ucx_am_context, for machines without
 * UCX: two contexts in one process joined by a loopback endpoint, the topology
 * of test_code/test_cuda_connection.cpp:256-297.  It keeps the observable
 * behaviour of connection_send / connection_recv_header / connection_recv_buffer
 * (ucx_context/ucx_context_concept.hpp:247-470):
 *   - a send needs a non-empty header; the payload may be empty
 *     (ucx_am_context.hpp:2275-2284);
 *   - a contiguous payload below the zcopy threshold (UCX_ZCOPY_THRESH, default
 *     4096; ucx_connection.cpp:45,113-124) is eager: header and payload are copied
 *     to host memory at send time and the send is complete; otherwise, and always
 *     for an iov payload (ucx_connection.cpp:417-419), it is a rendezvous: only
 *     the header is copied, the receiver fetches the payload with
 *     axr_am_recv_buffer*, and the send completes then;
 *   - messages are delivered in FIFO order per receiving context;
 *   - an iov payload received into a contiguous buffer is the concatenation of
 *     its entries in order (ucx_am_connection_test.cpp:1051-1108).
 * Payload bytes move with device copies on `stream` (one per iov entry), which
 * is also what UCX's rocm_copy transport would do for the reference's iov send. */

typedef struct axr_am_context axr_am_context_t;

/* == ucx_am_data_t / ucx_am_iovec_t (ucx_context/ucx_context_def.h:80-129) */
typedef struct axr_am_data {
  axr_buffer_t header;
  axr_buffer_t buffer;
  int buffer_type;   /* axr_memory_type_t */
  void* mem_h;
} axr_am_data_t;
typedef struct axr_am_iovec {
  axr_buffer_t header;
  axr_buffer_t* buffer_vec;
  size_t buffer_count;
  int buffer_type;
  void* mem_h;
} axr_am_iovec_t;

/* What connection_recv_header yields: for a rendezvous message the key under
 * which the payload is parked, for an eager one the payload itself (host
 * memory).  header / eager_data stay valid until axr_am_message_release. */
typedef struct axr_am_message {
  uint64_t key;
  uint64_t conn_id;       /* reply connection, learned from the sender        */
  axr_buffer_t header;    /* host copy of the AM header                       */
  uint64_t data_length;
  int is_rndv;
  int buffer_type;        /* memory type of the sender's payload              */
  axr_buffer_t eager_data;
} axr_am_message_t;

/* zcopy_thresh 0 reads UCX_ZCOPY_THRESH, else 4096. */
AXR_API int axr_am_context_create(const char* name, size_t zcopy_thresh, axr_am_context_t** ctx);
AXR_API int axr_am_context_destroy(axr_am_context_t* ctx);
/* Endpoint from `from` to `to`; *conn_id names it in axr_am_send*.  Sending on it
 * after `to` has been destroyed fails with AXR_ERR_INVALID. */
AXR_API int axr_am_connect(axr_am_context_t* from, axr_am_context_t* to, uint64_t* conn_id);
/* *request identifies the send for axr_am_request_test. */
AXR_API int axr_am_send(axr_am_context_t* ctx, uint64_t conn_id, const axr_am_data_t* data,
                        void* stream, uint64_t* request);
AXR_API int axr_am_send_iov(axr_am_context_t* ctx, uint64_t conn_id, const axr_am_iovec_t* data,
                            void* stream, uint64_t* request);
/* *done: 0 pending, 1 complete, -1 cancelled or failed. */
AXR_API int axr_am_request_test(axr_am_context_t* ctx, uint64_t request, int* done);
/* Cancel a send that has not completed (the sender-side stop request of the reference's
 * send operation, ucx_am_context.hpp:2234-2642): a send that still waits for room is
 * dropped, a rendezvous that the receiver has not fetched disappears from its queue (a
 * fetch under way elsewhere fails with AXR_ERR_CANCELED); the request then tests as -1.
 * A completed send is left as it is. */
AXR_API int axr_am_request_cancel(axr_am_context_t* ctx, uint64_t request);
/* A context admits 256 sends that have started and not completed (rendezvous sends whose
 * payload has not been fetched), the reference's kCompletionQueueEntryCount
 * (ucx_am_context.hpp:94,836-839).  Further sends are accepted, wait in order, and start as
 * completions make room (ucx_am_context.cpp:271-274); eager sends behind them wait too, so
 * the order of delivery is the order of the calls.  Completions are noticed inside
 * axr_am_send*, axr_am_request_test, axr_am_request_cancel and here.  Either result may be
 * NULL. */
AXR_API int axr_am_progress(axr_am_context_t* ctx, size_t* in_flight, size_t* waiting);
/* Next message in arrival order; AXR_ERR_NO_MESSAGE when none is queued. */
AXR_API int axr_am_recv_header(axr_am_context_t* ctx, axr_am_message_t* message);
/* Fetch a rendezvous payload into one contiguous buffer of memory type
 * dst_type (blocking on `stream`).  Unknown key -> AXR_ERR_NO_MESSAGE; eager
 * message -> AXR_ERR_NOT_IMPLEMENTED (ucx_am_context.hpp:1570-1574, 1643-1651);
 * dst_bytes below data_length -> AXR_ERR_LENGTH. */
AXR_API int axr_am_recv_buffer(axr_am_context_t* ctx, uint64_t key, int dst_type, void* dst,
                               size_t dst_bytes, void* stream);
/* Same, but only enqueues the copies on `stream`: the data is in place for work
 * ordered after them on that stream, and the sender's request completes when
 * they have run (for pipelines that must not block the host). */
AXR_API int axr_am_recv_buffer_async(axr_am_context_t* ctx, uint64_t key, int dst_type, void* dst,
                                     size_t dst_bytes, void* stream);
/* Same into an iov: entries must be non-null and non-empty and add up to at
 * least data_length (ucx_am_context.hpp:1808-1818); filled in order. */
AXR_API int axr_am_recv_buffer_iov(axr_am_context_t* ctx, uint64_t key, int dst_type,
                                   const axr_buffer_t* buffer_vec, size_t buffer_count,
                                   void* stream);
/* Zero-copy fetch of a rendezvous payload (in place of the ucp_am_recv_data_nbx of
 * ucx_connection.cpp:376-399, which copies into the receiver's buffer): the receiver is handed the
 * sender's buffer (what a same-process rocm_ipc zero-copy rendezvous gives two endpoints
 * that share a device: UCX maps the sender's registered memory and the "receive" is a
 * pointer).  Only for a message whose payload is ONE contiguous buffer in memory the
 * receiver can address (ROCM, ROCM_MANAGED or HOST of the same process); an iov message ->
 * AXR_ERR_UNSUPPORTED (fetch it with axr_am_recv_buffer*).  Unknown key ->
 * AXR_ERR_NO_MESSAGE, eager message -> AXR_ERR_NOT_IMPLEMENTED, cancelled by the sender ->
 * AXR_ERR_CANCELED.  On success the message is claimed (the sender can no longer cancel),
 * *data / *bytes / *memory_type describe the sender's buffer, and the send stays incomplete
 * until axr_am_borrow_release: the sender must not touch the buffer before its request
 * tests complete, exactly as for a copying fetch that is still running. */
AXR_API int axr_am_recv_buffer_borrow(axr_am_context_t* ctx, uint64_t key, void** data, size_t* bytes,
                                      int* memory_type);
/* The receiver has enqueued its last read of a borrowed buffer on `stream`: the sender's
 * request completes when the work that `stream` holds now has run (no host wait).  Unknown
 * key -> AXR_ERR_NO_MESSAGE.  A receiving context that is destroyed with borrows not yet
 * released completes those sends at once: drain whatever still reads the borrowed buffers
 * before destroying the context. */
AXR_API int axr_am_borrow_release(axr_am_context_t* ctx, uint64_t key, void* stream);
/* Drop a message's host copies (and, for an unfetched rendezvous, complete the
 * sender's request as cancelled). */
AXR_API int axr_am_message_release(axr_am_context_t* ctx, uint64_t key);
/* What axr_am_recv_header said about a message that is still parked (a rendezvous whose
 * payload has not been fetched, an eager message not yet released): its payload length,
 * the reply connection and whether it is a rendezvous.  Any result may be NULL.  Unknown
 * key -> AXR_ERR_NO_MESSAGE.  The receive-buffer operation of the reference learns the
 * length the same way, from the parked descriptor (ucx_am_context.hpp:1568-1621). */
AXR_API int axr_am_message_info(axr_am_context_t* ctx, uint64_t key, uint64_t* data_length,
                                uint64_t* conn_id, int* is_rndv);
/* Messages queued and not yet taken by axr_am_recv_header. */
AXR_API int axr_am_pending(axr_am_context_t* ctx, size_t* count);

/* ------------------------------------------------------------- UCX, probed */

/* What a real UCX backend needs from the machine, found at run time: the reference links
 * OpenUCX at build time (ucp_init / ucp_worker_create, ucx_am_context.cpp:694-749; ucp_mem_map,
 * :1128-1147; ucp_am_send_nbx and ucp_am_recv_data_nbx, ucx_connection.cpp:353-453;
 * ucp_worker_progress, ucx_am_context.cpp:218-296).  This library looks for libucp.so.0
 * (or the file named by the environment variable AXR_UCX_LIBRARY) with dlopen, resolves those
 * entry points and reads the version.  It calls nothing else: the parameter structures of the
 * UCX calls come from ucp.h, which this build was made without. */
#define AXR_UCX_SYMBOLS 6
typedef struct axr_ucx_probe {
  int available;                      /* 1: the library loaded and every entry point is there */
  unsigned version_major, version_minor, version_release;   /* ucp_get_version, 0 when unknown */
  int have_symbol[AXR_UCX_SYMBOLS];   /* in the order of axr_ucx_symbol_name */
  char library[256];                  /* the name dlopen accepted, "" when none */
  char message[512];                  /* one line for a log */
} axr_ucx_probe_t;
/* Probes once per process; later calls return the first result. */
AXR_API int axr_ucx_probe(axr_ucx_probe_t* probe);
AXR_API const char* axr_ucx_symbol_name(int index);
/* The UCX-backed counterpart of axr_am_context_create.  Always AXR_ERR_UNSUPPORTED in this
 * build, with a message that says which of the two things is missing: the UCX library on
 * this machine, or (when it is there) the UCX headers at build time.  *ctx is NULL. */
AXR_API int axr_am_context_create_ucx(const char* name, axr_am_context_t** ctx);

/* ------------------------------------------------------- streamed transfers */

/* A large payload moved in chunks: pack -> connection_send -> connection_recv_buffer
 * -> unpack per chunk (ucx_am_context.hpp:2234-2642 for the send, :1511-1844 for the
 * receive), double-buffered: `lanes` lanes (2 is the classic double buffer), each a
 * send slot and a receive slot of slot_bytes from `pool` (NULL: the default pool),
 * over `streams` streams (1 <= streams <= lanes).  Chunk k uses lane k % lanes on
 * stream (k % lanes) % streams.  streams == lanes: while chunk k is on the wire and
 * being scattered, chunk k + 1 is gathered on the other stream.  streams == 1: the
 * chunks run back to back on one stream and the second lane only lets the host queue
 * one chunk ahead; on one GPU, where gather, wire copy and scatter all compete for
 * the same HBM, this is the faster arrangement.  The transport is a loopback context
 * pair inside the object: every chunk with a payload is a rendezvous whose fetch is
 * either a borrow of the send slot (the default) or a stream-ordered device copy from
 * the send slot to a receive slot (axr_transfer_set_zero_copy).
 *
 * The caller keeps ONE sender plan and ONE receiver plan (axr_plan_from_header of
 * the sender's header, bound to the destination tensors) for all chunks of one
 * geometry; send_delta / recv_delta say how far this chunk's tensors lie from the
 * ones the plans are bound to (see axr_job_t.tensor_delta).  axr_transfer_submit
 * never plans, uploads or allocates (after each plan's first use); it waits on the
 * host only for the chunk that used the lane last.  AXR_ERR_MISMATCH when the
 * receiver's plan does not describe the sender's header, AXR_ERR_LENGTH when a
 * chunk exceeds a slot.  One thread at a time per transfer. */
typedef struct axr_transfer axr_transfer_t;
AXR_API int axr_transfer_create(axr_pool_t* pool, size_t slot_bytes, int lanes, int streams,
                                axr_transfer_t** transfer);
AXR_API int axr_transfer_submit(axr_transfer_t* transfer, axr_plan_t* send_plan, int64_t send_delta,
                                axr_plan_t* recv_plan, int64_t recv_delta);
/* How a chunk crosses the loopback wire.  1 (the default): the receiver borrows the sender's
 * slot (axr_am_recv_buffer_borrow) and unpacks straight out of it, the send completing after
 * the unpack: 4P bytes per chunk, what a zero-copy rendezvous between two endpoints on one
 * device costs.  0: the payload is copied from the send slot to a receive slot first
 * (axr_am_recv_buffer_async), 6P bytes per chunk, what a transport that stages through its
 * own buffers costs.  Call between chunks only (AXR_ERR_BUSY while chunks are in flight). */
AXR_API int axr_transfer_set_zero_copy(axr_transfer_t* transfer, int enable);
/* Returns when every submitted chunk has arrived in its destination tensors. */
AXR_API int axr_transfer_finish(axr_transfer_t* transfer);
/* Finishes, then releases the slots, streams and contexts. */
AXR_API int axr_transfer_destroy(axr_transfer_t* transfer);

/* -------------------------------------------------- verification utilities */

/* data[i] /= 2.0f in place; the device-side "process" step of the reference's
 * send -> process -> reply tests
 * (ucx_am_context/ucx_am_context_test_cuda_helper.cu:23-78). */
AXR_API int axr_divide_by_two(float* data, size_t count, void* stream);
/* Number of differing bytes between two device-accessible ranges (blocking). */
AXR_API int axr_compare(const void* a, const void* b, size_t bytes, uint64_t* mismatches);
/* Position-weighted checksum: sum over bytes b[i] * (1 + ((start + i) mod 65521))
 * mod 2^64 (blocking).  Additive over a split of the range, so the checksum of
 * a packed buffer equals the sum of its tensors' checksums taken with
 * start = offset[i]. */
AXR_API int axr_checksum(const void* data, size_t bytes, uint64_t start, uint64_t* sum);
/* --------------------------------------------------------------- calibration */

/* The entry points below are NOT part of the drop-in surface: nothing of the reference
 * corresponds to them and no caller of the bundle path needs them.  They are the yardsticks
 * the measurements are read against (what a plain copy, and a plain gather of equal rows,
 * reach on the same device), kept in the library so that they run with the same compiler
 * flags, streams and timing harness as the kernels they calibrate. */

/* Plain device copy kernel (16 B per lane, grid-stride); calibration
 * reference for profiler counters and bandwidth. */
AXR_API int axr_copy_reference(void* dst, const void* src, size_t bytes, void* stream);

/* Plain device copy in the shape of the bundle kernels' wavefronts: workgroups of `threads`
 * threads (a multiple of 64 up to 1024), every wavefront moving kib_per_wave KiB (1, 2 or 4:
 * that many 16-byte loads per lane, issued before the stores), streaming accesses when
 * nontemporal != 0.  `bytes` must be a whole number of wavefront tiles.  No tables and no
 * segments: the ceiling of a wavefront shape on this device, next to which the bundle
 * kernels' rates are read. */
AXR_API int axr_copy_reference_shaped(void* dst, const void* src, size_t bytes, uint32_t threads,
                                      uint32_t kib_per_wave, int nontemporal, void* stream);

/* Plain gather (scatter == 0) or scatter of `rows` rows of run_bytes bytes that lie
 * `pitch` bytes apart at `strided` and back to back at `packed`: one 16-byte access per
 * lane, no tables, nothing decoded beyond a division.  Calibration reference for what the
 * access pattern of a strided view allows (rows that cover parts of 128-byte lines cost
 * whole lines when read and partial-line writes when written), next to which the bundle
 * kernel's element mode is judged.  16 <= run_bytes <= 4096, pitch >= run_bytes;
 * `nontemporal` bit 0 marks the strided side's accesses as streaming, bit 1 the packed
 * side's.  No counterpart in the reference. */
AXR_API int axr_rows_reference(void* strided, size_t pitch, void* packed, size_t run_bytes,
                               size_t rows, int scatter, uint32_t nontemporal, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AXON_ROCM_H_ */
