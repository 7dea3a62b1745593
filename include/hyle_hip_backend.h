/*
 * hyle_hip_backend.h -- C ABI of the MI355X backend under the compute provider of
 * hyle_hip.h: devices, memory resources, queues, sequences with completions, and
 * queue-ordered copy and fill.  It is the twin of the reference's private backend
 * contract, struct BackendVTable (src/compute/backend_internal.h:14-67), which its
 * CUDA backend fills in src/compute_backend_cuda/cuda_backend.cc; each function
 * below names the member it stands for, so that an adapter inside the reference can wrap
 * these calls member for member.
 *
 * One queue owns or borrows one HIP stream of default priority.  Nothing here
 * blocks except the functions whose names say wait or drain.
 */
#ifndef HYLE_HIP_BACKEND_H_
#define HYLE_HIP_BACKEND_H_

#include "hyle_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* DeviceProperties (include/hyle/compute/device.h) of one HIP device. */
typedef struct hyle_hip_device_properties {
  int32_t ordinal;
  int32_t compute_units;
  uint64_t total_memory_bytes;
  uint32_t unified_memory;       /* 0: device and host memory are separate resources */
  uint32_t asynchronous_queues;  /* 1 */
  char name[128];
  char architecture[64];         /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
} hyle_hip_device_properties;

/* BackendVTable::device_count (cuda_backend.cc:790-799). */
HYLE_HIP_API hyle_hip_status hyle_hip_backend_device_count(size_t *count);
/* BackendVTable::device + properties (cuda_backend.cc:808-823). */
HYLE_HIP_API hyle_hip_status hyle_hip_backend_device_properties(size_t index,
                                                                hyle_hip_device_properties *properties);

/* BackendVTable::same_device (src/compute_backend_cuda/cuda_backend.cc:803-806): 1 when both
 * indices name an existing device and it is the same one (a device is its ordinal), else 0. */
HYLE_HIP_API int hyle_hip_backend_same_device(size_t left, size_t right);

/* ---- memory resources (include/hyle/mem/resource.h:108-151) ------------------------- */
/* MemoryProperty bits (include/hyle/mem/resource.h:19-33). */
enum {
  HYLE_HIP_MEMORY_HOST_ACCESSIBLE = 1u << 0,
  HYLE_HIP_MEMORY_DEVICE_ACCESSIBLE = 1u << 1,
  HYLE_HIP_MEMORY_HOST_DEVICE_COHERENT = 1u << 2,
  HYLE_HIP_MEMORY_HOST_PINNED = 1u << 3,
  HYLE_HIP_MEMORY_HOST_ADDRESS_IDENTITY = 1u << 7
};
/* MemoryKind of the CUDA backend's resources (src/compute_backend_cuda/cuda_memory.cc). */
enum { HYLE_HIP_MEMORY_KIND_DEVICE = 0, HYLE_HIP_MEMORY_KIND_PINNED_HOST = 1 };

typedef struct hyle_hip_memory_properties {
  uint32_t flags;            /* HYLE_HIP_MEMORY_* */
  uint32_t kind;             /* HYLE_HIP_MEMORY_KIND_* */
  size_t minimum_alignment;  /* every allocation is at least this aligned */
  size_t maximum_allocation;
} hyle_hip_memory_properties;

/* ResourceStats (include/hyle/mem/resource.h:76-84). */
typedef struct hyle_hip_memory_stats {
  size_t used_bytes, peak_bytes;
  uint64_t live_allocations, total_allocations;
} hyle_hip_memory_stats;

typedef struct hyle_hip_memory_resource hyle_hip_memory_resource;

/* A resource bound to the context's device: device memory (kDeviceAccessible) or
 * pinned host memory (kHostAccessible | kDeviceAccessible | kHostDeviceCoherent |
 * kHostPinned | kHostAddressIdentity).  Pinned memory is allocated as such; memory
 * that already exists cannot be registered. */
HYLE_HIP_API hyle_hip_status hyle_hip_memory_resource_create(hyle_hip_context *context, uint32_t kind,
                                                             hyle_hip_memory_resource **resource);
/* Frees whatever is still allocated. */
HYLE_HIP_API void hyle_hip_memory_resource_destroy(hyle_hip_memory_resource *resource);
/* MemoryResource::properties. */
HYLE_HIP_API hyle_hip_status hyle_hip_memory_resource_properties(const hyle_hip_memory_resource *resource,
                                                                 hyle_hip_memory_properties *properties);
/* MemoryResource::allocate / deallocate.  `alignment` is a power of two; a zero size
 * is INVALID_ARGUMENT, no memory RESOURCE_EXHAUSTED. */
HYLE_HIP_API hyle_hip_status hyle_hip_memory_allocate(hyle_hip_memory_resource *resource, size_t size,
                                                      size_t alignment, void **address);
HYLE_HIP_API hyle_hip_status hyle_hip_memory_deallocate(hyle_hip_memory_resource *resource, void *address);
/* MemoryResource::stats. */
HYLE_HIP_API hyle_hip_status hyle_hip_memory_resource_stats(const hyle_hip_memory_resource *resource,
                                                            hyle_hip_memory_stats *stats);
/* BackendVTable::validate_resource (cuda_backend.cc:825-838): OK when the resource
 * belongs to the context's device, FAILED_PRECONDITION otherwise. */
HYLE_HIP_API hyle_hip_status hyle_hip_backend_validate_resource(const hyle_hip_context *context,
                                                                const hyle_hip_memory_resource *resource);

/* ---- queues, sequences, completions --------------------------------------------------- */
typedef struct hyle_hip_queue hyle_hip_queue;
typedef struct hyle_hip_sequence hyle_hip_sequence;
typedef struct hyle_hip_completion hyle_hip_completion;

/* BackendVTable::create_queue / destroy_queue (cuda_backend.cc:950-997).  `stream` is a
 * hipStream_t the queue borrows, or NULL for a stream of its own (non-blocking, default
 * priority).  Destroying a queue drains it first. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_create(hyle_hip_context *context, void *stream,
                                                   hyle_hip_queue **queue);
HYLE_HIP_API void hyle_hip_queue_destroy(hyle_hip_queue *queue);
/* cuda::stream(sequence) (include/hyle/compute/backends/cuda.h:106-110): the hipStream_t
 * providers enqueue on, e.g. the `stream` argument of hyle_hip_plan_launch. */
HYLE_HIP_API void *hyle_hip_queue_stream(const hyle_hip_queue *queue);
/* BackendVTable::reserve_completions (cuda_backend.cc:1091-1093): make sure `minimum`
 * completions can be in flight without any allocation in begin / finish. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_reserve_completions(hyle_hip_queue *queue, size_t minimum);
/* BackendVTable::begin_sequence (cuda_backend.cc:1029-1042): reserves everything finish
 * needs.  One sequence per queue at a time (FAILED_PRECONDITION otherwise). */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_begin_sequence(hyle_hip_queue *queue, hyle_hip_sequence **sequence);
/* BackendVTable::finish_sequence (cuda_backend.cc:1044-1089).  `accepted` = some command
 * of the sequence was enqueued: the completion then finishes when the queue reaches this
 * point and reports `terminal` if that is an error; otherwise it is complete at once
 * with `terminal`.  A completion is always returned for the queue's active sequence
 * (NULL only for a sequence that is not). */
HYLE_HIP_API hyle_hip_completion *hyle_hip_queue_finish_sequence(hyle_hip_queue *queue,
                                                                hyle_hip_sequence *sequence, int accepted,
                                                                hyle_hip_status terminal);
/* Completion::poll / wait (include/hyle/compute/completion.h): *done = 1 once finished;
 * the returned status is the completion's terminal status (OK while still pending). */
HYLE_HIP_API hyle_hip_status hyle_hip_completion_poll(hyle_hip_completion *completion, int *done);
HYLE_HIP_API hyle_hip_status hyle_hip_completion_wait(hyle_hip_completion *completion);
/* Returns the completion to its queue.  A pending one is waited for first. */
HYLE_HIP_API void hyle_hip_completion_release(hyle_hip_completion *completion);
/* BackendVTable::wait_completion (cuda_backend.cc:1155-1213): work enqueued on `queue`
 * after this call starts only once `completion` (of any queue of the same device) has
 * finished.  The host does not wait. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_wait_completion(hyle_hip_queue *queue,
                                                            hyle_hip_completion *completion);

/* TransferMode / TransferProperties (include/hyle/compute/transfer.h:19-30). */
enum { HYLE_HIP_TRANSFER_IMMEDIATE = 0, HYLE_HIP_TRANSFER_QUEUED_DIRECT = 1 };
typedef struct hyle_hip_transfer_properties {
  uint32_t mode; /* HYLE_HIP_TRANSFER_* */
  uint32_t peer; /* always 0: one device */
} hyle_hip_transfer_properties;
/* BackendVTable::transfer_properties (cuda_backend.cc:1100-1115): the route a copy between two
 * resources would take on `queue`, asked cold before the copies are enqueued.  Storage of the
 * queue's own device -- device memory or pinned host memory, on either side -- travels as one
 * stream-ordered copy (QUEUED_DIRECT, no peer).  Anything else is UNIMPLEMENTED: no hidden
 * staging and no host wait is passed off as an asynchronous copy.  The same admission as
 * hyle_hip_queue_copy_async. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_transfer_properties(const hyle_hip_queue *queue,
                                                                const hyle_hip_memory_resource *destination,
                                                                const hyle_hip_memory_resource *source,
                                                                hyle_hip_transfer_properties *properties);

/* CompletionEndpoint (include/hyle/compute/completion.h; src/compute/backend_internal.h:54-62):
 * who emits a queue's completions.  `authority` is one address for every queue of this library,
 * `identity` the queue: equal endpoints are one ordered queue, not merely queues whose events can
 * meet. */
typedef struct hyle_hip_completion_endpoint {
  const void *authority;
  const void *identity;
} hyle_hip_completion_endpoint;
/* BackendVTable::completion_endpoint (cuda_backend.cc:1214-1226): cold; a null queue gives the
 * invalid endpoint {NULL, NULL}. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_completion_endpoint(const hyle_hip_queue *queue,
                                                                hyle_hip_completion_endpoint *endpoint);
/* BackendVTable::can_wait_endpoint (cuda_backend.cc:1228-1239): 1 commits
 * hyle_hip_queue_wait_completion on `destination` to accepting a pending completion emitted by
 * `source` without a host wait (a queue of this library on the same device); 0 -- another
 * library's endpoint, an invalid one, another device -- leaves the caller to wait on the host. */
HYLE_HIP_API int hyle_hip_queue_can_wait_endpoint(const hyle_hip_queue *destination,
                                                  hyle_hip_completion_endpoint source);

/* BackendVTable::copy_async (cuda_backend.cc:1117-1135): `bytes` from `source` (inside an
 * allocation of `source_resource`) to `destination` (inside one of
 * `destination_resource`), ordered on the queue.  Both resources must belong to the
 * queue's device: anything else is UNIMPLEMENTED and nothing is enqueued
 * (EnqueueResult::rejected); a range outside a live allocation is OUT_OF_RANGE. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_copy_async(hyle_hip_queue *queue,
                                                       hyle_hip_memory_resource *destination_resource,
                                                       void *destination,
                                                       hyle_hip_memory_resource *source_resource,
                                                       const void *source, size_t bytes);
/* BackendVTable::fill_async (cuda_backend.cc:1137-1153): device memory only (pinned host
 * memory is UNIMPLEMENTED, as in the reference).  Done by a small kernel, so the call may
 * be captured into a HIP graph. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_fill_async(hyle_hip_queue *queue,
                                                       hyle_hip_memory_resource *destination_resource,
                                                       void *destination, uint8_t value, size_t bytes);
/* BackendVTable::drain_queue / drain_context: block until the queue's stream, or every
 * stream of the context's device, is idle. */
HYLE_HIP_API hyle_hip_status hyle_hip_queue_drain(hyle_hip_queue *queue);
HYLE_HIP_API hyle_hip_status hyle_hip_context_drain(hyle_hip_context *context);

#ifdef __cplusplus
}
#endif
#endif /* HYLE_HIP_BACKEND_H_ */
