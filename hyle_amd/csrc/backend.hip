// backend.hip -- the C ABI of include/hyle_hip_backend.h: the members of the reference's
// BackendVTable (src/compute/backend_internal.h:14-67) over the HIP runtime: device enumeration,
// memory resources, queues (one HIP stream each), sequences that end in event completions, and
// queue-ordered copy and fill.  Host code, plus the one fill kernel.
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/hyle_hip_backend.h"

struct hyle_hip_context;
namespace hyle_hip {
int context_device(const hyle_hip_context *context);
int record_error(int status, const char *text);
}  // namespace hyle_hip

namespace {

hyle_hip_status fail(hyle_hip_status status, const char *format, ...) {
  char text[320];
  va_list args;
  va_start(args, format);
  vsnprintf(text, sizeof text, format, args);
  va_end(args);
  return static_cast<hyle_hip_status>(hyle_hip::record_error(status, text));
}
hyle_hip_status hip_fail(hipError_t error, const char *what) {
  return fail(error == hipErrorOutOfMemory ? HYLE_HIP_RESOURCE_EXHAUSTED : HYLE_HIP_INTERNAL, "%s: %s", what,
              hipGetErrorString(error));
}

// Keeps the calling thread's current device as it found it.
struct DeviceScope {
  int previous = -1;
  hipError_t error = hipSuccess;
  explicit DeviceScope(int device) {
    error = hipGetDevice(&previous);
    if (error == hipSuccess && previous != device) error = hipSetDevice(device);
    else if (error == hipSuccess) previous = -1;
  }
  ~DeviceScope() {
    if (previous >= 0) (void)hipSetDevice(previous);
  }
};

// Bytes set to one value: 16-byte stores over the aligned middle, single bytes at the ends.
__global__ __launch_bounds__(256) void fill_bytes(unsigned char *destination, size_t bytes, uint32_t value4) {
  const size_t head = ((16 - (reinterpret_cast<uintptr_t>(destination) & 15u)) & 15u) < bytes
                          ? ((16 - (reinterpret_cast<uintptr_t>(destination) & 15u)) & 15u)
                          : bytes;
  const size_t vectors = (bytes - head) / 16;
  const size_t tail_first = head + vectors * 16;
  const size_t thread = (size_t)blockIdx.x * blockDim.x + threadIdx.x, threads = (size_t)gridDim.x * blockDim.x;
  uint4 *middle = reinterpret_cast<uint4 *>(destination + head);
  const uint4 word = make_uint4(value4, value4, value4, value4);
  for (size_t v = thread; v < vectors; v += threads) middle[v] = word;
  if (thread < head) destination[thread] = (unsigned char)value4;
  if (thread < bytes - tail_first) destination[tail_first + thread] = (unsigned char)value4;
}

struct Allocation {
  void *base;  // what the runtime returned
  size_t bytes;
};

}  // namespace

struct hyle_hip_memory_resource {
  int device = 0;
  uint32_t kind = 0;
  mutable std::mutex mutex;
  std::map<uintptr_t, Allocation> live;  // by the (aligned) address handed out
  size_t used = 0, peak = 0;
  uint64_t total = 0;
  // the allocation that holds [address, address + bytes), if any
  bool holds(const void *address, size_t bytes) const {
    std::lock_guard<std::mutex> lock(mutex);
    const uintptr_t at = reinterpret_cast<uintptr_t>(address);
    auto next = live.upper_bound(at);
    if (next == live.begin()) return false;
    --next;
    return at >= next->first && bytes <= next->second.bytes && at - next->first <= next->second.bytes - bytes;
  }
};

struct hyle_hip_completion {
  hyle_hip_queue *owner = nullptr;
  hipEvent_t event = nullptr;
  // A completion may be polled and waited for from any thread (the reference's Completion is
  // pollable from any thread): its state moves through atomics, never through plain fields.
  std::atomic<bool> pending{false};  // the event was recorded and has not been seen finished
  bool in_use = false;               // handed out by begin_sequence / finish_sequence, not yet released (queue mutex)
  std::atomic<int> terminal{HYLE_HIP_OK};
};
// A sequence is its completion slot, reserved by begin.
struct hyle_hip_sequence {
  hyle_hip_completion slot;
};

struct hyle_hip_queue {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  std::mutex mutex;
  std::vector<hyle_hip_sequence *> slots;  // every slot ever created for this queue
  hyle_hip_sequence *active = nullptr;
};

namespace {

hyle_hip_sequence *new_slot(hyle_hip_queue *queue, hyle_hip_status *status) {
  auto *slot = new (std::nothrow) hyle_hip_sequence();
  if (slot == nullptr) {
    *status = fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
    return nullptr;
  }
  const hipError_t err = hipEventCreateWithFlags(&slot->slot.event, hipEventDisableTiming);
  if (err != hipSuccess) {
    *status = hip_fail(err, "hipEventCreateWithFlags");
    delete slot;
    return nullptr;
  }
  slot->slot.owner = queue;
  return slot;
}

hyle_hip_status settle(hyle_hip_completion *completion, bool wait, int *done) {
  if (completion->pending.load(std::memory_order_acquire)) {
    DeviceScope scope(completion->owner->device);
    if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
    const hipError_t err = wait ? hipEventSynchronize(completion->event) : hipEventQuery(completion->event);
    if (err == hipErrorNotReady) {
      (void)hipGetLastError();
      if (done) *done = 0;
      return HYLE_HIP_OK;
    }
    if (err != hipSuccess) {  // the first failure seen stays the completion's status
      int expected = HYLE_HIP_OK;
      completion->terminal.compare_exchange_strong(expected, (int)hip_fail(err, wait ? "hipEventSynchronize" : "hipEventQuery"));
    }
    completion->pending.store(false, std::memory_order_release);
  }
  if (done) *done = 1;
  const hyle_hip_status terminal = (hyle_hip_status)completion->terminal.load(std::memory_order_acquire);
  if (terminal != HYLE_HIP_OK) return fail(terminal, "the sequence ended with %s", hyle_hip_status_name(terminal));
  return HYLE_HIP_OK;
}

// What a CompletionEndpoint of this backend carries as its authority: one address per library.
const char kCompletionAuthority = 0;

}  // namespace

extern "C" {

hyle_hip_status hyle_hip_backend_device_count(size_t *count) {
  if (count == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "count output is null");
  int found = 0;
  const hipError_t err = hipGetDeviceCount(&found);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    if (err == hipErrorNoDevice) {  // a machine without a GPU has zero devices
      *count = 0;
      return HYLE_HIP_OK;
    }
    return fail(HYLE_HIP_UNAVAILABLE, "hipGetDeviceCount: %s", hipGetErrorString(err));
  }
  *count = found < 0 ? 0 : (size_t)found;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_backend_device_properties(size_t index, hyle_hip_device_properties *properties) {
  if (properties == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "properties output is null");
  size_t count = 0;
  hyle_hip_status status = hyle_hip_backend_device_count(&count);
  if (status != HYLE_HIP_OK) return status;
  if (index >= count) return fail(HYLE_HIP_OUT_OF_RANGE, "device %zu of %zu", index, count);
  hipDeviceProp_t props;
  const hipError_t err = hipGetDeviceProperties(&props, (int)index);
  if (err != hipSuccess) return hip_fail(err, "hipGetDeviceProperties");
  std::memset(properties, 0, sizeof *properties);
  properties->ordinal = (int32_t)index;
  properties->compute_units = props.multiProcessorCount;
  properties->total_memory_bytes = props.totalGlobalMem;
  properties->unified_memory = 0;
  properties->asynchronous_queues = 1;
  std::snprintf(properties->name, sizeof properties->name, "%s", props.name);
  std::snprintf(properties->architecture, sizeof properties->architecture, "%s", props.gcnArchName);
  return HYLE_HIP_OK;
}

// ---- memory resources -------------------------------------------------------------------
hyle_hip_status hyle_hip_memory_resource_create(hyle_hip_context *context, uint32_t kind,
                                                hyle_hip_memory_resource **resource) {
  if (resource == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "resource output is null");
  *resource = nullptr;
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "a memory resource requires a context");
  if (kind != HYLE_HIP_MEMORY_KIND_DEVICE && kind != HYLE_HIP_MEMORY_KIND_PINNED_HOST)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "memory kind %u is not device or pinned host", kind);
  auto *made = new (std::nothrow) hyle_hip_memory_resource();
  if (made == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  made->device = hyle_hip::context_device(context);
  made->kind = kind;
  *resource = made;
  return HYLE_HIP_OK;
}

void hyle_hip_memory_resource_destroy(hyle_hip_memory_resource *resource) {
  if (resource == nullptr) return;
  {
    DeviceScope scope(resource->device);
    for (auto &entry : resource->live) {
      if (resource->kind == HYLE_HIP_MEMORY_KIND_DEVICE) (void)hipFree(entry.second.base);
      else (void)hipHostFree(entry.second.base);
    }
  }
  delete resource;
}

hyle_hip_status hyle_hip_memory_resource_properties(const hyle_hip_memory_resource *resource,
                                                    hyle_hip_memory_properties *properties) {
  if (resource == nullptr || properties == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  properties->kind = resource->kind;
  properties->minimum_alignment = 256;
  properties->maximum_allocation = SIZE_MAX;
  properties->flags = resource->kind == HYLE_HIP_MEMORY_KIND_DEVICE
                          ? HYLE_HIP_MEMORY_DEVICE_ACCESSIBLE
                          : (HYLE_HIP_MEMORY_HOST_ACCESSIBLE | HYLE_HIP_MEMORY_DEVICE_ACCESSIBLE |
                             HYLE_HIP_MEMORY_HOST_DEVICE_COHERENT | HYLE_HIP_MEMORY_HOST_PINNED |
                             HYLE_HIP_MEMORY_HOST_ADDRESS_IDENTITY);
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_memory_allocate(hyle_hip_memory_resource *resource, size_t size, size_t alignment,
                                         void **address) {
  if (address == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "address output is null");
  *address = nullptr;
  if (resource == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "resource is null");
  if (size == 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "allocation size is zero");
  if (alignment == 0) alignment = 256;
  if ((alignment & (alignment - 1)) != 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "alignment is not a power of two");
  // the runtime aligns to 256 bytes at least; a wider alignment is found inside a longer block
  const size_t extra = alignment > 256 ? alignment : 0;
  if (size > SIZE_MAX - extra) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "allocation size overflows");
  DeviceScope scope(resource->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  void *base = nullptr;
  const hipError_t err = resource->kind == HYLE_HIP_MEMORY_KIND_DEVICE
                             ? hipMalloc(&base, size + extra)
                             : hipHostMalloc(&base, size + extra, hipHostMallocDefault);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return hip_fail(err, resource->kind == HYLE_HIP_MEMORY_KIND_DEVICE ? "hipMalloc" : "hipHostMalloc");
  }
  const uintptr_t aligned = (reinterpret_cast<uintptr_t>(base) + alignment - 1) & ~(uintptr_t)(alignment - 1);
  std::lock_guard<std::mutex> lock(resource->mutex);
  resource->live[aligned] = Allocation{base, size};
  resource->used += size;
  resource->peak = resource->used > resource->peak ? resource->used : resource->peak;
  ++resource->total;
  *address = reinterpret_cast<void *>(aligned);
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_memory_deallocate(hyle_hip_memory_resource *resource, void *address) {
  if (resource == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "resource is null");
  if (address == nullptr) return HYLE_HIP_OK;
  Allocation found{};
  {
    std::lock_guard<std::mutex> lock(resource->mutex);
    auto at = resource->live.find(reinterpret_cast<uintptr_t>(address));
    if (at == resource->live.end())
      return fail(HYLE_HIP_INVALID_ARGUMENT, "address was not allocated from this resource");
    found = at->second;
    resource->used -= found.bytes;
    resource->live.erase(at);
  }
  DeviceScope scope(resource->device);
  const hipError_t err = resource->kind == HYLE_HIP_MEMORY_KIND_DEVICE ? hipFree(found.base) : hipHostFree(found.base);
  if (err != hipSuccess) return hip_fail(err, "free");
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_memory_resource_stats(const hyle_hip_memory_resource *resource, hyle_hip_memory_stats *stats) {
  if (resource == nullptr || stats == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(resource->mutex);
  stats->used_bytes = resource->used;
  stats->peak_bytes = resource->peak;
  stats->live_allocations = resource->live.size();
  stats->total_allocations = resource->total;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_backend_validate_resource(const hyle_hip_context *context,
                                                   const hyle_hip_memory_resource *resource) {
  if (context == nullptr || resource == nullptr)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "HIP tensor resource is invalid");
  if (resource->device != hyle_hip::context_device(context))
    return fail(HYLE_HIP_FAILED_PRECONDITION, "HIP tensor resource belongs to a different device");
  return HYLE_HIP_OK;
}

// ---- queues ------------------------------------------------------------------------------
hyle_hip_status hyle_hip_queue_create(hyle_hip_context *context, void *stream, hyle_hip_queue **queue) {
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue output is null");
  *queue = nullptr;
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "a queue requires a context");
  auto *made = new (std::nothrow) hyle_hip_queue();
  if (made == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  made->device = hyle_hip::context_device(context);
  if (stream != nullptr) {
    made->stream = static_cast<hipStream_t>(stream);
  } else {
    DeviceScope scope(made->device);
    hipError_t err = scope.error;
    if (err == hipSuccess) err = hipStreamCreateWithFlags(&made->stream, hipStreamNonBlocking);
    if (err != hipSuccess) {
      delete made;
      return hip_fail(err, "hipStreamCreateWithFlags");
    }
    made->owns_stream = true;
  }
  *queue = made;
  return HYLE_HIP_OK;
}

void hyle_hip_queue_destroy(hyle_hip_queue *queue) {
  if (queue == nullptr) return;
  DeviceScope scope(queue->device);
  (void)hipStreamSynchronize(queue->stream);
  for (hyle_hip_sequence *slot : queue->slots) {
    (void)hipEventDestroy(slot->slot.event);
    delete slot;
  }
  if (queue->owns_stream) (void)hipStreamDestroy(queue->stream);
  delete queue;
}

void *hyle_hip_queue_stream(const hyle_hip_queue *queue) { return queue ? queue->stream : nullptr; }

hyle_hip_status hyle_hip_queue_reserve_completions(hyle_hip_queue *queue, size_t minimum) {
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue is null");
  DeviceScope scope(queue->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  std::lock_guard<std::mutex> lock(queue->mutex);
  while (queue->slots.size() < minimum) {
    hyle_hip_status status = HYLE_HIP_OK;
    hyle_hip_sequence *slot = new_slot(queue, &status);
    if (slot == nullptr) return status;
    queue->slots.push_back(slot);
  }
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_queue_begin_sequence(hyle_hip_queue *queue, hyle_hip_sequence **sequence) {
  if (sequence == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "sequence output is null");
  *sequence = nullptr;
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue is null");
  std::lock_guard<std::mutex> lock(queue->mutex);
  if (queue->active != nullptr) return fail(HYLE_HIP_FAILED_PRECONDITION, "a sequence is already active on this queue");
  hyle_hip_sequence *found = nullptr;
  for (hyle_hip_sequence *slot : queue->slots)
    if (!slot->slot.in_use) {
      found = slot;
      break;
    }
  if (found == nullptr) {  // nothing reserved is free: grow by one
    DeviceScope scope(queue->device);
    if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
    hyle_hip_status status = HYLE_HIP_OK;
    found = new_slot(queue, &status);
    if (found == nullptr) return status;
    queue->slots.push_back(found);
  }
  found->slot.in_use = true;
  found->slot.pending.store(false, std::memory_order_relaxed);
  found->slot.terminal.store(HYLE_HIP_OK, std::memory_order_relaxed);
  queue->active = found;
  *sequence = found;
  return HYLE_HIP_OK;
}

hyle_hip_completion *hyle_hip_queue_finish_sequence(hyle_hip_queue *queue, hyle_hip_sequence *sequence, int accepted,
                                                    hyle_hip_status terminal) {
  bool owned = queue != nullptr && sequence != nullptr && sequence->slot.owner == queue;
  if (owned) {
    std::lock_guard<std::mutex> lock(queue->mutex);
    owned = queue->active == sequence;
  }
  if (!owned) {
    (void)fail(HYLE_HIP_INTERNAL, "sequence does not belong to the queue");
    return nullptr;
  }
  hyle_hip_completion *completion = &sequence->slot;
  completion->terminal.store(terminal, std::memory_order_relaxed);
  if (accepted) {
    DeviceScope scope(queue->device);
    const hipError_t err = scope.error != hipSuccess ? scope.error : hipEventRecord(completion->event, queue->stream);
    if (err == hipSuccess) {
      completion->pending.store(true, std::memory_order_release);
    } else {
      // no event to wait on: fall back to draining the stream now, as the reference's stream fallback does
      (void)hipStreamSynchronize(queue->stream);
      int expected = HYLE_HIP_OK;
      completion->terminal.compare_exchange_strong(expected, (int)hip_fail(err, "hipEventRecord"));
    }
  }
  std::lock_guard<std::mutex> lock(queue->mutex);
  queue->active = nullptr;
  return completion;
}

hyle_hip_status hyle_hip_completion_poll(hyle_hip_completion *completion, int *done) {
  if (completion == nullptr || done == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  return settle(completion, false, done);
}

hyle_hip_status hyle_hip_completion_wait(hyle_hip_completion *completion) {
  if (completion == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "completion is null");
  return settle(completion, true, nullptr);
}

void hyle_hip_completion_release(hyle_hip_completion *completion) {
  if (completion == nullptr) return;
  (void)settle(completion, true, nullptr);
  std::lock_guard<std::mutex> lock(completion->owner->mutex);
  completion->in_use = false;
}

hyle_hip_status hyle_hip_queue_wait_completion(hyle_hip_queue *queue, hyle_hip_completion *completion) {
  if (queue == nullptr || completion == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  if (completion->owner->device != queue->device)
    return fail(HYLE_HIP_UNIMPLEMENTED, "a queue waits for completions of its own device only");
  if (!completion->pending.load(std::memory_order_acquire)) return HYLE_HIP_OK;  // already finished: nothing to order after
  DeviceScope scope(queue->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  const hipError_t err = hipStreamWaitEvent(queue->stream, completion->event, 0);
  if (err != hipSuccess) return hip_fail(err, "hipStreamWaitEvent");
  return HYLE_HIP_OK;
}

int hyle_hip_backend_same_device(size_t left, size_t right) {
  size_t count = 0;
  if (hyle_hip_backend_device_count(&count) != HYLE_HIP_OK || left >= count || right >= count) return 0;
  return left == right ? 1 : 0;  // a device is its ordinal
}

hyle_hip_status hyle_hip_queue_transfer_properties(const hyle_hip_queue *queue,
                                                   const hyle_hip_memory_resource *destination,
                                                   const hyle_hip_memory_resource *source,
                                                   hyle_hip_transfer_properties *properties) {
  if (queue == nullptr || properties == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  properties->mode = HYLE_HIP_TRANSFER_IMMEDIATE;
  properties->peer = 0;
  // the same admission as copy_async: storage of the queue's own device, device or pinned host on
  // either side; nothing else is offered (no hidden staging, no host wait dressed up as a copy)
  if (destination == nullptr || source == nullptr || destination->device != queue->device ||
      source->device != queue->device)
    return fail(HYLE_HIP_UNIMPLEMENTED, "HIP async transfer requires device or pinned storage of the queue's own device");
  properties->mode = HYLE_HIP_TRANSFER_QUEUED_DIRECT;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_queue_completion_endpoint(const hyle_hip_queue *queue, hyle_hip_completion_endpoint *endpoint) {
  if (endpoint == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "endpoint output is null");
  endpoint->authority = queue != nullptr ? &kCompletionAuthority : nullptr;
  endpoint->identity = queue;  // equality means one ordered endpoint: this queue
  return HYLE_HIP_OK;
}

int hyle_hip_queue_can_wait_endpoint(const hyle_hip_queue *destination, hyle_hip_completion_endpoint source) {
  if (destination == nullptr || source.authority != &kCompletionAuthority || source.identity == nullptr) return 0;
  // what hyle_hip_queue_wait_completion accepts: completions of queues of the same device
  return static_cast<const hyle_hip_queue *>(source.identity)->device == destination->device ? 1 : 0;
}

hyle_hip_status hyle_hip_queue_copy_async(hyle_hip_queue *queue, hyle_hip_memory_resource *destination_resource,
                                          void *destination, hyle_hip_memory_resource *source_resource,
                                          const void *source, size_t bytes) {
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue is null");
  if (destination_resource == nullptr || source_resource == nullptr ||
      destination_resource->device != queue->device || source_resource->device != queue->device)
    return fail(HYLE_HIP_UNIMPLEMENTED, "HIP async copy requires storage of the queue's own device");
  if (bytes == 0) return HYLE_HIP_OK;
  if (!destination_resource->holds(destination, bytes) || !source_resource->holds(source, bytes))
    return fail(HYLE_HIP_OUT_OF_RANGE, "copy range lies outside a live allocation of its resource");
  DeviceScope scope(queue->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  const hipError_t err = hipMemcpyAsync(destination, source, bytes, hipMemcpyDefault, queue->stream);
  if (err != hipSuccess) return hip_fail(err, "hipMemcpyAsync");
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_queue_fill_async(hyle_hip_queue *queue, hyle_hip_memory_resource *destination_resource,
                                          void *destination, uint8_t value, size_t bytes) {
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue is null");
  if (destination_resource == nullptr || destination_resource->device != queue->device ||
      destination_resource->kind == HYLE_HIP_MEMORY_KIND_PINNED_HOST)
    return fail(HYLE_HIP_UNIMPLEMENTED, "HIP async fill requires device storage of the queue's own device");
  if (bytes == 0) return HYLE_HIP_OK;
  if (!destination_resource->holds(destination, bytes))
    return fail(HYLE_HIP_OUT_OF_RANGE, "fill range lies outside a live allocation of its resource");
  DeviceScope scope(queue->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  const size_t vectors = bytes / 16 + 1;
  size_t blocks = (vectors + 255) / 256;
  blocks = blocks > 4096 ? 4096 : blocks;
  const uint32_t value4 = 0x01010101u * value;
  hipLaunchKernelGGL(fill_bytes, dim3((uint32_t)blocks), dim3(256), 0, queue->stream,
                     static_cast<unsigned char *>(destination), bytes, value4);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return hip_fail(err, "fill kernel launch");
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_queue_drain(hyle_hip_queue *queue) {
  if (queue == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "queue is null");
  DeviceScope scope(queue->device);
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  const hipError_t err = hipStreamSynchronize(queue->stream);
  if (err != hipSuccess) return hip_fail(err, "hipStreamSynchronize");
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_context_drain(hyle_hip_context *context) {
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "context is null");
  DeviceScope scope(hyle_hip::context_device(context));
  if (scope.error != hipSuccess) return hip_fail(scope.error, "hipSetDevice");
  const hipError_t err = hipDeviceSynchronize();
  if (err != hipSuccess) return hip_fail(err, "hipDeviceSynchronize");
  return HYLE_HIP_OK;
}

}  // extern "C"
