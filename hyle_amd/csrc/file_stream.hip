// file_stream.hip -- the C ABI of include/hyle_hip_stream.h: a stream-ordered batch of copies
// (the copy endpoint a route gives the reference's file streamer,
// src/compute_stream_cuda/file_stream.cc:8-21) and a staging loop that reads file ranges into
// pinned slots and copies each filled slot to its device destinations
// (the slot discipline of src/compute_stream/file_stream.cc: a slot is refilled only after the
// copies that read it have finished).  Host code only.
#include <hip/hip_runtime.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <unistd.h>

#include "../../include/hyle_hip_stream.h"

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
  return fail(HYLE_HIP_INTERNAL, "%s: %s", what, hipGetErrorString(error));
}

constexpr uint32_t kMaxSlots = 64;

struct Slot {
  unsigned char *bytes = nullptr;  // pinned
  hipEvent_t drained = nullptr;    // recorded after the last copy that reads the slot
  bool in_flight = false;
};

}  // namespace

struct hyle_hip_file_pipeline {
  int device = 0;
  uint32_t slot_count = 0;
  size_t slot_bytes = 0;
  Slot slots[kMaxSlots];
  uint32_t next_slot = 0;
};

extern "C" {

hyle_hip_status hyle_hip_copy_batch_submit(hyle_hip_context *context, const hyle_hip_copy_phase *phases,
                                           uint32_t phase_count, const hyle_hip_copy_range *ranges,
                                           uint32_t range_count, void *stream_handle) {
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "copy batch requires a context");
  if (phase_count > 64) return fail(HYLE_HIP_INVALID_ARGUMENT, "copy batch holds at most 64 phases");
  if ((phase_count != 0 && phases == nullptr) || (range_count != 0 && ranges == nullptr))
    return fail(HYLE_HIP_INVALID_ARGUMENT, "copy batch arrays are null");
  for (uint32_t p = 0; p < phase_count; ++p) {
    const uint64_t earlier = p == 0 ? 0 : (p >= 64 ? ~0ull : ((1ull << p) - 1));
    if ((phases[p].dependency_mask & ~earlier) != 0)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "copy phase %u depends on itself or on a later phase", p);
  }
  for (uint32_t r = 0; r < range_count; ++r) {
    if (ranges[r].phase >= phase_count)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "copy range %u names phase %u of %u", r, ranges[r].phase, phase_count);
    if (ranges[r].bytes != 0 && (ranges[r].source == nullptr || ranges[r].destination == nullptr))
      return fail(HYLE_HIP_INVALID_ARGUMENT, "copy range %u has a null address", r);
  }
  hipError_t err = hipSetDevice(hyle_hip::context_device(context));
  if (err != hipSuccess) return hip_fail(err, "hipSetDevice");
  hipStream_t stream = static_cast<hipStream_t>(stream_handle);
  for (uint32_t p = 0; p < phase_count; ++p) {
    for (uint32_t r = 0; r < range_count; ++r) {
      if (ranges[r].phase != p || ranges[r].bytes == 0) continue;
      err = hipMemcpyAsync(ranges[r].destination, ranges[r].source, ranges[r].bytes, hipMemcpyDefault, stream);
      if (err != hipSuccess) return hip_fail(err, "hipMemcpyAsync");
    }
  }
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_file_pipeline_create(hyle_hip_context *context,
                                              const hyle_hip_file_stream_options *options,
                                              hyle_hip_file_pipeline **out) {
  if (out == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "pipeline output is null");
  *out = nullptr;
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "file pipeline requires a context");
  const uint32_t slots = options && options->in_flight_slots ? options->in_flight_slots : 2;
  const size_t bytes = options && options->staging_bytes_per_slot ? options->staging_bytes_per_slot : (1u << 20);
  const size_t alignment = options && options->staging_alignment ? options->staging_alignment : 256;
  if (slots > kMaxSlots) return fail(HYLE_HIP_INVALID_ARGUMENT, "at most %u staging slots", kMaxSlots);
  if ((alignment & (alignment - 1)) != 0 || alignment > 4096)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "staging alignment must be a power of two up to 4096");
  hipError_t err = hipSetDevice(hyle_hip::context_device(context));
  if (err != hipSuccess) return hip_fail(err, "hipSetDevice");
  hyle_hip_file_pipeline *p = new (std::nothrow) hyle_hip_file_pipeline();
  if (p == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  p->device = hyle_hip::context_device(context);
  p->slot_count = slots;
  p->slot_bytes = (bytes + alignment - 1) / alignment * alignment;
  for (uint32_t s = 0; s < slots; ++s) {
    void *pinned = nullptr;
    err = hipHostMalloc(&pinned, p->slot_bytes, hipHostMallocDefault);  // page aligned
    if (err == hipSuccess) {
      p->slots[s].bytes = static_cast<unsigned char *>(pinned);
      err = hipEventCreateWithFlags(&p->slots[s].drained, hipEventDisableTiming);
    }
    if (err != hipSuccess) {
      const hyle_hip_status status = hip_fail(err, "pinned staging");
      hyle_hip_file_pipeline_destroy(p);
      return status == HYLE_HIP_INTERNAL && err == hipErrorOutOfMemory
                 ? fail(HYLE_HIP_RESOURCE_EXHAUSTED, "pinned staging: out of memory")
                 : status;
    }
  }
  *out = p;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_file_pipeline_wait(hyle_hip_file_pipeline *p) {
  if (p == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "pipeline is null");
  for (uint32_t s = 0; s < p->slot_count; ++s) {
    if (!p->slots[s].in_flight) continue;
    const hipError_t err = hipEventSynchronize(p->slots[s].drained);
    if (err != hipSuccess) return hip_fail(err, "hipEventSynchronize");
    p->slots[s].in_flight = false;
  }
  return HYLE_HIP_OK;
}

void hyle_hip_file_pipeline_destroy(hyle_hip_file_pipeline *p) {
  if (p == nullptr) return;
  (void)hipSetDevice(p->device);
  for (uint32_t s = 0; s < p->slot_count; ++s) {
    if (p->slots[s].in_flight) (void)hipEventSynchronize(p->slots[s].drained);
    if (p->slots[s].drained != nullptr) (void)hipEventDestroy(p->slots[s].drained);
    if (p->slots[s].bytes != nullptr) (void)hipHostFree(p->slots[s].bytes);
  }
  delete p;
}

hyle_hip_status hyle_hip_file_pipeline_read(hyle_hip_file_pipeline *p, int fd, const hyle_hip_read_range *ranges,
                                            uint32_t range_count, void *stream_handle,
                                            hyle_hip_stream_result *result) {
  hyle_hip_stream_result local{};
  hyle_hip_stream_result &out = result ? *result : local;
  out = hyle_hip_stream_result{};
  out.total_ranges = range_count;
  auto finish = [&](hyle_hip_status status) {
    out.status = status;
    return status;
  };
  if (p == nullptr) return finish(fail(HYLE_HIP_INVALID_ARGUMENT, "pipeline is null"));
  if (fd < 0) return finish(fail(HYLE_HIP_INVALID_ARGUMENT, "file descriptor is invalid"));
  if (range_count != 0 && ranges == nullptr) return finish(fail(HYLE_HIP_INVALID_ARGUMENT, "ranges are null"));
  for (uint32_t r = 0; r < range_count; ++r)
    if (ranges[r].bytes != 0 && ranges[r].destination == nullptr)
      return finish(fail(HYLE_HIP_INVALID_ARGUMENT, "range %u has no destination", r));
  hipError_t err = hipSetDevice(p->device);
  if (err != hipSuccess) return finish(hip_fail(err, "hipSetDevice"));
  hipStream_t stream = static_cast<hipStream_t>(stream_handle);

  // Ranges are packed into a slot back to back (several small ranges share one, a large one
  // takes many in turn); a slot goes to the device as soon as it is full or the ranges end.
  uint32_t r = 0;
  size_t done_in_range = 0;
  while (r < range_count) {
    Slot &slot = p->slots[p->next_slot];
    if (slot.in_flight) {
      ++out.host_waits;
      err = hipEventSynchronize(slot.drained);
      if (err != hipSuccess) return finish(hip_fail(err, "hipEventSynchronize"));
      slot.in_flight = false;
    }
    size_t used = 0;
    bool enqueued = false;
    while (r < range_count && used < p->slot_bytes) {
      const size_t left = ranges[r].bytes - done_in_range;
      if (left == 0) {
        ++r;
        done_in_range = 0;
        ++out.ready_ranges;
        continue;
      }
      const size_t piece = left < p->slot_bytes - used ? left : p->slot_bytes - used;
      size_t got = 0;
      while (got < piece) {
        const ssize_t n = pread(fd, slot.bytes + used + got, piece - got,
                                (off_t)(ranges[r].file_offset + done_in_range + got));
        ++out.io_calls;
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) {
          // what was read so far still goes nowhere: the range is incomplete
          if (enqueued && hipEventRecord(slot.drained, stream) == hipSuccess) slot.in_flight = true;
          out.read_bytes += got;
          return finish(n == 0 ? fail(HYLE_HIP_OUT_OF_RANGE, "end of file inside range %u at offset %llu", r,
                                      (unsigned long long)(ranges[r].file_offset + done_in_range + got))
                               : fail(HYLE_HIP_INTERNAL, "pread: %s", strerror(errno)));
        }
        got += (size_t)n;
      }
      out.read_bytes += piece;
      err = hipMemcpyAsync(static_cast<unsigned char *>(ranges[r].destination) + done_in_range, slot.bytes + used,
                           piece, hipMemcpyHostToDevice, stream);
      if (err != hipSuccess) return finish(hip_fail(err, "hipMemcpyAsync"));
      enqueued = true;
      ++out.native_calls;
      out.copied_bytes += piece;
      used += piece;
      done_in_range += piece;
    }
    if (enqueued) {
      err = hipEventRecord(slot.drained, stream);
      if (err != hipSuccess) return finish(hip_fail(err, "hipEventRecord"));
      slot.in_flight = true;
      p->next_slot = (p->next_slot + 1) % p->slot_count;
    }
  }
  return finish(HYLE_HIP_OK);
}

}  // extern "C"
