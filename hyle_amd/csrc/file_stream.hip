// file_stream.hip -- the C ABI of include/hyle_hip_stream.h: a stream-ordered batch of copies
// (the copy endpoint a route gives the reference's file streamer,
// src/compute_stream_cuda/file_stream.cc:8-21) and a staging loop in both directions: file
// ranges read into pinned slots and copied to their device destinations, device ranges copied
// into pinned slots and written to a file (the slot discipline of
// src/compute_stream/file_stream.cc: a slot is reused only after the copies that touch it have
// finished), on the caller's thread or behind a ticket, with cooperative cancellation at slot
// boundaries.  Host code only.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <type_traits>
#include <unistd.h>
#include <vector>

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

struct hyle_hip_stream_ticket;

struct hyle_hip_file_pipeline {
  int device = 0;
  uint32_t slot_count = 0;
  size_t slot_bytes = 0;
  Slot slots[kMaxSlots];  // touched by the thread of the running request only (or, idle, by the caller)
  uint32_t next_slot = 0;
  std::atomic<bool> busy{false};  // a request (on the caller's thread or behind a ticket) is running
  std::mutex guard;                         // protects `live`
  hyle_hip_stream_ticket *live = nullptr;   // the ticket whose thread may still use the slots
};

namespace {
// Waits for every copy that still reads or writes a slot.  Only the thread that runs the
// pipeline's request, or a caller of an idle pipeline, may call it.
hyle_hip_status wait_slots(hyle_hip_file_pipeline *p) {
  for (uint32_t s = 0; s < p->slot_count; ++s) {
    if (!p->slots[s].in_flight) continue;
    const hipError_t err = hipEventSynchronize(p->slots[s].drained);
    if (err != hipSuccess) return hip_fail(err, "hipEventSynchronize");
    p->slots[s].in_flight = false;
  }
  return HYLE_HIP_OK;
}
void end_live_ticket(hyle_hip_file_pipeline *p);
}  // namespace

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
  // the slots belong to the running request's thread: wait for the ticket instead
  if (p->busy.load(std::memory_order_acquire))
    return fail(HYLE_HIP_FAILED_PRECONDITION, "the pipeline is running a request: wait for its ticket");
  return wait_slots(p);
}

void hyle_hip_file_pipeline_destroy(hyle_hip_file_pipeline *p) {
  if (p == nullptr) return;
  // a ticket's thread may still fill, copy from or wait for the slots: ask it to stop and let it
  // end before anything is freed (its ticket stays valid and reports the progress it made)
  end_live_ticket(p);
  (void)hipSetDevice(p->device);
  for (uint32_t s = 0; s < p->slot_count; ++s) {
    if (p->slots[s].in_flight) (void)hipEventSynchronize(p->slots[s].drained);
    if (p->slots[s].drained != nullptr) (void)hipEventDestroy(p->slots[s].drained);
    if (p->slots[s].bytes != nullptr) (void)hipHostFree(p->slots[s].bytes);
  }
  delete p;
}

}  // extern "C"

namespace {

// Marks the slot as read by copies still in flight; if the event cannot be recorded the
// stream is drained instead, so that the slot is never refilled or freed under a copy.
void seal_slot(Slot &slot, hipStream_t stream) {
  if (hipEventRecord(slot.drained, stream) == hipSuccess) {
    slot.in_flight = true;
  } else {
    (void)hipGetLastError();
    (void)hipStreamSynchronize(stream);
    slot.in_flight = false;
  }
}

hyle_hip_status wait_slot(Slot &slot, hyle_hip_stream_result &out) {
  if (!slot.in_flight) return HYLE_HIP_OK;
  ++out.host_waits;
  const hipError_t err = hipEventSynchronize(slot.drained);
  if (err != hipSuccess) return hip_fail(err, "hipEventSynchronize");
  slot.in_flight = false;
  return HYLE_HIP_OK;
}

bool cancelled(const std::atomic<bool> *cancel) { return cancel != nullptr && cancel->load(std::memory_order_relaxed); }

// What another thread may read of a running request: a copy of the counters, refreshed at
// every slot boundary under a lock (the request's own counters are its thread's alone).
struct Progress {
  std::mutex lock;
  hyle_hip_stream_result shown{};
  void publish(const hyle_hip_stream_result &now) {
    std::lock_guard<std::mutex> hold(lock);
    shown = now;
  }
};
void publish(Progress *progress, const hyle_hip_stream_result &now) {
  if (progress != nullptr) progress->publish(now);
}

// file -> pinned slots -> device.  Ranges are packed into a slot back to back (several small
// ranges share one, a large one takes many in turn); a slot goes to the device as soon as it is
// full or the ranges end.  `out` is updated as the work proceeds, so another thread may read
// the progress; a cancellation request is honoured before each slot is filled.
hyle_hip_status run_read(hyle_hip_file_pipeline *p, int fd, const hyle_hip_read_range *ranges, uint32_t range_count,
                         hipStream_t stream, hyle_hip_stream_result &out, const std::atomic<bool> *cancel,
                         Progress *progress) {
  hipError_t err = hipSetDevice(p->device);
  if (err != hipSuccess) return hip_fail(err, "hipSetDevice");
  uint32_t r = 0;
  size_t done_in_range = 0;
  while (r < range_count) {
    publish(progress, out);
    if (cancelled(cancel)) return fail(HYLE_HIP_CANCELLED, "the read was cancelled");
    Slot &slot = p->slots[p->next_slot];
    hyle_hip_status status = wait_slot(slot, out);
    if (status != HYLE_HIP_OK) return status;
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
          const int saved = errno;
          if (enqueued) seal_slot(slot, stream);
          out.read_bytes += got;
          return n == 0 ? fail(HYLE_HIP_OUT_OF_RANGE, "end of file inside range %u at offset %llu", r,
                               (unsigned long long)(ranges[r].file_offset + done_in_range + got))
                        : fail(HYLE_HIP_INTERNAL, "pread: %s", strerror(saved));
        }
        got += (size_t)n;
      }
      out.read_bytes += piece;
      err = hipMemcpyAsync(static_cast<unsigned char *>(ranges[r].destination) + done_in_range, slot.bytes + used,
                           piece, hipMemcpyHostToDevice, stream);
      if (err != hipSuccess) {
        if (enqueued) seal_slot(slot, stream);  // earlier pieces of this slot are still being read
        return hip_fail(err, "hipMemcpyAsync");
      }
      enqueued = true;
      ++out.native_calls;
      out.copied_bytes += piece;
      used += piece;
      done_in_range += piece;
    }
    if (enqueued) {
      seal_slot(slot, stream);
      p->next_slot = (p->next_slot + 1) % p->slot_count;
    }
  }
  return HYLE_HIP_OK;
}

// device -> pinned slots -> file.  Up to slot_count pieces are on their way from the device
// while the oldest one is written to the file; pieces leave in range order.
hyle_hip_status run_write(hyle_hip_file_pipeline *p, int fd, const hyle_hip_write_range *ranges, uint32_t range_count,
                          hipStream_t stream, hyle_hip_stream_result &out, const std::atomic<bool> *cancel,
                          Progress *progress) {
  hipError_t err = hipSetDevice(p->device);
  if (err != hipSuccess) return hip_fail(err, "hipSetDevice");
  hyle_hip_status status = HYLE_HIP_OK;
  for (uint32_t s = 0; s < p->slot_count; ++s)  // leftovers of an earlier read
    if ((status = wait_slot(p->slots[s], out)) != HYLE_HIP_OK) return status;
  struct Piece {
    uint32_t range;
    uint64_t file_offset;
    size_t bytes;
    bool closes_range;
  };
  Piece in_slot[kMaxSlots];
  uint32_t head = 0, filled = 0;  // slots [head, head + filled) hold pieces on their way, oldest first
  uint32_t r = 0;
  size_t done_in_range = 0;
  auto retire_oldest = [&]() -> hyle_hip_status {
    Slot &slot = p->slots[head];
    const Piece piece = in_slot[head];
    hyle_hip_status waited = wait_slot(slot, out);
    if (waited != HYLE_HIP_OK) return waited;
    size_t put = 0;
    while (put < piece.bytes) {
      const ssize_t n = pwrite(fd, slot.bytes + put, piece.bytes - put, (off_t)(piece.file_offset + put));
      ++out.io_calls;
      if (n < 0 && errno == EINTR) continue;
      if (n <= 0) {
        out.written_bytes += put;
        return fail(HYLE_HIP_INTERNAL, "pwrite at offset %llu: %s", (unsigned long long)(piece.file_offset + put),
                    n == 0 ? "no progress" : strerror(errno));
      }
      put += (size_t)n;
    }
    out.written_bytes += piece.bytes;
    if (piece.closes_range) ++out.ready_ranges;
    head = (head + 1) % p->slot_count;
    --filled;
    return HYLE_HIP_OK;
  };
  auto drain_in_flight = [&]() {  // on an error exit: no copy may still write into a slot
    for (uint32_t s = 0; s < p->slot_count; ++s)
      if (p->slots[s].in_flight && hipEventSynchronize(p->slots[s].drained) == hipSuccess) p->slots[s].in_flight = false;
  };
  while (r < range_count || filled != 0) {
    publish(progress, out);
    if (cancelled(cancel)) {
      drain_in_flight();
      return fail(HYLE_HIP_CANCELLED, "the write was cancelled");
    }
    while (r < range_count && ranges[r].bytes == done_in_range) {  // empty or finished ranges
      if (ranges[r].bytes == 0) ++out.ready_ranges;
      ++r;
      done_in_range = 0;
    }
    if (r < range_count && filled < p->slot_count) {
      const uint32_t at = (head + filled) % p->slot_count;
      Slot &slot = p->slots[at];
      const size_t left = ranges[r].bytes - done_in_range;
      const size_t piece = left < p->slot_bytes ? left : p->slot_bytes;
      err = hipMemcpyAsync(slot.bytes, static_cast<const unsigned char *>(ranges[r].source) + done_in_range, piece,
                           hipMemcpyDeviceToHost, stream);
      if (err != hipSuccess) {
        drain_in_flight();
        return hip_fail(err, "hipMemcpyAsync");
      }
      seal_slot(slot, stream);
      ++out.native_calls;
      out.copied_bytes += piece;
      in_slot[at] = Piece{r, ranges[r].file_offset + done_in_range, piece, piece == left};
      ++filled;
      done_in_range += piece;
      continue;
    }
    if (filled != 0 && (status = retire_oldest()) != HYLE_HIP_OK) {
      drain_in_flight();
      return status;
    }
  }
  p->next_slot = 0;
  return HYLE_HIP_OK;
}

hyle_hip_status check_request(hyle_hip_file_pipeline *p, int fd, const void *ranges, uint32_t range_count) {
  if (p == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "pipeline is null");
  if (fd < 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "file descriptor is invalid");
  if (range_count != 0 && ranges == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "ranges are null");
  return HYLE_HIP_OK;
}
hyle_hip_status check_ranges(const hyle_hip_read_range *ranges, uint32_t range_count) {
  for (uint32_t r = 0; r < range_count; ++r)
    if (ranges[r].bytes != 0 && ranges[r].destination == nullptr)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "range %u has no destination", r);
  return HYLE_HIP_OK;
}
hyle_hip_status check_ranges(const hyle_hip_write_range *ranges, uint32_t range_count) {
  for (uint32_t r = 0; r < range_count; ++r)
    if (ranges[r].bytes != 0 && ranges[r].source == nullptr)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "range %u has no source", r);
  return HYLE_HIP_OK;
}

// One request at a time per pipeline.
bool claim(hyle_hip_file_pipeline *p) {
  bool idle = false;
  return p->busy.compare_exchange_strong(idle, true);
}

}  // namespace

// A request running on a thread of its own.  `result` is that thread's alone until `ended`;
// while it runs, readers get `progress.shown`, a copy refreshed at every slot boundary.
struct hyle_hip_stream_ticket {
  // null once the pipeline has been destroyed or has taken a later request
  std::atomic<hyle_hip_file_pipeline *> pipeline{nullptr};
  std::thread worker;
  std::mutex join_lock;  // the worker is joined once, by whichever of wait / release / pipeline destroy comes first
  std::atomic<bool> cancel{false};
  std::atomic<bool> ended{false};
  hyle_hip_stream_result result{};
  Progress progress;
  std::vector<hyle_hip_read_range> reads;
  std::vector<hyle_hip_write_range> writes;
  char error_text[320] = "";
  int fd = -1;
  hipStream_t stream = nullptr;
  bool is_write = false;
};

namespace {

void join_worker(hyle_hip_stream_ticket *t) {
  std::lock_guard<std::mutex> hold(t->join_lock);
  if (t->worker.joinable()) t->worker.join();
}

void ticket_main(hyle_hip_stream_ticket *t) {
  hyle_hip_file_pipeline *p = t->pipeline.load();  // alive until this thread has been joined
  hyle_hip_status status;
  if (t->is_write)
    status = run_write(p, t->fd, t->writes.data(), (uint32_t)t->writes.size(), t->stream, t->result, &t->cancel, &t->progress);
  else
    status = run_read(p, t->fd, t->reads.data(), (uint32_t)t->reads.size(), t->stream, t->result, &t->cancel, &t->progress);
  // the copies too; after a failure or a cancellation as well, so that no copy still touches a
  // slot when the request reports its end
  const hyle_hip_status drained = wait_slots(p);
  if (status == HYLE_HIP_OK) status = drained;
  std::snprintf(t->error_text, sizeof t->error_text, "%s", hyle_hip_last_error());  // this thread's text
  t->result.status = status;
  t->result.complete = 1;
  // the ticket reports its end before the pipeline takes the next request
  t->ended.store(true, std::memory_order_release);
  p->busy.store(false, std::memory_order_release);
}

// hyle_hip_file_pipeline_destroy: the live ticket's thread must be gone before the slots are.
void end_live_ticket(hyle_hip_file_pipeline *p) {
  hyle_hip_stream_ticket *t = nullptr;
  {
    std::lock_guard<std::mutex> hold(p->guard);
    t = p->live;
    p->live = nullptr;
  }
  if (t == nullptr) return;
  t->cancel.store(true, std::memory_order_relaxed);
  join_worker(t);
  t->pipeline.store(nullptr);
}

template <class Range>
hyle_hip_status submit(hyle_hip_file_pipeline *p, int fd, const Range *ranges, uint32_t range_count, void *stream,
                       hyle_hip_stream_ticket **out, bool is_write) {
  if (out == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "ticket output is null");
  *out = nullptr;
  hyle_hip_status status = check_request(p, fd, ranges, range_count);
  if (status == HYLE_HIP_OK) status = check_ranges(ranges, range_count);
  if (status != HYLE_HIP_OK) return status;
  auto *t = new (std::nothrow) hyle_hip_stream_ticket();
  if (t == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  if (!claim(p)) {
    delete t;
    return fail(HYLE_HIP_FAILED_PRECONDITION, "the pipeline is running another request");
  }
  t->pipeline = p;
  t->fd = fd;
  t->stream = static_cast<hipStream_t>(stream);
  t->is_write = is_write;
  t->result.total_ranges = range_count;
  try {
    if constexpr (std::is_same<Range, hyle_hip_write_range>::value) t->writes.assign(ranges, ranges + range_count);
    else t->reads.assign(ranges, ranges + range_count);
    std::lock_guard<std::mutex> hold(p->guard);
    // an earlier ticket has ended (the pipeline was idle): it no longer needs the slots, and must
    // not look for this pipeline when it is released after the pipeline is gone
    if (p->live != nullptr) p->live->pipeline.store(nullptr);
    t->worker = std::thread(ticket_main, t);
    p->live = t;
  } catch (...) {
    p->busy.store(false);
    delete t;
    return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "the request's thread could not be started");
  }
  *out = t;
  return HYLE_HIP_OK;
}

}  // namespace

extern "C" {

hyle_hip_status hyle_hip_file_pipeline_read(hyle_hip_file_pipeline *p, int fd, const hyle_hip_read_range *ranges,
                                            uint32_t range_count, void *stream_handle,
                                            hyle_hip_stream_result *result) {
  hyle_hip_stream_result local{};
  hyle_hip_stream_result &out = result ? *result : local;
  out = hyle_hip_stream_result{};
  out.total_ranges = range_count;
  hyle_hip_status status = check_request(p, fd, ranges, range_count);
  if (status == HYLE_HIP_OK) status = check_ranges(ranges, range_count);
  if (status == HYLE_HIP_OK && !claim(p))
    status = fail(HYLE_HIP_FAILED_PRECONDITION, "the pipeline is running another request");
  else if (status == HYLE_HIP_OK) {
    status = run_read(p, fd, ranges, range_count, static_cast<hipStream_t>(stream_handle), out, nullptr, nullptr);
    p->busy.store(false);
  }
  out.status = status;
  out.complete = 1;
  return status;
}

hyle_hip_status hyle_hip_file_pipeline_write(hyle_hip_file_pipeline *p, int fd, const hyle_hip_write_range *ranges,
                                             uint32_t range_count, void *stream_handle,
                                             hyle_hip_stream_result *result) {
  hyle_hip_stream_result local{};
  hyle_hip_stream_result &out = result ? *result : local;
  out = hyle_hip_stream_result{};
  out.total_ranges = range_count;
  hyle_hip_status status = check_request(p, fd, ranges, range_count);
  if (status == HYLE_HIP_OK) status = check_ranges(ranges, range_count);
  if (status == HYLE_HIP_OK && !claim(p))
    status = fail(HYLE_HIP_FAILED_PRECONDITION, "the pipeline is running another request");
  else if (status == HYLE_HIP_OK) {
    status = run_write(p, fd, ranges, range_count, static_cast<hipStream_t>(stream_handle), out, nullptr, nullptr);
    p->busy.store(false);
  }
  out.status = status;
  out.complete = 1;
  return status;
}

hyle_hip_status hyle_hip_file_pipeline_submit_read(hyle_hip_file_pipeline *p, int fd, const hyle_hip_read_range *ranges,
                                                   uint32_t range_count, void *stream, hyle_hip_stream_ticket **ticket) {
  return submit(p, fd, ranges, range_count, stream, ticket, false);
}

hyle_hip_status hyle_hip_file_pipeline_submit_write(hyle_hip_file_pipeline *p, int fd,
                                                    const hyle_hip_write_range *ranges, uint32_t range_count,
                                                    void *stream, hyle_hip_stream_ticket **ticket) {
  return submit(p, fd, ranges, range_count, stream, ticket, true);
}

hyle_hip_status hyle_hip_stream_ticket_result(hyle_hip_stream_ticket *ticket, hyle_hip_stream_result *result) {
  if (ticket == nullptr || result == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  if (ticket->ended.load(std::memory_order_acquire)) {
    *result = ticket->result;
    return HYLE_HIP_OK;
  }
  {  // a running request: the progress it last published; its status is not known yet
    std::lock_guard<std::mutex> hold(ticket->progress.lock);
    *result = ticket->progress.shown;
  }
  result->total_ranges = (uint32_t)(ticket->is_write ? ticket->writes.size() : ticket->reads.size());
  result->status = HYLE_HIP_OK;
  result->complete = 0;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_stream_ticket_wait(hyle_hip_stream_ticket *ticket, hyle_hip_stream_result *result) {
  if (ticket == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "ticket is null");
  join_worker(ticket);
  if (result != nullptr) *result = ticket->result;
  if (ticket->result.status != HYLE_HIP_OK) return fail(ticket->result.status, "%s", ticket->error_text);
  return HYLE_HIP_OK;
}

void hyle_hip_stream_ticket_request_cancel(hyle_hip_stream_ticket *ticket) {
  if (ticket != nullptr) ticket->cancel.store(true, std::memory_order_relaxed);
}

void hyle_hip_stream_ticket_release(hyle_hip_stream_ticket *ticket) {
  if (ticket == nullptr) return;
  ticket->cancel.store(true, std::memory_order_relaxed);
  join_worker(ticket);
  if (hyle_hip_file_pipeline *p = ticket->pipeline.load()) {  // still there: it must forget this ticket
    std::lock_guard<std::mutex> hold(p->guard);
    if (p->live == ticket) p->live = nullptr;
  }
  delete ticket;
}

}  // extern "C"
