/*
 * hyle_hip_stream.h -- C ABI of the MI355X copy endpoint and file -> pinned
 * staging -> HBM pipeline that feeds the tensor operators of hyle_hip.h with
 * weights (GGUF Q8_0 blocks included: they are copied as bytes).
 *
 * The reference splits this work in two.  Its route-neutral file streamer
 * (src/compute_stream/file_stream.cc) reads file ranges into pinned staging
 * slots and hands each filled slot to a route's *copy endpoint*; the CUDA route
 * contributes only that endpoint, a prepared batch of stream-ordered copies
 * (src/compute_stream_cuda/file_stream.cc:8-21 over CopyBatchProgram /
 * CopyBatchInvocation, include/hyle/compute/batch_transfer.h:30-140).  This
 * header is the HIP counterpart of the endpoint (hyle_hip_copy_batch_submit)
 * plus a staging loop over it (hyle_hip_file_pipeline_*) for callers that do not
 * run the reference's streamer: both directions (file -> device and device ->
 * file), run on the calling thread or behind a ticket on a thread of the
 * pipeline, with cooperative cancellation at slot boundaries and the progress
 * made so far reported either way.  The reference's leases, budgets and ready
 * groups are its streamer's own and are not part of this surface.
 */
#ifndef HYLE_HIP_STREAM_H_
#define HYLE_HIP_STREAM_H_

#include "hyle_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* CopyRange (include/hyle/compute/batch_transfer.h:30-38) with plain addresses:
 * `bytes` from `source` to `destination`, either side host (pinned for an
 * asynchronous transfer) or device memory. */
typedef struct hyle_hip_copy_range {
  const void *source;
  void *destination;
  size_t bytes;
  uint32_t phase; /* index into the phases of the same submission */
} hyle_hip_copy_range;

/* CopyPhase (include/hyle/compute/batch_transfer.h:40-45): bit p of
 * dependency_mask names phase p, which must precede this one. */
typedef struct hyle_hip_copy_phase {
  uint64_t dependency_mask;
  uint64_t group_tag;
} hyle_hip_copy_phase;

/* CopyBatchInvocation::prepare_replay + submit
 * (include/hyle/compute/batch_transfer.h:131-132): enqueue every range on
 * `stream`, phase by phase in index order, and return without waiting.  On one
 * in-order stream a dependency on a lower-numbered phase holds by construction;
 * a mask bit that names the phase itself or a later one is INVALID_ARGUMENT,
 * as are more than 64 phases, a range whose phase does not exist, and a null
 * address with a nonzero length.  Nothing is enqueued on error. */
HYLE_HIP_API hyle_hip_status hyle_hip_copy_batch_submit(hyle_hip_context *context,
                                                        const hyle_hip_copy_phase *phases,
                                                        uint32_t phase_count,
                                                        const hyle_hip_copy_range *ranges,
                                                        uint32_t range_count, void *stream);

/* The fields of FileStreamOptions (include/hyle/compute/file_stream.h:19-28)
 * that shape the staging: slots in flight and bytes per slot.  Zero fields take
 * the reference's defaults (2 slots of 1 MiB, 256-byte alignment). */
typedef struct hyle_hip_file_stream_options {
  uint32_t in_flight_slots;
  size_t staging_bytes_per_slot;
  size_t staging_alignment;
} hyle_hip_file_stream_options;

/* StreamReadRange (include/hyle/compute/file_stream.h:85-90): `bytes` at
 * `file_offset` of the file go to the device address `destination`. */
typedef struct hyle_hip_read_range {
  uint64_t file_offset;
  void *destination;
  size_t bytes;
} hyle_hip_read_range;

/* StreamResult (include/hyle/compute/file_stream.h:111-118): partial progress
 * survives a failure. */
typedef struct hyle_hip_stream_result {
  hyle_hip_status status;
  uint64_t read_bytes;   /* bytes read from the file into staging */
  uint64_t copied_bytes; /* bytes whose copy to the device was enqueued */
  uint32_t ready_ranges; /* ranges enqueued completely */
  uint32_t total_ranges;
  uint32_t io_calls;     /* pread calls */
  uint32_t native_calls; /* device copies enqueued */
  uint32_t host_waits;   /* waits for a staging slot still in flight */
  uint64_t written_bytes; /* bytes written to the file (write direction) */
  uint32_t complete;      /* 1 once the request has ended, successfully or not */
} hyle_hip_stream_result;

/* StreamWriteRange::ready (include/hyle/compute/file_stream.h:92-105): `bytes` at the
 * device address `source` go to `file_offset` of the file. */
typedef struct hyle_hip_write_range {
  const void *source;
  uint64_t file_offset;
  size_t bytes;
} hyle_hip_write_range;

typedef struct hyle_hip_file_pipeline hyle_hip_file_pipeline;
typedef struct hyle_hip_stream_ticket hyle_hip_stream_ticket;

/* cuda::create_file_pipeline (src/compute_stream_cuda/file_stream.cc:8-21):
 * binds the context's device and allocates the pinned staging slots. */
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_create(hyle_hip_context *context,
                                                           const hyle_hip_file_stream_options *options,
                                                           hyle_hip_file_pipeline **pipeline);
/* Frees the staging.  A request still running behind a ticket is asked to cancel and its
 * thread has ended (no copy touches a slot any more) before anything is freed; the ticket stays
 * valid, reports CANCELLED (or what it had reached) with its progress, and must still be
 * released.  Slots left in flight by a finished request are waited for.  Must not run
 * concurrently with another call on this pipeline or with the release of its ticket. */
HYLE_HIP_API void hyle_hip_file_pipeline_destroy(hyle_hip_file_pipeline *pipeline);

/* Read every range from the open file `fd` (pread: the file position is not
 * used) through the staging slots into device memory, copies enqueued on
 * `stream`.  File reads happen on the calling thread and overlap the copies of
 * the other slots.  Returns when the last copy is enqueued; the data is
 * complete once `stream` has drained or hyle_hip_file_pipeline_wait returned.
 * End of file before a range is satisfied is OUT_OF_RANGE, an IO error
 * INTERNAL; `result` (optional) then holds how far the call came. */
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_read(hyle_hip_file_pipeline *pipeline, int fd,
                                                         const hyle_hip_read_range *ranges,
                                                         uint32_t range_count, void *stream,
                                                         hyle_hip_stream_result *result);
/* StreamTicket::wait (include/hyle/compute/file_stream.h:171): block until
 * every copy this pipeline enqueued has finished.  While a request runs behind a ticket the
 * slots belong to its thread: FAILED_PRECONDITION, wait for the ticket instead. */
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_wait(hyle_hip_file_pipeline *pipeline);

/* The write direction (FileResourcePipeline::write, include/hyle/compute/file_stream.h:205-206;
 * src/compute_stream/file_stream.cc:519-560): every range goes from device memory through
 * the pinned slots to the open file `fd` (pwrite).  The device-to-host copies are
 * enqueued on `stream`, so they are ordered after whatever produced the data there;
 * the copy of one slot overlaps the file write of another.  Returns when the last byte
 * has been written.  A short write or an IO error is INTERNAL. */
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_write(hyle_hip_file_pipeline *pipeline, int fd,
                                                          const hyle_hip_write_range *ranges,
                                                          uint32_t range_count, void *stream,
                                                          hyle_hip_stream_result *result);

/* StreamTicket (include/hyle/compute/file_stream.h:158-180; FileResourcePipeline::read and
 * ::write return one, :203-206): the same two requests
 * run on a thread of the pipeline; the call returns at once with a ticket.  One request
 * (with or without a ticket) runs on a pipeline at a time: a second one is
 * FAILED_PRECONDITION.  The ranges are copied; the file must stay open and the device
 * memory alive until the ticket has ended.  Order of teardown: release the ticket, then destroy
 * the pipeline; a pipeline destroyed first ends the ticket's request itself (see
 * hyle_hip_file_pipeline_destroy), and the ticket is then released afterwards. */
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_submit_read(hyle_hip_file_pipeline *pipeline, int fd,
                                                                const hyle_hip_read_range *ranges,
                                                                uint32_t range_count, void *stream,
                                                                hyle_hip_stream_ticket **ticket);
HYLE_HIP_API hyle_hip_status hyle_hip_file_pipeline_submit_write(hyle_hip_file_pipeline *pipeline, int fd,
                                                                 const hyle_hip_write_range *ranges,
                                                                 uint32_t range_count, void *stream,
                                                                 hyle_hip_stream_ticket **ticket);
/* StreamTicket::result: the progress so far, without waiting (`complete` says whether the
 * request has ended).  Of a running request this is the state at its last slot boundary. */
HYLE_HIP_API hyle_hip_status hyle_hip_stream_ticket_result(hyle_hip_stream_ticket *ticket,
                                                           hyle_hip_stream_result *result);
/* StreamTicket::wait: block until the request has ended and, for a read, until its copies
 * have finished on the device; returns the request's status. */
HYLE_HIP_API hyle_hip_status hyle_hip_stream_ticket_wait(hyle_hip_stream_ticket *ticket,
                                                         hyle_hip_stream_result *result);
/* StreamTicket::request_cancel: cooperative, honoured at the next slot boundary; the
 * request then ends with HYLE_HIP_CANCELLED (1) and the progress it had made.  Work
 * already enqueued on the device is not recalled. */
HYLE_HIP_API void hyle_hip_stream_ticket_request_cancel(hyle_hip_stream_ticket *ticket);
/* Waits for the request to end (after asking it to cancel) and frees the ticket. */
HYLE_HIP_API void hyle_hip_stream_ticket_release(hyle_hip_stream_ticket *ticket);

#ifdef __cplusplus
}
#endif
#endif /* HYLE_HIP_STREAM_H_ */
