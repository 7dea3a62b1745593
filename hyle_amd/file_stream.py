"""Host mirror of include/hyle_hip_stream.h: the copy endpoint and the file -> pinned staging ->
HBM pipeline, under the names of the reference (include/hyle/compute/file_stream.h,
include/hyle/compute/batch_transfer.h)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

from . import capi
from .compute import Context, StatusError, _check


@dataclass(frozen=True)
class FileStreamOptions:  # include/hyle/compute/file_stream.h:19-28 (the staging fields)
    in_flight_slots: int = 2
    staging_bytes_per_slot: int = 1024 * 1024
    staging_alignment: int = 256


@dataclass(frozen=True)
class StreamReadRange:  # include/hyle/compute/file_stream.h:85-90
    file_offset: int
    destination: int  # device address
    bytes: int


@dataclass(frozen=True)
class StreamResult:  # include/hyle/compute/file_stream.h:111-118
    status: int
    read_bytes: int
    copied_bytes: int
    ready_ranges: int
    total_ranges: int
    io_calls: int
    native_calls: int
    host_waits: int
    written_bytes: int = 0
    complete: int = 0


@dataclass(frozen=True)
class StreamWriteRange:  # include/hyle/compute/file_stream.h:92-105 (StreamWriteRange::ready)
    source: int  # device address
    file_offset: int
    bytes: int


class StreamTicket:
    """include/hyle/compute/file_stream.h:158-180: a request running on a thread of the pipeline."""

    def __init__(self, handle: int, pipeline: "Optional[FileResourcePipeline]" = None):
        self._handle: Optional[int] = handle
        # the request's thread uses the pipeline's staging: the pipeline lives as long as its ticket
        self._pipeline = pipeline

    @staticmethod
    def _snapshot(c_result) -> StreamResult:
        return StreamResult(*[getattr(c_result, name) for name, _ in capi.StreamResultC._fields_])

    def result(self) -> StreamResult:
        c_result = capi.StreamResultC()
        _check(capi.load().hyle_hip_stream_ticket_result(self._handle, C.byref(c_result)))
        return self._snapshot(c_result)

    def wait(self) -> StreamResult:
        """Blocks until the request has ended; raises StatusError if it failed or was cancelled
        (`last_result` keeps the progress)."""
        c_result = capi.StreamResultC()
        code = capi.load().hyle_hip_stream_ticket_wait(self._handle, C.byref(c_result))
        self.last_result = self._snapshot(c_result)
        if code != capi.OK:
            raise StatusError(code, capi.last_error())
        return self.last_result

    def request_cancel(self) -> None:
        capi.load().hyle_hip_stream_ticket_request_cancel(self._handle)

    def close(self) -> None:
        if self._handle:
            capi.load().hyle_hip_stream_ticket_release(self._handle)
            self._handle = None
        self._pipeline = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass(frozen=True)
class CopyRange:  # include/hyle/compute/batch_transfer.h:30-38
    source: int
    destination: int
    bytes: int
    phase: int = 0


@dataclass(frozen=True)
class CopyPhase:  # include/hyle/compute/batch_transfer.h:40-45
    dependency_mask: int = 0
    group_tag: int = 0


def submit_copy_batch(context: Context, phases: Sequence[CopyPhase], ranges: Sequence[CopyRange], stream: int) -> None:
    """CopyBatchInvocation::prepare_replay + submit: enqueue and return."""
    cp = (capi.CopyPhaseC * max(len(phases), 1))(*[capi.CopyPhaseC(p.dependency_mask, p.group_tag) for p in phases])
    cr = (capi.CopyRangeC * max(len(ranges), 1))(*[capi.CopyRangeC(r.source, r.destination, r.bytes, r.phase)
                                                    for r in ranges])
    _check(capi.load().hyle_hip_copy_batch_submit(context._handle, cp, len(phases), cr, len(ranges), stream))


class FileResourcePipeline:
    """create_file_pipeline (src/compute_stream_cuda/file_stream.cc:8-21) for a HIP context."""

    def __init__(self, handle: int):
        self._handle: Optional[int] = handle
        self.last_result: Optional[StreamResult] = None

    @staticmethod
    def create(context: Context, options: FileStreamOptions = FileStreamOptions()) -> "FileResourcePipeline":
        handle = C.c_void_p()
        c_options = capi.FileStreamOptionsC(options.in_flight_slots, options.staging_bytes_per_slot,
                                            options.staging_alignment)
        _check(capi.load().hyle_hip_file_pipeline_create(context._handle, C.byref(c_options), C.byref(handle)))
        return FileResourcePipeline(handle.value)

    def read(self, fd: int, ranges: Sequence[StreamReadRange], stream: int) -> StreamResult:
        """Enqueue every range; raises StatusError on failure (last_result keeps the progress)."""
        c_ranges = (capi.ReadRangeC * max(len(ranges), 1))(*[capi.ReadRangeC(r.file_offset, r.destination, r.bytes)
                                                             for r in ranges])
        c_result = capi.StreamResultC()
        code = capi.load().hyle_hip_file_pipeline_read(self._handle, fd, c_ranges, len(ranges), stream,
                                                       C.byref(c_result))
        self.last_result = StreamResult(*[getattr(c_result, name) for name, _ in capi.StreamResultC._fields_])
        if code != capi.OK:
            raise StatusError(code, capi.last_error())
        return self.last_result

    def write(self, fd: int, ranges: Sequence["StreamWriteRange"], stream: int) -> StreamResult:
        """Device ranges to the file; returns when the last byte is written."""
        c_ranges = (capi.WriteRangeC * max(len(ranges), 1))(*[capi.WriteRangeC(r.source, r.file_offset, r.bytes)
                                                              for r in ranges])
        c_result = capi.StreamResultC()
        code = capi.load().hyle_hip_file_pipeline_write(self._handle, fd, c_ranges, len(ranges), stream,
                                                        C.byref(c_result))
        self.last_result = StreamResult(*[getattr(c_result, name) for name, _ in capi.StreamResultC._fields_])
        if code != capi.OK:
            raise StatusError(code, capi.last_error())
        return self.last_result

    def submit_read(self, fd: int, ranges: Sequence[StreamReadRange], stream: int) -> "StreamTicket":
        c_ranges = (capi.ReadRangeC * max(len(ranges), 1))(*[capi.ReadRangeC(r.file_offset, r.destination, r.bytes)
                                                             for r in ranges])
        handle = C.c_void_p()
        _check(capi.load().hyle_hip_file_pipeline_submit_read(self._handle, fd, c_ranges, len(ranges), stream,
                                                              C.byref(handle)))
        return self._ticket(handle.value)

    def submit_write(self, fd: int, ranges: Sequence["StreamWriteRange"], stream: int) -> "StreamTicket":
        c_ranges = (capi.WriteRangeC * max(len(ranges), 1))(*[capi.WriteRangeC(r.source, r.file_offset, r.bytes)
                                                              for r in ranges])
        handle = C.c_void_p()
        _check(capi.load().hyle_hip_file_pipeline_submit_write(self._handle, fd, c_ranges, len(ranges), stream,
                                                               C.byref(handle)))
        return self._ticket(handle.value)

    def _ticket(self, handle: int) -> "StreamTicket":
        return StreamTicket(handle, self)

    def wait(self) -> None:
        _check(capi.load().hyle_hip_file_pipeline_wait(self._handle))

    def close(self) -> None:
        """Ends a request still running behind a ticket (it is cancelled; the ticket keeps its
        progress and stays usable), then frees the staging."""
        if self._handle:
            capi.load().hyle_hip_file_pipeline_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
