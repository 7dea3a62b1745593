"""Host mirror of include/hyle_hip_backend.h: the reference's backend contract
(src/compute/backend_internal.h:14-67) over HIP: devices, memory resources, queues, sequences and
completions, queue-ordered copy and fill."""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass
from typing import Optional

from . import capi
from .compute import Context, StatusError, _check


class MemoryProperty(enum.IntFlag):  # include/hyle/mem/resource.h:19-33
    kNone = 0
    kHostAccessible = 1 << 0
    kDeviceAccessible = 1 << 1
    kHostDeviceCoherent = 1 << 2
    kHostPinned = 1 << 3
    kHostAddressIdentity = 1 << 7


class MemoryKind(enum.IntEnum):
    kDevice = 0
    kPinnedHost = 1


@dataclass(frozen=True)
class DeviceProperties:
    ordinal: int
    compute_units: int
    total_memory_bytes: int
    unified_memory: bool
    asynchronous_queues: bool
    name: str
    architecture: str


def device_count() -> int:
    count = C.c_size_t(0)
    _check(capi.load().hyle_hip_backend_device_count(C.byref(count)))
    return count.value


def device_properties(index: int) -> DeviceProperties:
    raw = capi.DevicePropertiesC()
    _check(capi.load().hyle_hip_backend_device_properties(index, C.byref(raw)))
    return DeviceProperties(raw.ordinal, raw.compute_units, raw.total_memory_bytes, bool(raw.unified_memory),
                            bool(raw.asynchronous_queues), raw.name.decode(), raw.architecture.decode())


class MemoryResource:
    """include/hyle/mem/resource.h:108-151 for device or pinned host memory of one HIP device."""

    def __init__(self, context: Context, kind: MemoryKind):
        handle = C.c_void_p()
        _check(capi.load().hyle_hip_memory_resource_create(context._handle, int(kind), C.byref(handle)))
        self._handle: Optional[int] = handle.value
        self.kind = kind

    def properties(self):
        raw = capi.MemoryPropertiesC()
        _check(capi.load().hyle_hip_memory_resource_properties(self._handle, C.byref(raw)))
        return MemoryProperty(raw.flags), raw.minimum_alignment, raw.maximum_allocation

    def allocate(self, size: int, alignment: int = 256) -> int:
        address = C.c_void_p()
        _check(capi.load().hyle_hip_memory_allocate(self._handle, size, alignment, C.byref(address)))
        return address.value

    def deallocate(self, address: int) -> None:
        _check(capi.load().hyle_hip_memory_deallocate(self._handle, address))

    def stats(self):
        raw = capi.MemoryStatsC()
        _check(capi.load().hyle_hip_memory_resource_stats(self._handle, C.byref(raw)))
        return raw.used_bytes, raw.peak_bytes, raw.live_allocations, raw.total_allocations

    def close(self) -> None:
        if self._handle:
            capi.load().hyle_hip_memory_resource_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class TransferMode(enum.IntEnum):  # include/hyle/compute/transfer.h:19-22
    kImmediate = 0
    kQueuedDirect = 1


@dataclass(frozen=True)
class TransferProperties:  # include/hyle/compute/transfer.h:27-30
    mode: TransferMode
    peer: bool


@dataclass(frozen=True)
class CompletionEndpoint:  # who emits a queue's completions: (authority, identity) as addresses
    authority: int = 0
    identity: int = 0

    def valid(self) -> bool:
        return bool(self.authority) and bool(self.identity)


def same_device(left: int, right: int) -> bool:
    """BackendVTable::same_device over device indices."""
    return bool(capi.load().hyle_hip_backend_same_device(left, right))


def validate_resource(context: Context, resource: MemoryResource) -> None:
    _check(capi.load().hyle_hip_backend_validate_resource(context._handle, resource._handle))


class Completion:
    def __init__(self, handle: int):
        self._handle: Optional[int] = handle

    def poll(self) -> bool:
        """True once finished; the terminal status is reported by wait()."""
        done = C.c_int(0)
        code = capi.load().hyle_hip_completion_poll(self._handle, C.byref(done))
        if code != capi.OK and not done.value:
            raise StatusError(code, capi.last_error())
        return bool(done.value)

    def wait(self) -> None:
        _check(capi.load().hyle_hip_completion_wait(self._handle))

    def release(self) -> None:
        if self._handle:
            capi.load().hyle_hip_completion_release(self._handle)
            self._handle = None


class Queue:
    """One HIP stream: BackendVTable::create_queue ... drain_queue."""

    def __init__(self, context: Context, stream: int = 0):
        handle = C.c_void_p()
        _check(capi.load().hyle_hip_queue_create(context._handle, stream or None, C.byref(handle)))
        self._handle: Optional[int] = handle.value
        self._sequence: Optional[int] = None

    @property
    def stream(self) -> int:
        return capi.load().hyle_hip_queue_stream(self._handle) or 0

    def reserve_completions(self, minimum: int) -> None:
        _check(capi.load().hyle_hip_queue_reserve_completions(self._handle, minimum))

    def begin_sequence(self) -> None:
        sequence = C.c_void_p()
        _check(capi.load().hyle_hip_queue_begin_sequence(self._handle, C.byref(sequence)))
        self._sequence = sequence.value

    def finish_sequence(self, accepted: bool = True, terminal: int = capi.OK) -> Completion:
        handle = capi.load().hyle_hip_queue_finish_sequence(self._handle, self._sequence, int(accepted), terminal)
        self._sequence = None
        if not handle:
            raise StatusError(capi.INTERNAL, capi.last_error())
        return Completion(handle)

    def wait_completion(self, completion: Completion) -> None:
        _check(capi.load().hyle_hip_queue_wait_completion(self._handle, completion._handle))

    def transfer_properties(self, destination: "Optional[MemoryResource]", source: "Optional[MemoryResource]") -> "TransferProperties":
        """transfer_properties(queue, destination, source) (include/hyle/compute/transfer.h:31-33): the
        route a copy between the two resources takes on this queue; StatusError(Unimplemented) when none is offered."""
        out = capi.TransferPropertiesC()
        _check(capi.load().hyle_hip_queue_transfer_properties(
            self._handle, destination._handle if destination else None, source._handle if source else None, C.byref(out)))
        return TransferProperties(TransferMode(out.mode), bool(out.peer))

    def completion_endpoint(self) -> "CompletionEndpoint":
        out = capi.CompletionEndpointC()
        _check(capi.load().hyle_hip_queue_completion_endpoint(self._handle, C.byref(out)))
        return CompletionEndpoint(out.authority or 0, out.identity or 0)

    def can_wait_endpoint(self, source: "CompletionEndpoint") -> bool:
        """True commits wait_completion() on this queue to a pending completion emitted by `source`."""
        return bool(capi.load().hyle_hip_queue_can_wait_endpoint(
            self._handle, capi.CompletionEndpointC(source.authority or None, source.identity or None)))

    def copy_async(self, destination_resource: MemoryResource, destination: int, source_resource: MemoryResource,
                   source: int, size: int) -> None:
        _check(capi.load().hyle_hip_queue_copy_async(self._handle, destination_resource._handle, destination,
                                                     source_resource._handle, source, size))

    def fill_async(self, resource: MemoryResource, destination: int, value: int, size: int) -> None:
        _check(capi.load().hyle_hip_queue_fill_async(self._handle, resource._handle, destination, value, size))

    def drain(self) -> None:
        _check(capi.load().hyle_hip_queue_drain(self._handle))

    def close(self) -> None:
        if self._handle:
            capi.load().hyle_hip_queue_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def drain_context(context: Context) -> None:
    _check(capi.load().hyle_hip_context_drain(context._handle))
