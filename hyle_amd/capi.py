"""ctypes view of include/hyle_hip.h (the C ABI of libhyle_hip.so).

The structures mirror the header field for field.  The library is loaded once; if it has
not been built the import fails loudly rather than falling back to any CPU path.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhyle_hip.so")

MAX_RANK, MAX_INPUTS, MAX_OUTPUTS, ABI_VERSION = 8, 4, 2, 1

# hyle_hip_status
OK, CANCELLED, INVALID_ARGUMENT, RESOURCE_EXHAUSTED, FAILED_PRECONDITION = 0, 1, 3, 8, 9
OUT_OF_RANGE, UNIMPLEMENTED, INTERNAL, UNAVAILABLE = 11, 12, 13, 14


class TensorDescC(C.Structure):
    _fields_ = [
        ("dtype", C.c_uint8), ("rank", C.c_uint8), ("storage", C.c_uint8), ("block_axis", C.c_uint8),
        ("elements_per_block", C.c_uint32), ("bytes_per_block", C.c_uint32), ("reserved", C.c_uint32),
        ("dims", C.c_int64 * MAX_RANK), ("byte_strides", C.c_int64 * MAX_RANK),
    ]


class OpDescC(C.Structure):
    _fields_ = [
        ("abi_version", C.c_uint32), ("op", C.c_uint32), ("kind", C.c_uint32), ("kind2", C.c_uint32),
        ("axis", C.c_int32), ("mask", C.c_uint32), ("accumulation", C.c_uint32),
        ("keep_dimensions", C.c_uint32), ("epsilon", C.c_float), ("scale", C.c_float),
        ("count", C.c_uint64), ("largest", C.c_uint32), ("input_count", C.c_uint32),
        ("inputs", TensorDescC * MAX_INPUTS),
        ("axes_count", C.c_uint32), ("axes", C.c_int32 * MAX_RANK),
    ]


class CopyRangeC(C.Structure):  # include/hyle_hip_stream.h
    _fields_ = [("source", C.c_void_p), ("destination", C.c_void_p), ("bytes", C.c_size_t), ("phase", C.c_uint32)]


class CopyPhaseC(C.Structure):
    _fields_ = [("dependency_mask", C.c_uint64), ("group_tag", C.c_uint64)]


class FileStreamOptionsC(C.Structure):
    _fields_ = [("in_flight_slots", C.c_uint32), ("staging_bytes_per_slot", C.c_size_t),
                ("staging_alignment", C.c_size_t)]


class ReadRangeC(C.Structure):
    _fields_ = [("file_offset", C.c_uint64), ("destination", C.c_void_p), ("bytes", C.c_size_t)]


class StreamResultC(C.Structure):
    _fields_ = [("status", C.c_int), ("read_bytes", C.c_uint64), ("copied_bytes", C.c_uint64),
                ("ready_ranges", C.c_uint32), ("total_ranges", C.c_uint32), ("io_calls", C.c_uint32),
                ("native_calls", C.c_uint32), ("host_waits", C.c_uint32),
                ("written_bytes", C.c_uint64), ("complete", C.c_uint32)]


class WriteRangeC(C.Structure):
    _fields_ = [("source", C.c_void_p), ("file_offset", C.c_uint64), ("bytes", C.c_size_t)]


class DevicePropertiesC(C.Structure):  # include/hyle_hip_backend.h
    _fields_ = [("ordinal", C.c_int32), ("compute_units", C.c_int32), ("total_memory_bytes", C.c_uint64),
                ("unified_memory", C.c_uint32), ("asynchronous_queues", C.c_uint32),
                ("name", C.c_char * 128), ("architecture", C.c_char * 64)]


class MemoryPropertiesC(C.Structure):
    _fields_ = [("flags", C.c_uint32), ("kind", C.c_uint32), ("minimum_alignment", C.c_size_t),
                ("maximum_allocation", C.c_size_t)]


class TransferPropertiesC(C.Structure):
    _fields_ = [("mode", C.c_uint32), ("peer", C.c_uint32)]


class CompletionEndpointC(C.Structure):
    _fields_ = [("authority", C.c_void_p), ("identity", C.c_void_p)]


class MemoryStatsC(C.Structure):
    _fields_ = [("used_bytes", C.c_size_t), ("peak_bytes", C.c_size_t), ("live_allocations", C.c_uint64),
                ("total_allocations", C.c_uint64)]


EXPORTS = {
    # name: (restype, argtypes)
    "hyle_hip_abi_version": (C.c_uint32, []),
    "hyle_hip_last_error": (C.c_char_p, []),
    "hyle_hip_status_name": (C.c_char_p, [C.c_int]),
    "hyle_hip_context_create": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "hyle_hip_context_destroy": (None, [C.c_void_p]),
    "hyle_hip_context_compute_units": (C.c_int, [C.c_void_p]),
    "hyle_hip_infer_outputs": (C.c_int, [C.POINTER(OpDescC), C.POINTER(TensorDescC), C.POINTER(C.c_uint32)]),
    "hyle_hip_plan_create": (C.c_int, [C.c_void_p, C.POINTER(OpDescC), C.POINTER(TensorDescC), C.c_uint32,
                                       C.POINTER(C.c_void_p)]),
    "hyle_hip_plan_destroy": (None, [C.c_void_p]),
    "hyle_hip_plan_workspace": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "hyle_hip_plan_outputs": (C.c_int, [C.c_void_p, C.POINTER(TensorDescC), C.POINTER(C.c_uint32)]),
    "hyle_hip_plan_alias_support": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32]),
    "hyle_hip_plan_dispatch_count": (C.c_uint32, [C.c_void_p]),
    "hyle_hip_plan_route_name": (C.c_char_p, [C.c_void_p]),
    "hyle_hip_variant_count": (C.c_uint32, []),
    "hyle_hip_variant_label": (C.c_char_p, [C.c_uint32]),
    "hyle_hip_last_launch_variant": (C.c_char_p, []),
    "hyle_hip_plan_launch": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_uint32, C.POINTER(C.c_void_p),
                                       C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p]),
    "hyle_hip_plan_device_status": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "hyle_hip_plan_device_status_offset": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t)]),
    "hyle_hip_plan_launch_static": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_uint32, C.POINTER(C.c_void_p),
                                              C.c_uint32, C.c_void_p]),
    "hyle_hip_static_scratch_bytes": (C.c_size_t, []),
    # include/hyle_hip_stream.h
    "hyle_hip_copy_batch_submit": (C.c_int, [C.c_void_p, C.POINTER(CopyPhaseC), C.c_uint32, C.POINTER(CopyRangeC),
                                             C.c_uint32, C.c_void_p]),
    "hyle_hip_file_pipeline_create": (C.c_int, [C.c_void_p, C.POINTER(FileStreamOptionsC), C.POINTER(C.c_void_p)]),
    "hyle_hip_file_pipeline_destroy": (None, [C.c_void_p]),
    "hyle_hip_file_pipeline_read": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(ReadRangeC), C.c_uint32, C.c_void_p,
                                              C.POINTER(StreamResultC)]),
    "hyle_hip_file_pipeline_wait": (C.c_int, [C.c_void_p]),
    "hyle_hip_file_pipeline_write": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(WriteRangeC), C.c_uint32, C.c_void_p,
                                               C.POINTER(StreamResultC)]),
    "hyle_hip_file_pipeline_submit_read": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(ReadRangeC), C.c_uint32, C.c_void_p,
                                                     C.POINTER(C.c_void_p)]),
    "hyle_hip_file_pipeline_submit_write": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(WriteRangeC), C.c_uint32,
                                                      C.c_void_p, C.POINTER(C.c_void_p)]),
    "hyle_hip_stream_ticket_result": (C.c_int, [C.c_void_p, C.POINTER(StreamResultC)]),
    "hyle_hip_stream_ticket_wait": (C.c_int, [C.c_void_p, C.POINTER(StreamResultC)]),
    "hyle_hip_stream_ticket_request_cancel": (None, [C.c_void_p]),
    "hyle_hip_stream_ticket_release": (None, [C.c_void_p]),
    # include/hyle_hip_backend.h
    "hyle_hip_backend_device_count": (C.c_int, [C.POINTER(C.c_size_t)]),
    "hyle_hip_backend_device_properties": (C.c_int, [C.c_size_t, C.POINTER(DevicePropertiesC)]),
    "hyle_hip_memory_resource_create": (C.c_int, [C.c_void_p, C.c_uint32, C.POINTER(C.c_void_p)]),
    "hyle_hip_memory_resource_destroy": (None, [C.c_void_p]),
    "hyle_hip_memory_resource_properties": (C.c_int, [C.c_void_p, C.POINTER(MemoryPropertiesC)]),
    "hyle_hip_memory_allocate": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, C.POINTER(C.c_void_p)]),
    "hyle_hip_memory_deallocate": (C.c_int, [C.c_void_p, C.c_void_p]),
    "hyle_hip_memory_resource_stats": (C.c_int, [C.c_void_p, C.POINTER(MemoryStatsC)]),
    "hyle_hip_backend_validate_resource": (C.c_int, [C.c_void_p, C.c_void_p]),
    "hyle_hip_queue_create": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
    "hyle_hip_queue_destroy": (None, [C.c_void_p]),
    "hyle_hip_queue_stream": (C.c_void_p, [C.c_void_p]),
    "hyle_hip_queue_reserve_completions": (C.c_int, [C.c_void_p, C.c_size_t]),
    "hyle_hip_queue_begin_sequence": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "hyle_hip_queue_finish_sequence": (C.c_void_p, [C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    "hyle_hip_completion_poll": (C.c_int, [C.c_void_p, C.POINTER(C.c_int)]),
    "hyle_hip_completion_wait": (C.c_int, [C.c_void_p]),
    "hyle_hip_completion_release": (None, [C.c_void_p]),
    "hyle_hip_queue_wait_completion": (C.c_int, [C.c_void_p, C.c_void_p]),
    "hyle_hip_backend_same_device": (C.c_int, [C.c_size_t, C.c_size_t]),
    "hyle_hip_queue_transfer_properties": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(TransferPropertiesC)]),
    "hyle_hip_queue_completion_endpoint": (C.c_int, [C.c_void_p, C.POINTER(CompletionEndpointC)]),
    "hyle_hip_queue_can_wait_endpoint": (C.c_int, [C.c_void_p, CompletionEndpointC]),
    "hyle_hip_queue_copy_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "hyle_hip_queue_fill_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint8, C.c_size_t]),
    "hyle_hip_queue_drain": (C.c_int, [C.c_void_p]),
    "hyle_hip_context_drain": (C.c_int, [C.c_void_p]),
}

_lib = None


def load() -> C.CDLL:
    """Load libhyle_hip.so and bind every symbol that include/hyle_hip.h, include/hyle_hip_stream.h and
    include/hyle_hip_backend.h declare."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the gfx950 library has not been built "
            "(run `python -m hyle_amd.build`); there is no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in EXPORTS.items():
        fn = getattr(lib, name)  # AttributeError here means the ABI and the header disagree
        fn.restype, fn.argtypes = restype, argtypes
    if lib.hyle_hip_abi_version() != ABI_VERSION:
        raise RuntimeError("libhyle_hip.so ABI version differs from hyle_amd/capi.py")
    _lib = lib
    return lib


def last_error() -> str:
    return load().hyle_hip_last_error().decode()


def status_name(code: int) -> str:
    return load().hyle_hip_status_name(code).decode()
