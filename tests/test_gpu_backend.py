"""The HIP backend (include/hyle_hip_backend.h) through its C ABI, by byte identity: devices, memory
resources, queue-ordered copy and fill, sequences and completions, waits across queues; and the
write direction, tickets and cancellation of the file pipeline (include/hyle_hip_stream.h).  In the
shape of the reference's backend tests (tests/compute_backend_cuda: allocate, transfer, complete)."""
from __future__ import annotations

import ctypes as C
import os
import tempfile
import time

import numpy as np
import pytest
import torch

from hyle_amd import backend as hb
from hyle_amd import capi
from hyle_amd import compute as hc
from hyle_amd import file_stream as fs

from gpu_support import DEVICE, context, note

pytestmark = pytest.mark.gpu


def host_view(address: int, size: int) -> np.ndarray:
    return np.ctypeslib.as_array((C.c_uint8 * size).from_address(address))


def test_devices_and_properties():
    assert hb.device_count() >= 1
    props = hb.device_properties(0)
    assert props.architecture.startswith("gfx950") and props.compute_units == context().compute_units
    assert props.asynchronous_queues and not props.unified_memory and props.total_memory_bytes > (64 << 30)
    with pytest.raises(hc.StatusError) as missing:
        hb.device_properties(hb.device_count())
    assert missing.value.is_out_of_range()


def test_memory_resources_allocate_account_and_validate():
    ctx = context()
    device, pinned = hb.MemoryResource(ctx, hb.MemoryKind.kDevice), hb.MemoryResource(ctx, hb.MemoryKind.kPinnedHost)
    flags, alignment, _ = device.properties()
    assert flags == hb.MemoryProperty.kDeviceAccessible and alignment == 256
    flags, _, _ = pinned.properties()
    assert flags & hb.MemoryProperty.kHostPinned and flags & hb.MemoryProperty.kHostAccessible
    assert flags & hb.MemoryProperty.kDeviceAccessible and flags & hb.MemoryProperty.kHostAddressIdentity
    hb.validate_resource(ctx, device)
    a = device.allocate(1000)
    b = device.allocate(5000, 4096)
    assert a % 256 == 0 and b % 4096 == 0
    assert device.stats()[:3] == (6000, 6000, 2)
    device.deallocate(a)
    assert device.stats() == (5000, 6000, 1, 2)
    with pytest.raises(hc.StatusError):
        device.deallocate(a)                         # not (any longer) an allocation of this resource
    with pytest.raises(hc.StatusError):
        device.allocate(0)
    with pytest.raises(hc.StatusError):
        device.allocate(64, 48)                      # alignment is not a power of two
    device.deallocate(b)
    device.close()
    pinned.close()


def test_copy_fill_sequences_and_completions_by_byte_identity():
    ctx = context()
    device, pinned = hb.MemoryResource(ctx, hb.MemoryKind.kDevice), hb.MemoryResource(ctx, hb.MemoryKind.kPinnedHost)
    queue = hb.Queue(ctx)
    queue.reserve_completions(4)
    size = (3 << 20) + 77
    rng = np.random.default_rng(1900)
    payload = rng.integers(0, 256, size, dtype=np.uint8)
    h_in, h_out = pinned.allocate(size), pinned.allocate(size)
    d_a, d_b = device.allocate(size), device.allocate(size)
    host_view(h_in, size)[:] = payload
    host_view(h_out, size)[:] = 0
    note("backend: pinned -> device -> device -> pinned inside one sequence")
    queue.begin_sequence()
    with pytest.raises(hc.StatusError) as twice:
        queue.begin_sequence()                       # one sequence per queue at a time
    assert twice.value.code == hc.StatusCode.kFailedPrecondition
    queue.copy_async(device, d_a, pinned, h_in, size)
    queue.copy_async(device, d_b, device, d_a, size)
    queue.fill_async(device, d_b + 5, 0xAB, 1001)    # unaligned start, odd length
    queue.copy_async(pinned, h_out, device, d_b, size)
    done = queue.finish_sequence(accepted=True)
    done.wait()
    assert done.poll()
    want = payload.copy()
    want[5:1006] = 0xAB
    assert np.array_equal(host_view(h_out, size), want)
    done.release()
    note("backend: fill of every length 0..70 at every offset 0..17")
    for offset in range(18):
        for length in (0, 1, 2, 15, 16, 17, 31, 33, 64, 70):
            queue.fill_async(device, d_a, 0, 256)
            queue.fill_async(device, d_a + offset, 0x5C, length)
    queue.fill_async(device, d_a, 0, 256)
    queue.fill_async(device, d_a + 3, 0x5C, 70)
    queue.copy_async(pinned, h_out, device, d_a, 256)
    queue.drain()
    want = np.zeros(256, np.uint8)
    want[3:73] = 0x5C
    assert np.array_equal(host_view(h_out, 256), want)
    note("backend: a rejected sequence completes at once with its status; ranges are checked")
    queue.begin_sequence()
    with pytest.raises(hc.StatusError) as outside:
        queue.copy_async(device, d_a + size - 10, pinned, h_in, 100)
    assert outside.value.is_out_of_range()
    with pytest.raises(hc.StatusError) as host_fill:
        queue.fill_async(pinned, h_out, 1, 16)
    assert host_fill.value.is_unimplemented()
    failed = queue.finish_sequence(accepted=False, terminal=capi.OUT_OF_RANGE)
    assert failed.poll()
    with pytest.raises(hc.StatusError) as terminal:
        failed.wait()
    assert terminal.value.is_out_of_range()
    failed.release()
    for address, resource in ((h_in, pinned), (h_out, pinned), (d_a, device), (d_b, device)):
        resource.deallocate(address)
    queue.close()
    device.close()
    pinned.close()


def test_a_queue_waits_for_another_queues_completion():
    ctx = context()
    device, pinned = hb.MemoryResource(ctx, hb.MemoryKind.kDevice), hb.MemoryResource(ctx, hb.MemoryKind.kPinnedHost)
    producer, consumer = hb.Queue(ctx), hb.Queue(ctx)
    size = 64 << 20
    d_src, d_dst = device.allocate(size), device.allocate(size)
    h_out = pinned.allocate(4096)
    note("backend: consumer queue ordered after the producer's sequence")
    producer.begin_sequence()
    for value in (1, 2, 3, 4, 5, 6, 7):              # a few large fills: the last one decides the bytes
        producer.fill_async(device, d_src, value, size)
    filled = producer.finish_sequence()
    consumer.wait_completion(filled)
    consumer.copy_async(device, d_dst, device, d_src, size)
    consumer.copy_async(pinned, h_out, device, d_dst + size - 4096, 4096)
    consumer.drain()
    assert np.all(host_view(h_out, 4096) == 7)
    filled.release()
    hb.drain_context(ctx)
    for queue in (producer, consumer):
        queue.close()
    device.close()
    pinned.close()


def test_endpoints_say_which_completions_a_queue_may_wait_for_and_which_copies_are_direct():
    """BackendVTable::completion_endpoint / can_wait_endpoint / transfer_properties / same_device
    (src/compute/backend_internal.h:22-23,45-47,57-62): Graph asks them cold, before it lets one
    queue wait for another's completion without a host wait, or records a copy as queue-ordered."""
    ctx = context()
    device, pinned = hb.MemoryResource(ctx, hb.MemoryKind.kDevice), hb.MemoryResource(ctx, hb.MemoryKind.kPinnedHost)
    producer, consumer = hb.Queue(ctx), hb.Queue(ctx)
    note("backend: endpoints of two queues of one device")
    own, other = consumer.completion_endpoint(), producer.completion_endpoint()
    assert own.valid() and other.valid()
    assert own.authority == other.authority and own.identity != other.identity   # one library, two ordered queues
    assert consumer.completion_endpoint() == own                                  # stable
    assert consumer.can_wait_endpoint(other) and consumer.can_wait_endpoint(own) and producer.can_wait_endpoint(own)
    # a foreign endpoint (another authority), an invalid one, and one without identity are refused
    assert not consumer.can_wait_endpoint(hb.CompletionEndpoint(other.authority + 8, other.identity))
    assert not consumer.can_wait_endpoint(hb.CompletionEndpoint())
    assert not consumer.can_wait_endpoint(hb.CompletionEndpoint(other.authority, 0))
    # what can_wait_endpoint promised holds: the consumer accepts the producer's pending completion
    size = 32 << 20
    d_src, h_out = device.allocate(size), pinned.allocate(4096)
    producer.begin_sequence()
    for value in (9, 8, 7):
        producer.fill_async(device, d_src, value, size)
    filled = producer.finish_sequence()
    consumer.wait_completion(filled)
    consumer.copy_async(pinned, h_out, device, d_src + size - 4096, 4096)
    consumer.drain()
    assert np.all(host_view(h_out, 4096) == 7)
    filled.release()
    note("backend: transfer properties of every resource pair")
    for destination, source in ((device, device), (device, pinned), (pinned, device), (pinned, pinned)):
        route = consumer.transfer_properties(destination, source)
        assert route.mode == hb.TransferMode.kQueuedDirect and not route.peer
    for destination, source in ((device, None), (None, pinned)):
        with pytest.raises(hc.StatusError) as unsupported:
            consumer.transfer_properties(destination, source)
        assert unsupported.value.is_unimplemented()
    assert hb.same_device(0, 0)
    assert not hb.same_device(0, hb.device_count())       # an index that names no device
    device.deallocate(d_src)
    pinned.deallocate(h_out)
    for queue in (producer, consumer):
        queue.close()
    device.close()
    pinned.close()


def test_provider_launches_on_a_backend_queue():
    """The stream a provider enqueues on is the queue's (cuda::stream(sequence) in the reference)."""
    ctx = context()
    queue = hb.Queue(ctx)
    x = torch.arange(-8, 8, dtype=torch.float32, device=DEVICE)
    out = torch.empty_like(x)
    torch.cuda.synchronize()
    prepared = hc.prepare(ctx, hc.Unary(hc.UnaryKind.kRelu), hc.TensorDesc.dense(hc.DataType.kFloat32, [16]))
    queue.begin_sequence()
    prepared.create_invocation().submit(queue.stream, [x.data_ptr()], [out.data_ptr()])
    done = queue.finish_sequence()
    done.wait()
    assert torch.equal(out, torch.relu(x))
    done.release()
    queue.close()


# ---- the file pipeline: device -> file, tickets, cancellation ---------------------------------
def stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


def test_device_ranges_reach_the_file_unchanged_and_come_back():
    rng = np.random.default_rng(1901)
    total = 5 * 1024 * 1024 + 321
    payload = torch.from_numpy(rng.integers(0, 256, total, dtype=np.uint8)).to(DEVICE)
    host = payload.cpu().numpy()
    for slots, slot_bytes in ((2, 1 << 20), (1, 4096), (3, 100_000)):
        with tempfile.NamedTemporaryFile(delete=False) as handle:
            path = handle.name
        fd = os.open(path, os.O_RDWR)
        try:
            pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(slots, slot_bytes))
            # ragged ranges written to scattered file offsets: tiny, empty, larger than a slot
            spans = [(0, 1, 10), (9, 0, 50), (100, 4095, 4096), (70_001, 300_001, 1_000_000),
                     (1_000_003, 2_500_000, 2_000_000), (total - 5, 5, 4_600_000)]
            ranges = [fs.StreamWriteRange(payload.data_ptr() + source, offset, size) for source, size, offset in spans]
            note(f"file pipeline write {slots} slots of {slot_bytes} bytes")
            result = pipeline.write(fd, ranges, stream_handle())
            assert result.status == 0 and result.complete == 1 and result.ready_ranges == len(spans)
            assert result.written_bytes == result.copied_bytes == sum(size for _, size, _ in spans)
            written = np.fromfile(path, dtype=np.uint8)
            for source, size, offset in spans:
                assert np.array_equal(written[offset:offset + size], host[source:source + size])
            # and back through the read direction of the same pipeline
            back = torch.zeros(2_500_000, dtype=torch.uint8, device=DEVICE)
            pipeline.read(fd, [fs.StreamReadRange(2_000_000, back.data_ptr(), 2_500_000)], stream_handle())
            pipeline.wait()
            assert torch.equal(back, payload[1_000_003:1_000_003 + 2_500_000])
            pipeline.close()
        finally:
            os.close(fd)
            os.unlink(path)


def test_tickets_report_progress_and_cancellation_keeps_what_was_done():
    rng = np.random.default_rng(1902)
    total = 48 * 1024 * 1024
    payload = rng.integers(0, 256, total, dtype=np.uint8)
    with tempfile.NamedTemporaryFile(delete=False) as handle:
        handle.write(payload.tobytes())
        path = handle.name
    fd = os.open(path, os.O_RDWR)
    try:
        pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(2, 64 * 1024))
        target = torch.zeros(total, dtype=torch.uint8, device=DEVICE)
        note("file pipeline: a read behind a ticket")
        ticket = pipeline.submit_read(fd, [fs.StreamReadRange(0, target.data_ptr(), total)], stream_handle())
        with pytest.raises(hc.StatusError) as busy:   # one request at a time
            pipeline.read(fd, [fs.StreamReadRange(0, target.data_ptr(), 16)], stream_handle())
        assert busy.value.code == hc.StatusCode.kFailedPrecondition
        result = ticket.wait()
        assert result.status == 0 and result.complete == 1 and result.copied_bytes == total
        assert np.array_equal(target.cpu().numpy(), payload)
        ticket.close()
        note("file pipeline: a read cancelled at a slot boundary")
        target.zero_()
        torch.cuda.synchronize()
        ticket = pipeline.submit_read(fd, [fs.StreamReadRange(0, target.data_ptr(), total)], stream_handle())
        ticket.request_cancel()
        try:  # the request may also have finished before it saw the cancellation: both are valid ends
            ticket.wait()
            assert ticket.last_result.copied_bytes == total and ticket.last_result.ready_ranges == 1
        except hc.StatusError as stopped:
            assert stopped.code == hc.StatusCode.kCancelled
            assert ticket.last_result.complete == 1 and ticket.last_result.status == capi.CANCELLED
            assert ticket.last_result.copied_bytes < total and ticket.last_result.copied_bytes % (64 * 1024) == 0
            assert ticket.last_result.ready_ranges == 0
        progress = ticket.last_result
        torch.cuda.synchronize()
        got = target.cpu().numpy()
        assert np.array_equal(got[:progress.copied_bytes], payload[:progress.copied_bytes])   # what was done stands
        assert not got[progress.copied_bytes:].any()                                            # nothing beyond it
        ticket.close()
        note("file pipeline: a write behind a ticket, then one cancelled")
        source = torch.from_numpy(payload[::-1].copy()).to(DEVICE)
        ticket = pipeline.submit_write(fd, [fs.StreamWriteRange(source.data_ptr(), 0, total)], stream_handle())
        seen = ticket.result()
        assert seen.complete in (0, 1) and seen.written_bytes <= total
        result = ticket.wait()
        assert result.written_bytes == total and result.ready_ranges == 1
        assert np.array_equal(np.fromfile(path, dtype=np.uint8), payload[::-1])
        ticket.close()
        ticket = pipeline.submit_write(fd, [fs.StreamWriteRange(target.data_ptr(), 0, total)], stream_handle())
        ticket.request_cancel()
        try:
            ticket.wait()
        except hc.StatusError as stopped_write:
            assert stopped_write.code == hc.StatusCode.kCancelled
            assert ticket.last_result.written_bytes < total
        ticket.close()
        # the pipeline is usable again after a cancelled request
        small = torch.zeros(4096, dtype=torch.uint8, device=DEVICE)
        pipeline.read(fd, [fs.StreamReadRange(total - 4096, small.data_ptr(), 4096)], stream_handle())
        pipeline.wait()
        pipeline.close()
    finally:
        os.close(fd)
        os.unlink(path)


def test_a_pipeline_closed_under_a_running_ticket_ends_the_request_first():
    """Destroying the pipeline while a ticket's thread still fills and drains the pinned slots must
    stop that thread before the slots are freed; the ticket stays valid, reports where it stopped,
    and what it copied stands.  While the request runs, the pipeline's own wait is refused."""
    rng = np.random.default_rng(1903)
    total = 64 * 1024 * 1024
    payload = rng.integers(0, 256, total, dtype=np.uint8)
    with tempfile.NamedTemporaryFile(delete=False) as handle:
        handle.write(payload.tobytes())
        path = handle.name
    fd = os.open(path, os.O_RDWR)
    try:
        for direction in ("read", "write"):
            pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(2, 64 * 1024))
            target = torch.zeros(total, dtype=torch.uint8, device=DEVICE)
            torch.cuda.synchronize()
            note(f"file pipeline: closed while a {direction} runs behind a ticket")
            if direction == "read":
                ticket = pipeline.submit_read(fd, [fs.StreamReadRange(0, target.data_ptr(), total)], stream_handle())
            else:
                ticket = pipeline.submit_write(fd, [fs.StreamWriteRange(target.data_ptr(), 0, total)], stream_handle())
            try:
                pipeline.wait()
                assert ticket.result().complete == 1   # only an ended request leaves the pipeline to its caller
            except hc.StatusError as refused:
                assert refused.code == hc.StatusCode.kFailedPrecondition
            pipeline.close()                            # the request's thread has ended when this returns
            seen = ticket.result()
            assert seen.complete == 1
            try:
                ticket.wait()
            except hc.StatusError as stopped:
                assert stopped.code == hc.StatusCode.kCancelled
            done = ticket.last_result
            assert done.complete == 1 and done.copied_bytes <= total
            if direction == "read":
                torch.cuda.synchronize()
                got = target.cpu().numpy()
                assert np.array_equal(got[:done.copied_bytes], payload[:done.copied_bytes])
                assert not got[done.copied_bytes:].any()
            ticket.close()                              # after its pipeline: must not look for it
        # and the other order: the ticket released first, then the pipeline
        pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(2, 64 * 1024))
        ticket = pipeline.submit_read(fd, [fs.StreamReadRange(0, target.data_ptr(), total)], stream_handle())
        ticket.close()
        pipeline.close()
        torch.cuda.synchronize()
    finally:
        os.close(fd)
        os.unlink(path)
