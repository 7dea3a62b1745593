"""The copy endpoint and the file -> pinned staging -> HBM pipeline (through the C ABI):
bytes arrive unchanged, whatever the cut into slots; Q8_0 weights streamed from a file dequantise
to the oracle's values; errors report how far the call came."""
from __future__ import annotations

import os
import tempfile

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from hyle_amd import file_stream as fs
from oracle import lib as orc

from gpu_support import DEVICE, context, note, run

pytestmark = pytest.mark.gpu


def stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


@pytest.fixture
def data_file():
    rng = np.random.default_rng(1300)
    payload = rng.integers(0, 256, 6 * 1024 * 1024 + 12345, dtype=np.uint8)
    with tempfile.NamedTemporaryFile(delete=False) as handle:
        handle.write(payload.tobytes())
        path = handle.name
    fd = os.open(path, os.O_RDONLY)
    yield payload, fd
    os.close(fd)
    os.unlink(path)


def test_file_ranges_arrive_unchanged_for_every_cut(data_file):
    payload, fd = data_file
    total = payload.size
    for slots, slot_bytes in ((2, 1 << 20), (1, 4096), (3, 100_000), (8, 1 << 16)):
        pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(slots, slot_bytes))
        # ragged ranges: tiny, empty, unaligned offsets, larger than a slot, up to the last byte
        spans = [(0, 1), (7, 0), (13, 4095), (4096 * 3 + 1, 300_001), (1_000_003, 2_500_000), (total - 5, 5)]
        buffers = [torch.zeros(max(size, 1), dtype=torch.uint8, device=DEVICE) for _, size in spans]
        ranges = [fs.StreamReadRange(offset, buffer.data_ptr(), size) for (offset, size), buffer in zip(spans, buffers)]
        note(f"file pipeline {slots} slots of {slot_bytes} bytes, {len(spans)} ranges")
        result = pipeline.read(fd, ranges, stream_handle())
        pipeline.wait()
        assert result.status == 0 and result.ready_ranges == len(spans) == result.total_ranges
        assert result.read_bytes == result.copied_bytes == sum(size for _, size in spans)
        for (offset, size), buffer in zip(spans, buffers):
            assert np.array_equal(buffer.cpu().numpy()[:size], payload[offset:offset + size])
        # a second call reuses the slots while the first call's copies may still be in flight
        whole = torch.zeros(total, dtype=torch.uint8, device=DEVICE)
        result = pipeline.read(fd, [fs.StreamReadRange(0, whole.data_ptr(), total)], stream_handle())
        torch.cuda.current_stream().synchronize()
        assert np.array_equal(whole.cpu().numpy(), payload)
        if slots * slot_bytes < total:
            assert result.host_waits > 0
        pipeline.close()


def test_file_pipeline_errors_keep_their_progress(data_file):
    payload, fd = data_file
    total = payload.size
    pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(2, 1 << 16))
    first = torch.zeros(1000, dtype=torch.uint8, device=DEVICE)
    beyond = torch.zeros(200_000, dtype=torch.uint8, device=DEVICE)
    note("file pipeline: a range that runs past the end of the file")
    with pytest.raises(hc.StatusError) as err:
        pipeline.read(fd, [fs.StreamReadRange(10, first.data_ptr(), 1000),
                           fs.StreamReadRange(total - 100_000, beyond.data_ptr(), 200_000)], stream_handle())
    assert err.value.is_out_of_range()
    progress = pipeline.last_result
    assert progress.ready_ranges == 1 and progress.total_ranges == 2 and 1000 <= progress.read_bytes < 201_000
    pipeline.wait()
    assert np.array_equal(first.cpu().numpy(), payload[10:1010])
    with pytest.raises(hc.StatusError) as err:
        pipeline.read(-1, [], stream_handle())
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(65, 4096))
    assert err.value.is_invalid_argument()
    pipeline.close()


def test_copy_batch_phases_and_validation():
    rng = np.random.default_rng(1301)
    host = torch.from_numpy(rng.integers(0, 256, 1 << 20, dtype=np.uint8)).pin_memory()
    device_a = torch.zeros(1 << 20, dtype=torch.uint8, device=DEVICE)
    device_b = torch.zeros(1 << 19, dtype=torch.uint8, device=DEVICE)
    back = torch.zeros(1 << 19, dtype=torch.uint8).pin_memory()
    note("copy batch: host -> device, device -> device, device -> host in three phases")
    phases = [fs.CopyPhase(0, 1), fs.CopyPhase(0b1, 2), fs.CopyPhase(0b11, 3)]
    ranges = [fs.CopyRange(device_b.data_ptr(), back.data_ptr(), 1 << 19, 2),          # listed first, runs last
              fs.CopyRange(host.data_ptr(), device_a.data_ptr(), 1 << 20, 0),
              fs.CopyRange(device_a.data_ptr() + 4096, device_b.data_ptr(), 1 << 19, 1),
              fs.CopyRange(0, 0, 0, 1)]
    fs.submit_copy_batch(context(), phases, ranges, stream_handle())
    torch.cuda.current_stream().synchronize()
    assert torch.equal(device_a.cpu(), host)
    assert torch.equal(back, host[4096:4096 + (1 << 19)])
    for bad_phases, bad_ranges in (([fs.CopyPhase(0b1, 0)], []),                              # depends on itself
                                   ([fs.CopyPhase(0, 0), fs.CopyPhase(0b100, 0)], []),        # on a later phase
                                   ([fs.CopyPhase()], [fs.CopyRange(host.data_ptr(), device_a.data_ptr(), 8, 1)]),
                                   ([fs.CopyPhase()], [fs.CopyRange(0, device_a.data_ptr(), 8, 0)])):
        with pytest.raises(hc.StatusError) as err:
            fs.submit_copy_batch(context(), bad_phases, bad_ranges, stream_handle())
        assert err.value.is_invalid_argument()


def test_q8_0_weights_streamed_from_a_file_dequantise_to_the_oracle():
    rng = np.random.default_rng(1302)
    rows, k = 96, 2048
    row_bytes = k // 32 * 34
    blocks = rng.integers(0, 256, (rows, row_bytes), dtype=np.uint8)
    scales = rng.normal(0, 0.05, (rows, k // 32)).astype(np.float16)
    blocks.reshape(rows, k // 32, 34)[:, :, :2] = scales.view(np.uint8).reshape(rows, k // 32, 2)
    header = rng.integers(0, 256, 1237, dtype=np.uint8)          # the tensor starts at an odd file offset
    with tempfile.NamedTemporaryFile(delete=False) as handle:
        handle.write(header.tobytes())
        handle.write(blocks.tobytes())
        path = handle.name
    fd = os.open(path, os.O_RDONLY)
    try:
        weights = torch.zeros(rows * row_bytes, dtype=torch.uint8, device=DEVICE)
        pipeline = fs.FileResourcePipeline.create(context(), fs.FileStreamOptions(2, 64 * 1024))
        note("Q8_0 blocks: file -> staging -> HBM -> dequant")
        pipeline.read(fd, [fs.StreamReadRange(header.size, weights.data_ptr(), rows * row_bytes)], stream_handle())
        desc = hc.TensorDesc.gguf_q8_0_weight(hc.DataType.kBFloat16, k, rows)
        out, sumsq = run(hc.Q8_0DequantSumSquares(), weights, descs=[desc])   # same stream: ordered after the copies
        pipeline.close()
        want, want_sumsq = orc.q8_0_dequant_bf16(blocks, rows, k)[:2]
        got = out.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, want)
        assert np.allclose(sumsq.cpu().numpy(), want_sumsq, rtol=1e-5)
    finally:
        os.close(fd)
        os.unlink(path)
