"""Parity of Concat (through the C ABI) with the CPU oracle: bit-exact, storage only.

The first test is the reference route test's matrix (tests/compute_route_vulkan/concat_test.cc:9-70:
base shape [2, 3, 5], every axis counted from either end, one to four inputs -- and five and nine in
groups of four --, lengths that include zero, byte strides that leave holes and unaligned elements);
then empty groups (…:72-88), the broadcast input repeated (…:96-110), dense shapes that take the
16-byte path, overlap rejection and a benchmark-sized join."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, context, note

pytestmark = pytest.mark.gpu

DT = hc.DataType
KINDS = {DT.kBool: (orc.BOOL, np.uint8), DT.kBFloat16: (orc.BF16, np.uint16), DT.kFloat16: (orc.F16, np.uint16),
         DT.kFloat32: (orc.F32, np.uint32), DT.kInt32: (orc.I32, np.uint32), DT.kInt8: (orc.BOOL, np.uint8)}


def device_bytes(raw: np.ndarray) -> torch.Tensor:
    flat = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    if flat.size == 0:
        return torch.empty(16, dtype=torch.uint8, device=DEVICE)
    return torch.from_numpy(flat.copy()).to(DEVICE)


def strided_part(rng, dtype, shape):
    size = np.dtype(dtype).itemsize
    strides = [size + 1, shape[2] * (shape[0] * (size + 1) + 3) + 5, shape[0] * (size + 1) + 3]
    values = rng.integers(0, int(np.iinfo(dtype).max) + 1, shape, dtype=np.uint64).astype(dtype)
    span = sum((d - 1) * s for d, s in zip(shape, strides)) + size if all(shape) else 0
    storage = rng.integers(0, 256, span + 8).astype(np.uint8)
    for index in np.ndindex(*shape):
        at = sum(i * s for i, s in zip(index, strides))
        storage[at:at + size] = np.frombuffer(values[index].tobytes(), np.uint8)
    return values, storage, strides


def concat_on_device(kind: DT, parts, axis: int):
    """parts: (storage, dims, byte_strides or None).  More than four go in groups into one output."""
    dtype = KINDS[kind][1]
    rank = len(parts[0][1])
    normal = axis + rank if axis < 0 else axis
    total = sum(int(p[1][normal]) for p in parts)
    shape = list(parts[0][1])
    shape[normal] = total
    count = int(np.prod(shape))
    out = torch.full((max(count, 1) * np.dtype(dtype).itemsize,), 0x5A, dtype=torch.uint8, device=DEVICE)
    stream = torch.cuda.current_stream().cuda_stream
    start, dispatches, kept = 0, 0, []
    for first in range(0, len(parts), 4):
        group = parts[first:first + 4]
        descs = [hc.TensorDesc.dense(kind, p[1]) if p[2] is None else hc.TensorDesc.strided_bytes(kind, p[1], p[2]) for p in group]
        grouped = len(parts) > 4
        prepared = hc.prepare(context(), hc.Concat(axis, total if grouped else 0, start if grouped else 0), *descs)
        assert prepared.output_description() == hc.TensorDesc.dense(kind, shape)
        tensors = [device_bytes(p[0]) for p in group]
        kept.append(tensors)
        prepared.create_invocation().submit(stream, [t.data_ptr() for t in tensors], [out.data_ptr()])
        dispatches += prepared.dispatch_count()
        start += sum(int(p[1][normal]) for p in group)
    torch.cuda.synchronize()
    host = out.cpu().numpy()[:count * np.dtype(dtype).itemsize]
    return host.view(dtype).reshape(shape), dispatches


@pytest.mark.parametrize("kind", [DT.kFloat32, DT.kBFloat16, DT.kBool])
def test_reference_route_matrix(kind):
    type_id, dtype = KINDS[kind]
    for arity in (1, 2, 3, 4, 5, 9):
        for axis in range(3):
            for pattern in range(2):
                note(f"concat {kind.name} arity {arity} axis {axis} pattern {pattern}")
                rng = np.random.default_rng(arity * 100 + axis * 10 + pattern + int(kind))
                values, parts = [], []
                for port in range(arity):
                    shape = [2, 3, 5]
                    shape[axis] = 1 if pattern == 0 else (port * 3 + 1) % 4
                    v, storage, strides = strided_part(rng, dtype, shape)
                    values.append(v)
                    parts.append((storage, shape, strides))
                got, _ = concat_on_device(kind, parts, axis - 3 if pattern else axis)
                want = np.concatenate(values, axis=axis)
                assert got.shape == want.shape and np.array_equal(got, want)
                if arity <= 4:
                    oracle = orc.concat(type_id, parts, axis)
                    assert np.array_equal(oracle.view(dtype), want)


def test_empty_groups_and_a_repeated_broadcast_input():
    rng = np.random.default_rng(21)
    for widths in ([0, 0, 0, 1, 2, 0, 0, 0, 0], [0, 0, 0, 0, 0]):
        note(f"concat int32 [7, w, 3] widths {widths}")
        values = [rng.integers(0, 1 << 32, (7, w, 3), dtype=np.uint64).astype(np.uint32) for w in widths]
        got, dispatches = concat_on_device(DT.kInt32, [(v, list(v.shape), None) for v in values], 1)
        assert np.array_equal(got, np.concatenate(values, axis=1))
        assert dispatches == sum(1 for g in range(0, len(widths), 4) if sum(widths[g:g + 4]))   # empty groups launch nothing
    note("concat: nine times the same broadcast element (concat_test.cc:96-110)")
    one = np.array([0x7FC5], np.uint16)
    shape = [1, 1, 1, 2, 1, 3, 1, 5]
    part = (one, shape, [2, 2, 2, 0, 2, 0, 2, 0])
    got, _ = concat_on_device(DT.kBFloat16, [part] * 9, -1)
    assert got.shape == (1, 1, 1, 2, 1, 3, 1, 45) and (got == 0x7FC5).all()


def test_dense_inputs_take_whole_vectors_or_elements():
    rng = np.random.default_rng(22)
    for kind, shapes, axis in ((DT.kFloat32, [[64, 128], [64, 256], [64, 4]], 1),      # 16-byte runs and offsets
                               (DT.kBFloat16, [[3, 7, 5], [3, 2, 5], [3, 9, 5]], 1),    # odd runs: element steps
                               (DT.kInt8, [[5, 33], [2, 33]], 0),
                               (DT.kFloat16, [[4, 6, 8], [4, 6, 24]], -1)):
        dtype = KINDS[kind][1]
        note(f"concat dense {kind.name} {shapes} axis {axis}")
        values = [rng.integers(0, int(np.iinfo(dtype).max) + 1, s, dtype=np.uint64).astype(dtype) for s in shapes]
        got, dispatches = concat_on_device(kind, [(v, list(v.shape), None) for v in values], axis)
        assert dispatches == 1 and np.array_equal(got, np.concatenate(values, axis=axis))


def test_schema_admission_and_overlap():
    ctx = context()
    D = hc.TensorDesc.dense
    with pytest.raises(hc.StatusError) as err:   # rank 0 has no axis
        hc.prepare(ctx, hc.Concat(0), D(DT.kFloat32, []))
    assert err.value.code == hc.StatusCode.kOutOfRange
    for bad in ([D(DT.kFloat32, [2, 3]), D(DT.kBFloat16, [2, 3])], [D(DT.kFloat32, [2, 3]), D(DT.kFloat32, [2, 3, 1])],
                [D(DT.kFloat32, [2, 3]), D(DT.kFloat32, [4, 3])]):
        with pytest.raises(hc.StatusError) as err:
            hc.prepare(ctx, hc.Concat(1), *bad)
        assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:   # a group that does not fit its output
        hc.prepare(ctx, hc.Concat(0, total=5, start=3), D(DT.kFloat32, [3, 2]))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    prepared = hc.prepare(ctx, hc.Concat(0), D(DT.kFloat32, [4, 8]), D(DT.kFloat32, [4, 8]))
    assert prepared.route_name() == "concat" and not prepared.alias_support(0, 0) and not prepared.alias_support(0, 1)
    note("concat: an input inside the output is rejected (no alias, no overlap)")
    storage = torch.zeros(1024, dtype=torch.uint8, device=DEVICE)
    with pytest.raises(hc.StatusError) as err:
        prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                            [storage.data_ptr() + 512, storage.data_ptr() + 128], [storage.data_ptr()])
    assert err.value.code == hc.StatusCode.kInvalidArgument


def test_benchmark_sized_join():
    note("concat bf16 [8192, 2048] + [8192, 4096] along the last axis")
    left = torch.randint(-32768, 32767, (8192, 2048), dtype=torch.int16, device=DEVICE)
    right = torch.randint(-32768, 32767, (8192, 4096), dtype=torch.int16, device=DEVICE)
    D = hc.TensorDesc.dense
    prepared = hc.prepare(context(), hc.Concat(-1), D(DT.kBFloat16, [8192, 2048]), D(DT.kBFloat16, [8192, 4096]))
    out = torch.empty((8192, 6144), dtype=torch.int16, device=DEVICE)
    prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream, [left.data_ptr(), right.data_ptr()], [out.data_ptr()])
    torch.cuda.synchronize()
    assert torch.equal(out, torch.cat([left, right], dim=1))
