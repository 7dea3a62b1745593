"""Every scalar type as storage: Copy, Fill, Select and Concat keep 1-, 2-, 4- and 8-byte elements
bit for bit whatever their type (include/hyle/compute/providers/cuda.h:19-24,42-46), checked
against the CPU oracle's width-only forms on dense, strided and broadcast operands."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gather_support import WORDS, byte_strides, lay_out
from gpu_support import DEVICE, context, note

pytestmark = pytest.mark.gpu

DT = hc.DataType
KINDS = [(DT.kFloat8E4M3FN, 1), (DT.kFloat8E5M2, 1), (DT.kUInt8, 1), (DT.kInt16, 2), (DT.kUInt16, 2), (DT.kBFloat16, 2),
         (DT.kUInt32, 4), (DT.kInt32, 4), (DT.kFloat64, 8), (DT.kInt64, 8), (DT.kUInt64, 8)]
RAW = {1: orc.RAW1, 2: orc.RAW2, 4: orc.RAW4, 8: orc.RAW8}


def on_device(raw: np.ndarray) -> torch.Tensor:
    flat = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    return torch.from_numpy(flat.copy()).to(DEVICE) if flat.size else torch.empty(16, dtype=torch.uint8, device=DEVICE)


def words(rng, shape, size):
    return rng.integers(0, 1 << 63, shape, dtype=np.uint64).astype(WORDS[size]) if size < 8 else \
        rng.integers(0, 1 << 63, shape, dtype=np.uint64) * np.uint64(2) + rng.integers(0, 2, shape, dtype=np.uint64)


def launch(operation, descs, buffers, out_shape, size, leads=None):
    prepared = hc.prepare(context(), operation, *descs)
    count = int(np.prod(out_shape)) if len(out_shape) else 1
    out = torch.full((count * size + 16,), 0x5A, dtype=torch.uint8, device=DEVICE)
    need = prepared.workspace_requirement()
    assert need.size == 0
    leads = leads or [0] * len(buffers)
    prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                        [b.data_ptr() + lead for b, lead in zip(buffers, leads)], [out.data_ptr()])
    torch.cuda.synchronize()
    host = out.cpu().numpy()
    assert (host[count * size:] == 0x5A).all()
    return host[:count * size].copy().view(WORDS[size]).reshape(out_shape), prepared


@pytest.mark.parametrize("kind,size", KINDS)
def test_copy_dense_and_strided(kind, size):
    rng = np.random.default_rng(int(kind))
    for shape, mode in (([3, 5, 7], 0), ([3, 5, 7], 1), ([4, 1, 6], 2), ([257, 130], 0), ([2, 2, 2, 2, 2, 2, 3], 1)):
        note(f"copy {kind.name} {shape} mode {mode}")
        strides = byte_strides(shape, size, 1, mode)
        storage, values = lay_out(words(rng, shape, size), strides, lead=size)
        desc = hc.TensorDesc.dense(kind, shape) if mode == 0 else hc.TensorDesc.strided_bytes(kind, shape, strides)
        got, _ = launch(hc.Copy(), [desc], [on_device(storage)], shape, size, leads=[size])
        want = orc.concat(RAW[size], [(storage[size:].copy(), shape, strides)], 0)   # a Concat of one part is a Copy
        assert np.array_equal(got, want) and np.array_equal(want, values)


@pytest.mark.parametrize("kind,size", KINDS)
def test_fill_keeps_the_pattern(kind, size):
    bits = 0xFFC00003_7FA5C3E1 & ((1 << (8 * size)) - 1)
    for shape in ([4099], [3, 5], [1], [64, 1024]):
        note(f"fill {kind.name} {shape}")
        got, _ = launch(hc.Fill(tuple(shape), kind, hc.ScalarValue.from_bits(kind, bits)), [], [], shape, size)
        want = orc.fill(RAW[size], shape, bits)
        assert np.array_equal(got, want) and (want == WORDS[size](bits)).all()


@pytest.mark.parametrize("kind,size", KINDS)
def test_select_flat_scalar_and_broadcast(kind, size):
    rng = np.random.default_rng(100 + int(kind))
    note(f"select {kind.name} flat")
    shape = [37, 129]
    flags = rng.integers(0, 2, shape).astype(np.uint8) * rng.integers(1, 256, shape).astype(np.uint8)
    a, b = words(rng, shape, size), words(rng, shape, size)
    descs = [hc.TensorDesc.dense(DT.kBool, shape), hc.TensorDesc.dense(kind, shape), hc.TensorDesc.dense(kind, shape)]
    got, _ = launch(hc.Select(), descs, [on_device(flags), on_device(a), on_device(b)], shape, size)
    want = orc.select(RAW[size], (flags, shape, None), (a, shape, None), (b, shape, None))
    assert np.array_equal(got, want) and np.array_equal(want, np.where(flags != 0, a, b))
    note(f"select {kind.name} rank-0 branch")
    zero = words(rng, [], size)
    descs[2] = hc.TensorDesc.dense(kind, [])
    got, _ = launch(hc.Select(), descs, [on_device(flags), on_device(a), on_device(zero)], shape, size)
    assert np.array_equal(got, np.where(flags != 0, a, zero))
    note(f"select {kind.name} broadcast and strided")
    row = words(rng, [129], size)
    column_flags = rng.integers(0, 2, [37, 1]).astype(np.uint8)
    strides = byte_strides(shape, size, 0, 1)
    storage, values = lay_out(a, strides)
    descs = [hc.TensorDesc.dense(DT.kBool, [37, 1]), hc.TensorDesc.strided_bytes(kind, shape, strides), hc.TensorDesc.dense(kind, [129])]
    got, _ = launch(hc.Select(), descs, [on_device(column_flags), on_device(storage), on_device(row)], shape, size)
    want = orc.select(RAW[size], (column_flags, [37, 1], None), (storage, shape, strides), (row, [129], None))
    assert np.array_equal(got, want) and np.array_equal(want, np.where(column_flags != 0, values, row[None, :]))


@pytest.mark.parametrize("kind,size", KINDS)
def test_concat_dense_and_strided(kind, size):
    rng = np.random.default_rng(200 + int(kind))
    for axis, mode in ((0, 0), (1, 0), (2, 0), (1, 1)):
        note(f"concat {kind.name} axis {axis} mode {mode}")
        parts, values, descs, buffers = [], [], [], []
        for extent in (3, 0, 4, 1):
            shape = [2, 6, 8]
            shape[axis] = extent
            strides = byte_strides(shape, size, axis, mode)
            storage, v = lay_out(words(rng, shape, size), strides)
            parts.append((storage, shape, strides))
            values.append(v)
            descs.append(hc.TensorDesc.dense(kind, shape) if mode == 0 else hc.TensorDesc.strided_bytes(kind, shape, strides))
            buffers.append(on_device(storage))
        out_shape = [2, 6, 8]
        out_shape[axis] = 8
        got, _ = launch(hc.Concat(axis), descs, buffers, out_shape, size)
        want = orc.concat(RAW[size], parts, axis)
        assert np.array_equal(got, want) and np.array_equal(want, np.concatenate(values, axis=axis))
