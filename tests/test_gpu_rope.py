"""Parity of RoPE (through the C ABI) with the CPU oracle.  The arithmetic is f32 with cos / sin
from the device's math library where the oracle uses libm's, so agreement is to tolerance: 4e-6
of the pair's magnitude for f32 (the reference's own tests allow 1e-5, tests/compute_provider_ggml/
cpu_provider_test.cc:1752-1753), and for f16 / bf16 one unit in the last place of the result on top
of that; elements past rotary_dimensions are bit-exact."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, context, note, to_device, to_host

pytestmark = pytest.mark.gpu

DT = hc.DataType


def rope_on_device(tag, storage, positions, frequencies, rotary, sequence_axis, half_split, in_place=False, offset=0):
    kind = TYPES[tag][0]
    layout = hc.RopeLayout.kHalfSplit if half_split else hc.RopeLayout.kInterleaved
    position_kind = DT.kInt64 if positions.dtype.itemsize == 8 else DT.kInt32
    prepared = hc.prepare(context(), hc.RoPE(rotary, sequence_axis, layout), hc.TensorDesc.dense(kind, storage.shape),
                          hc.TensorDesc.dense(position_kind, positions.shape), hc.TensorDesc.dense(DT.kFloat32, frequencies.shape))
    assert prepared.output_description() == hc.TensorDesc.dense(kind, storage.shape)
    assert prepared.workspace_requirement().size == 0 and prepared.alias_support(0, 0)
    size = storage.dtype.itemsize
    raw = np.zeros(storage.size * size + 64, np.uint8)
    raw[offset:offset + storage.size * size] = storage.reshape(-1).view(np.uint8)
    source = torch.from_numpy(raw).to(DEVICE)
    target = source if in_place else torch.full_like(source, 0x5A)
    ids = torch.from_numpy(np.ascontiguousarray(positions)).to(DEVICE)
    freq = torch.from_numpy(np.ascontiguousarray(frequencies, np.float32)).to(DEVICE)
    if storage.size:
        prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                            [source.data_ptr() + offset, ids.data_ptr(), freq.data_ptr()], [target.data_ptr() + offset])
    torch.cuda.synchronize()
    host = target.cpu().numpy()
    if not in_place:
        assert (host[:offset] == 0x5A).all() and (host[offset + storage.size * size:] == 0x5A).all()
    return host[offset:offset + storage.size * size].copy().view(storage.dtype).reshape(storage.shape)


def check(tag, values, positions, frequencies, rotary, sequence_axis=-2, half_split=False, **kwargs):
    type_id = TYPES[tag][1]
    storage = values if tag == "f32" else orc.from_f32(type_id, values)
    want = orc.rope(type_id, storage, positions, frequencies, rotary, sequence_axis, half_split)
    got = rope_on_device(tag, storage, positions, frequencies, rotary, sequence_axis, half_split, **kwargs)
    pairs = rotary // 2
    first = slice(0, pairs) if half_split else slice(0, rotary, 2)
    second = slice(pairs, rotary) if half_split else slice(1, rotary, 2)
    logical = values if tag == "f32" else orc.to_f32(type_id, storage)
    magnitude = np.abs(logical[..., first]) + np.abs(logical[..., second])
    if tag == "f32":
        got_values, want_values, unit = got, want, 0.0
    else:
        # the f32 results differ by the trigonometric functions' last places; after the one rounding to
        # storage that is at most one unit in the last place of the result on top
        got_values, want_values = orc.to_f32(type_id, got), orc.to_f32(type_id, want)
        unit = 2.0 ** -7 if tag == "bf16" else 2.0 ** -10
    for part in (first, second):
        allowed = 4e-6 * magnitude + unit * np.maximum(np.abs(want_values[..., part]), 2.0 ** -14 if tag == "f16" else 0.0) + 1e-30
        assert np.all(np.abs(got_values[..., part].astype(np.float64) - want_values[..., part]) <= allowed)
    assert np.array_equal(got[..., rotary:].view(np.uint8), want[..., rotary:].view(np.uint8))
    return got


@pytest.mark.parametrize("tag", ["f32", "f16", "bf16"])
def test_reference_known_answers(tag):
    positions, frequencies = np.array([0, 2], np.int32), np.array([0.5, 0.25], np.float32)
    note(f"rope known answers {tag}")
    check(tag, np.arange(1, 9, dtype=np.float32).reshape(1, 2, 1, 4), positions, frequencies, 4, sequence_axis=1)
    for half_split in (False, True):
        got = check(tag, np.arange(1, 17, dtype=np.float32).reshape(1, 2, 1, 8), positions, frequencies, 4, sequence_axis=1,
                    half_split=half_split)
        if tag == "f32":
            c1, s1 = np.cos(1.0), np.sin(1.0)
            want = 9 * c1 - (11 if half_split else 10) * s1
            assert abs(got.reshape(-1)[8] - want) <= 1e-5


def test_long_positions_keep_their_phase():
    positions = np.array([0, 2380, 65536], np.int32)
    frequencies = np.array([0.4728708267211914, -0.25, 0.0, 0.00137], np.float32)
    values = ((np.arange(120) % 29 - 14) / 8.0).astype(np.float32).reshape(2, 3, 2, 10)
    for half_split in (False, True):
        note(f"rope long positions half_split={half_split}")
        check("f32", values, positions, frequencies, 8, sequence_axis=1, half_split=half_split)
    note("rope positions up to 2^40")
    far = np.array([1 << 20, (1 << 31) + 5, (1 << 40) + 12345], np.int64)
    check("f32", values, far, frequencies, 8, sequence_axis=1)


@pytest.mark.parametrize("tag,shape,rotary,axis", [
    ("bf16", (1, 512, 16, 128), 128, 1), ("f32", (2, 33, 4, 64), 64, 1), ("f16", (3, 40, 2, 96), 64, 1),
    ("f32", (2, 5, 3, 16), 12, 1), ("bf16", (7, 3, 24), 10, 0), ("f32", (5, 2, 2, 2, 8), 8, -2), ("f16", (9, 130), 130, 0),
    ("f32", (2, 3, 5, 8192), 8192, 1),   # a table of phases too large for LDS: every thread takes its own
])
def test_shapes_layouts_and_operand_forms(tag, shape, rotary, axis):
    rng = np.random.default_rng(sum(shape) + rotary)
    values = rng.normal(0, 1, shape).astype(np.float32)
    normal = axis + len(shape) if axis < 0 else axis
    steps, pairs = shape[normal], rotary // 2
    base = (10000.0 ** (-np.arange(pairs) / pairs)).astype(np.float32)
    for half_split in (False, True):
        note(f"rope {tag} {shape} rotary {rotary} axis {axis} half_split {half_split}")
        check(tag, values, rng.integers(0, 8192, steps).astype(np.int32), base, rotary, axis, half_split)
        check(tag, values, rng.integers(0, 8192, shape[:normal + 1]).astype(np.int64), rng.uniform(0, 1, (steps, pairs)).astype(np.float32),
              rotary, axis, half_split)
        check(tag, values, np.arange(steps, dtype=np.int32), base, rotary, axis, half_split, in_place=True)
        check(tag, values, np.arange(steps, dtype=np.int32), base, rotary, axis, half_split, offset=values.dtype.itemsize if tag == "f32" else 2)


def test_empty_and_rejected():
    assert hc.prepare(context(), hc.RoPE(4, 1), hc.TensorDesc.dense(DT.kFloat32, [0, 3, 8]), hc.TensorDesc.dense(DT.kInt32, [3]),
                      hc.TensorDesc.dense(DT.kFloat32, [2])).dispatch_count() == 0
    with pytest.raises(hc.StatusError) as err:   # the schema admits every float, the kernels three
        hc.prepare(context(), hc.RoPE(4, 1), hc.TensorDesc.dense(DT.kFloat64, [2, 3, 8]), hc.TensorDesc.dense(DT.kInt32, [3]),
                   hc.TensorDesc.dense(DT.kFloat32, [2]))
    assert err.value.is_unimplemented()


def test_prefill_sized_rotation():
    note("rope [1, 8192, 16, 128] bf16 half-split")
    rng = np.random.default_rng(3)
    values = rng.normal(0, 1, (1, 8192, 16, 128)).astype(np.float32)
    base = (1000000.0 ** (-np.arange(64) / 64.0)).astype(np.float32)
    check("bf16", values, np.arange(8192, dtype=np.int32), base, 128, 1, True)
