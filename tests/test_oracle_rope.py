"""The oracle's RoPE against the reference tests' known answers (tests/compute_provider_ggml/
cpu_provider_test.cc:1571-1760: f16 / bf16 / f32 data [1, 2, 1, 4 or 8], positions {0, 2},
frequencies {0.5, 0.25}, both layouts, a partial tail; positions {0, 2380, 65536} with the
frequencies of the long-phase test), a float64 rotation, and what rotations obey."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc


def stored(type_id, values):
    values = np.asarray(values, np.float32)
    return values if type_id == orc.F32 else orc.from_f32(type_id, values)


def as_f32(type_id, storage):
    return storage if type_id == orc.F32 else orc.to_f32(type_id, storage)


def near(type_id, got, want):
    # tests/compute_provider_native/half_test_support.h expect_near: the storage type's resolution
    tolerance = {orc.F32: 1e-5, orc.F16: 2e-3, orc.BF16: 1.6e-2}[type_id]
    return np.all(np.abs(got.astype(np.float64) - want) <= tolerance * np.maximum(1.0, np.abs(want)))


@pytest.mark.parametrize("type_id", [orc.F16, orc.BF16, orc.F32])
def test_reference_known_answers(type_id):
    positions, frequencies = np.array([0, 2], np.int32), np.array([0.5, 0.25], np.float32)
    c1, s1, c5, s5 = np.cos(1.0), np.sin(1.0), np.cos(0.5), np.sin(0.5)
    data = stored(type_id, np.arange(1, 9).reshape(1, 2, 1, 4))
    got = as_f32(type_id, orc.rope(type_id, data, positions, frequencies, 4, sequence_axis=1))
    want = [1, 2, 3, 4, 5 * c1 - 6 * s1, 5 * s1 + 6 * c1, 7 * c5 - 8 * s5, 7 * s5 + 8 * c5]
    assert near(type_id, got.reshape(-1), np.array(want))
    data = stored(type_id, np.arange(1, 17).reshape(1, 2, 1, 8))
    want = np.arange(1, 17, dtype=np.float64)
    want[8:12] = [9 * c1 - 11 * s1, 10 * c5 - 12 * s5, 9 * s1 + 11 * c1, 10 * s5 + 12 * c5]
    got = as_f32(type_id, orc.rope(type_id, data, positions, frequencies, 4, sequence_axis=1, half_split=True))
    assert near(type_id, got.reshape(-1), want)
    want[8:12] = [9 * c1 - 10 * s1, 9 * s1 + 10 * c1, 11 * c5 - 12 * s5, 11 * s5 + 12 * c5]
    got = as_f32(type_id, orc.rope(type_id, data, positions, frequencies, 4, sequence_axis=1))
    assert near(type_id, got.reshape(-1), want)


@pytest.mark.parametrize("half_split", [False, True])
def test_long_positions_keep_their_phase_and_the_tail_passes(half_split):
    positions = np.array([0, 2380, 65536], np.int32)
    frequencies = np.array([0.4728708267211914, -0.25, 0.0, 0.00137], np.float32)
    values = ((np.arange(120) % 29 - 14) / 8.0).astype(np.float32).reshape(2, 3, 2, 10)
    got = orc.rope(orc.F32, values, positions, frequencies, 8, sequence_axis=1, half_split=half_split).reshape(12, 10)
    flat = values.reshape(12, 10)
    for row in range(12):
        for pair in range(4):
            first = pair if half_split else 2 * pair
            second = first + (4 if half_split else 1)
            phase = float(np.float32(positions[(row // 2) % 3]) * frequencies[pair])
            a, b = float(flat[row, first]), float(flat[row, second])
            assert abs(got[row, first] - (a * np.cos(phase) - b * np.sin(phase))) <= 1e-5
            assert abs(got[row, second] - (a * np.sin(phase) + b * np.cos(phase))) <= 1e-5
        assert np.array_equal(got[row, 8:].view(np.uint32), flat[row, 8:].view(np.uint32))


def test_rotations_obey_their_laws():
    rng = np.random.default_rng(11)
    data = rng.normal(0, 1, (2, 5, 3, 16)).astype(np.float32)
    frequencies = (10000.0 ** (-np.arange(6) / 6.0)).astype(np.float32)
    zero = np.zeros(5, np.int64)
    for half_split in (False, True):
        same = orc.rope(orc.F32, data, zero, frequencies, 12, half_split=half_split, sequence_axis=1)
        assert np.array_equal(same, data)                                # position 0 is the identity
        still = orc.rope(orc.F32, data, np.arange(5, dtype=np.int32), np.zeros(6, np.float32), 12, half_split=half_split,
                         sequence_axis=1)
        assert np.array_equal(still, data)                               # so is frequency 0
        positions = rng.integers(0, 4096, (2, 5)).astype(np.int32)       # batched positions, per-step frequencies
        stepped = rng.uniform(0, 1, (5, 6)).astype(np.float32)
        got = orc.rope(orc.F32, data, positions, stepped, 12, half_split=half_split, sequence_axis=1).astype(np.float64)
        first = slice(0, 6) if half_split else slice(0, 12, 2)
        second = slice(6, 12) if half_split else slice(1, 12, 2)
        a, b = data[..., first].astype(np.float64), data[..., second].astype(np.float64)
        phase = (positions.astype(np.float32)[:, :, None] * stepped[None, :, :]).astype(np.float64)[:, :, None, :]
        assert np.allclose(got[..., first], a * np.cos(phase) - b * np.sin(phase), atol=2e-6, rtol=0)
        assert np.allclose(got[..., second], a * np.sin(phase) + b * np.cos(phase), atol=2e-6, rtol=0)
        assert np.allclose(got[..., first] ** 2 + got[..., second] ** 2, a * a + b * b, rtol=1e-5)   # a rotation keeps norms
        assert np.array_equal(got[..., 12:], data[..., 12:].astype(np.float64))
