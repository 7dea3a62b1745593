"""The oracle's Concat against numpy.concatenate over raw words, in the shape of the reference
route test (tests/compute_route_vulkan/concat_test.cc:9-70: base shape [2, 3, 5], every axis, input
lengths 1 or (3 port + 1) % 4 on the axis -- zeros included --, byte strides that leave holes and
unaligned elements), plus the grouped form a caller with more than four inputs uses."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc

WORDS = {orc.BOOL: np.uint8, orc.BF16: np.uint16, orc.F32: np.uint32}


def strided_part(rng, dtype, shape):
    """Logical values and their storage with the reference test's hole-leaving byte strides."""
    size = np.dtype(dtype).itemsize
    strides = [size + 1, shape[2] * (shape[0] * (size + 1) + 3) + 5, shape[0] * (size + 1) + 3]
    values = rng.integers(0, int(np.iinfo(dtype).max) + 1, shape, dtype=np.uint64).astype(dtype)
    span = sum((d - 1) * s for d, s in zip(shape, strides)) + size if all(shape) else 0
    storage = rng.integers(0, 256, span + 8).astype(np.uint8)
    for index in np.ndindex(*shape):
        at = sum(i * s for i, s in zip(index, strides))
        storage[at:at + size] = np.frombuffer(values[index].tobytes(), np.uint8)
    return values, storage, strides


@pytest.mark.parametrize("type_id", sorted(WORDS))
@pytest.mark.parametrize("arity", [1, 2, 3, 4])
@pytest.mark.parametrize("axis", [0, 1, 2])
@pytest.mark.parametrize("pattern", [0, 1])
def test_reference_route_shapes(type_id, arity, axis, pattern):
    dtype = WORDS[type_id]
    rng = np.random.default_rng(arity * 100 + axis * 10 + pattern + type_id)
    values, parts = [], []
    for port in range(arity):
        shape = [2, 3, 5]
        shape[axis] = 1 if pattern == 0 else (port * 3 + 1) % 4
        v, storage, strides = strided_part(rng, dtype, shape)
        values.append(v)
        parts.append((storage, shape, strides))
    got = orc.concat(type_id, parts, axis - 3 if pattern else axis)
    want = np.concatenate(values, axis=axis)
    assert got.shape == want.shape and np.array_equal(got.view(dtype), want)


def test_groups_of_a_wider_concat_fill_one_output():
    rng = np.random.default_rng(3)
    widths = [0, 0, 0, 1, 2, 0, 3, 0, 5]   # tests/compute_route_vulkan/concat_test.cc:72-88 has runs of empty inputs
    values = [rng.integers(0, 1 << 32, (7, w, 3), dtype=np.uint64).astype(np.uint32) for w in widths]
    total = sum(widths)
    out = np.full((7, total, 3), 0xDEADBEEF, np.uint32)
    start = 0
    for first in range(0, len(values), 4):
        group = values[first:first + 4]
        orc.concat(orc.F32, [(v, list(v.shape), None) for v in group], 1, total=total, start=start, into=out.view(np.float32))
        start += sum(v.shape[1] for v in group)
    assert np.array_equal(out, np.concatenate(values, axis=1))
