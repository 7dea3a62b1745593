"""The oracle's Fill and Select against what fixes them: the reference route test's own
expectation (tests/compute_route_vulkan/tensor_test.cc:255-283: alternating Bool flags, a scalar
whose bits are a NaN payload or an odd byte, Select(mask, input, filled) keeps the input's bits
where the flag is set and the scalar's elsewhere), and numpy's broadcasting `where` over raw
words for broadcast, strided and rank-0 operands."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc

WORDS = {orc.BOOL: np.uint8, orc.F16: np.uint16, orc.BF16: np.uint16, orc.F32: np.uint32, orc.I32: np.uint32}
# the scalar bits tensor_test.cc:261-266 fills with, by element size
SCALAR_BITS = {1: 0xE3, 2: 0xFFC3, 4: 0xFFC00003}


def words(type_id, array):
    return np.ascontiguousarray(array).view(WORDS[type_id])


@pytest.mark.parametrize("type_id", sorted(WORDS))
@pytest.mark.parametrize("count", [1, 3, 5, 64, 257])
def test_reference_route_expectation(type_id, count):
    width = np.dtype(WORDS[type_id]).itemsize
    rng = np.random.default_rng(count * 8 + type_id)
    raw = rng.integers(0, 1 << (8 * width), count, dtype=np.uint64).astype(WORDS[type_id])
    flags = (np.arange(count) % 2).astype(np.uint8)
    bits = 1 if type_id == orc.BOOL else SCALAR_BITS[width]
    filled = orc.fill(type_id, [count], bits)
    assert words(type_id, filled).tolist() == [bits] * count
    selected = orc.select(type_id, (flags, [count], None), (raw, [count], None), (filled, [count], None))
    expected = raw.copy()
    expected[flags == 0] = bits
    assert words(type_id, selected).tolist() == expected.tolist()


def test_fill_keeps_only_the_low_bytes_and_every_shape():
    assert orc.fill(orc.F32, [2, 0, 3], 0x3F800000).shape == (2, 0, 3)
    assert orc.fill(orc.F32, [], 0x3F800000).view(np.float32).item() == 1.0
    assert words(orc.BF16, orc.fill(orc.BF16, [3, 2], 0x12343F80)).tolist() == [[0x3F80] * 2] * 3


@pytest.mark.parametrize("type_id", [orc.BOOL, orc.BF16, orc.F32])
@pytest.mark.parametrize("shapes", [
    ([4, 1, 6], [5, 6], [4, 5, 1]),     # every operand broadcast on a different axis
    ([3, 7], [], [7]),                   # rank-0 first branch, row second branch
    ([1], [2, 3, 4], [2, 3, 4]),         # one condition byte for everything
    ([2, 3, 4], [2, 3, 4], []),          # the graph route's masked residual: scalar zero branch
])
def test_select_is_numpy_where_over_words(type_id, shapes):
    dtype = WORDS[type_id]
    rng = np.random.default_rng(len(shapes[0]) * 131 + type_id)
    condition = rng.integers(0, 3, shapes[0]).astype(np.uint8)   # 2 counts as true: any non-zero byte
    condition.reshape(-1)[::5] = 0x80
    first = rng.integers(0, np.iinfo(dtype).max, shapes[1], dtype=np.uint64).astype(dtype)
    second = rng.integers(0, np.iinfo(dtype).max, shapes[2], dtype=np.uint64).astype(dtype)
    got = orc.select(type_id, (condition, shapes[0], None), (first, shapes[1], None), (second, shapes[2], None))
    want = np.where(condition != 0, first, second)
    assert got.shape == want.shape
    assert np.array_equal(words(type_id, got), want)


def test_select_reads_strided_operands_by_byte_offset():
    # a transposed first branch, a condition with a hole after every byte, a column second branch
    rng = np.random.default_rng(5)
    base = rng.integers(0, 1 << 32, (6, 4), dtype=np.uint64).astype(np.uint32)        # logical [4, 6] transposed
    holes = rng.integers(0, 2, (4, 6, 2)).astype(np.uint8)                             # stride 2 along the last axis
    column = rng.integers(0, 1 << 32, (4, 1), dtype=np.uint64).astype(np.uint32)
    got = orc.select(orc.F32, (holes, [4, 6], [12, 2]), (base, [4, 6], [4, 16]), (column, [4, 1], None))
    want = np.where(holes[:, :, 0] != 0, base.T, column)
    assert np.array_equal(words(orc.F32, got), want)
