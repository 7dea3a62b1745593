"""The oracle's TopK(count = k), pinned without the GPU: the reference test's special-value rows,
an independent numpy ordering (lexsort on (NaN?, -value, index)) over random shapes, axes, both
directions and strided storage, and agreement with the separately pinned count = 1 routine."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc


def numpy_topk(x32: np.ndarray, count: int, axis: int, largest: bool):
    """x32: float32 array.  Stable: numbers before NaNs, best first, ties by index."""
    moved = np.moveaxis(x32, axis, -1)
    nan = np.isnan(moved)
    key = np.where(nan, 0.0, moved).astype(np.float64) + 0.0     # -0 -> compares equal to +0 anyway
    key = -key if largest else key
    index = np.broadcast_to(np.arange(moved.shape[-1]), moved.shape)
    order = np.lexsort((index, key, nan), axis=-1)[..., :count]  # last key is the primary one
    values = np.take_along_axis(moved, order, axis=-1)
    return np.moveaxis(values, -1, axis), np.moveaxis(order, -1, axis).astype(np.int32)


def test_reference_special_value_rows():
    # tests/graph_route_cuda/topk_test.cc:458-476 (count = 1, one row of 8193)
    width = 8193
    bits = np.full(width, 0xFF800000, np.uint32)
    bits[0], bits[1], bits[2] = 0x7FC12345, 0x80000000, 0
    values, indices = orc.topk(orc.F32, bits.view(np.float32), [1, width], 1)
    assert indices.tolist() == [[1]] and values.view(np.uint32).tolist() == [[0x80000000]]
    bits = (0x7FC03000 + np.arange(width)).astype(np.uint32)       # all NaN: index order
    values, indices = orc.topk(orc.F32, bits.view(np.float32), [1, width], 3)
    assert indices.tolist() == [[0, 1, 2]] and values.view(np.uint32).tolist() == [bits[:3].tolist()]
    bits = np.full(width, 0xBF800000, np.uint32)
    bits[5] = bits[width - 1] = 0x40A00000
    values, indices = orc.topk(orc.F32, bits.view(np.float32), [1, width], 3)
    assert indices.tolist() == [[5, width - 1, 0]]
    # smallest first: NaN is still last, -0 and +0 still tie by index
    row = np.array([np.nan, 0.0, -0.0, -1.0, np.inf, -np.inf, np.nan], np.float32)
    values, indices = orc.topk(orc.F32, row, [7], 7, largest=False)
    assert indices.tolist() == [5, 3, 1, 2, 4, 0, 6]
    values, indices = orc.topk(orc.F32, row, [7], 7, largest=True)
    assert indices.tolist() == [4, 1, 2, 3, 5, 0, 6]
    assert values.view(np.uint32)[1:3].tolist() == [0x00000000, 0x80000000]   # source bits are kept


@pytest.mark.parametrize("largest", [True, False])
def test_brute_force_shapes_axes_and_strides(largest):
    rng = np.random.default_rng(71)
    for dims, axis in (([5, 37], -1), ([4, 9, 6], 1), ([3, 2, 50], 0), ([300], 0), ([2, 3, 4, 5], 2)):
        x = rng.integers(-6, 7, dims).astype(np.float32) / 2          # many ties
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, max(1, flat.size // 9))] = np.nan
        flat[rng.integers(0, flat.size, max(1, flat.size // 9))] = -0.0
        for count in (1, 2, dims[axis] // 2, dims[axis]):
            want_values, want_indices = numpy_topk(x, count, axis, largest)
            values, indices = orc.topk(orc.F32, x, dims, count, axis, largest)
            assert np.array_equal(indices, want_indices)
            assert np.array_equal(values.view(np.uint32), want_values.view(np.uint32))
            # the same tensor stored transposed, reached through strides
            perm = list(reversed(range(len(dims))))
            stored = np.ascontiguousarray(np.transpose(x, perm))
            strides = [0] * len(dims)
            for position, a in enumerate(perm):
                strides[a] = stored.strides[position]
            again_values, again_indices = orc.topk(orc.F32, stored, dims, count, axis, largest, strides)
            assert np.array_equal(again_indices, want_indices)
            assert np.array_equal(again_values.view(np.uint32), want_values.view(np.uint32))


def test_count_one_agrees_with_the_argmax_routine_and_narrow_types_keep_bits():
    rng = np.random.default_rng(72)
    x = rng.normal(0, 1, (7, 1000)).astype(np.float32)
    x[2, 5] = x[2, 900] = 9.0
    x[3, :] = np.nan
    x[4, 0] = np.nan
    values, indices = orc.topk(orc.F32, x, x.shape, 1)
    v1, i1 = orc.topk1(x)
    assert np.array_equal(indices[:, 0], i1) and np.array_equal(values[:, 0].view(np.uint32), v1.view(np.uint32))
    for type_id in (orc.BF16, orc.F16):
        stored = orc.from_f32(type_id, x)
        values, indices = orc.topk(type_id, stored, x.shape, 5)
        wide = orc.to_f32(type_id, stored)
        want_values, want_indices = numpy_topk(wide, 5, -1, True)
        assert np.array_equal(indices, want_indices)
        assert np.array_equal(values, np.take_along_axis(stored, want_indices.astype(np.int64), axis=-1))
