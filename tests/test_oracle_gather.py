"""The oracle's Gather against numpy.take over raw words, in the shape of the reference's tests
(tests/compute_provider_cuda/gather_collectives_test.cc:13-24,143-170: source [2, 7, 3], axes 0, 1,
-1, dense and hole-leaving strides for source and indices, every element width, both index widths,
a rank-8 source, a rank-0 index, 2-D indices) and their checked failures (…:176-212: -1, the
extent, the largest and the smallest index leave the output as it was)."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc

from gather_support import WORDS, byte_strides, expected, lay_out, reference_indices, reference_values


def run(shape, axis, index_shape, source_mode, index_mode, size, wide, checked=True):
    rank = len(shape)
    normal = axis + rank if axis < 0 else axis
    strides = byte_strides(shape, size, normal, source_mode)
    storage, values = lay_out(reference_values(shape, size), strides, lead=size)
    index_axis = len(index_shape) - 1 if index_shape else 0
    width = 8 if wide else 4
    index_strides = byte_strides(index_shape, width, index_axis, index_mode)
    index_storage, ids = lay_out(reference_indices(index_shape, shape[normal], wide), index_strides, lead=width)
    status, got = orc.gather(storage[size:].copy(), shape, strides, axis, index_storage[width:].copy(), index_shape,
                             index_strides, checked=checked, width=size, wide=wide,
                             into=np.zeros(list(shape[:normal]) + list(index_shape) + list(shape[normal + 1:]), WORDS[size]))
    return status, got, expected(values, ids, normal)


@pytest.mark.parametrize("size", [1, 2, 4, 8])
@pytest.mark.parametrize("wide", [False, True])
def test_reference_matrix(size, wide):
    for axis in (0, 1, -1):
        for source_mode in (0, 1):
            for index_mode in (0, 1):
                status, got, want = run([2, 7, 3], axis, [2, 3], source_mode, index_mode, size, wide)
                assert status == 0 and got.shape == want.shape and np.array_equal(got, want), (axis, source_mode, index_mode)


def test_reference_special_shapes():
    status, got, want = run([1, 2, 1, 3, 1, 5, 2, 1], 5, [4], 1, 1, 8, True)
    assert status == 0 and np.array_equal(got, want)
    status, got, want = run([2, 1, 7, 3, 1, 2], 2, [], 2, 0, 2, False)   # a rank-0 index drops the axis
    assert status == 0 and got.shape == (2, 1, 3, 1, 2) and np.array_equal(got, want)
    status, got, want = run([4, 3], 0, [2, 3], 0, 2, 1, True)            # indices broadcast along their last axis
    assert status == 0 and np.array_equal(got, want)


@pytest.mark.parametrize("wide", [False, True])
def test_checked_failure_writes_nothing(wide):
    source = np.arange(1, 13, dtype=np.uint64).reshape(4, 3)
    kind = np.int64 if wide else np.int32
    limits = np.iinfo(kind)
    for invalid in (-1, 4, limits.max, limits.min):
        ids = np.array([0, invalid], kind)
        kept = np.array([[8, 7, 6], [5, 4, 3]], np.uint64)
        status, out = orc.gather(source, [4, 3], None, 0, ids, [2], None, checked=True, into=kept.copy())
        assert status == 1 and np.array_equal(out, kept)
    status, out = orc.gather(source, [4, 3], None, 0, np.array([3, 1], kind), [2], None)
    assert status == 0 and np.array_equal(out, [[10, 11, 12], [4, 5, 6]])


def test_empty_cases():
    # tests/compute_provider_cuda/gather_collectives_test.cc:304-327: empty output is fine whatever the indices say
    source = np.zeros((4, 0), np.uint32)
    status, out = orc.gather(source, [4, 0], None, 0, np.array([-1, 7], np.int32), [2], None)
    assert status == 0 and out.shape == (2, 0)
    status, out = orc.gather(np.arange(4, dtype=np.uint32), [4], None, 0, np.zeros(0, np.int32), [0], None)
    assert status == 0 and out.shape == (0,)
    # src/compute_provider_native/indexing.cc:189-195: an empty axis cannot be indexed
    status, _ = orc.gather(np.zeros((0, 3), np.uint32), [0, 3], None, 0, np.array([0], np.int32), [1], None, checked=False)
    assert status == 1
