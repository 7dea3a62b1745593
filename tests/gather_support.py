"""Layouts of the reference's Gather tests (tests/compute_provider_cuda/collectives_test_support.h:
36-48,257-314): mode 0 dense, mode 1 byte strides of element size + 1 (holes, unaligned elements),
mode 2 the same with stride 0 on one axis; values i -> 0x7fc000018123 + i * 0x9e3779b1 truncated to
the element, indices (3 i + 1) % extent."""
from __future__ import annotations

import numpy as np

WORDS = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}


def byte_strides(shape, size: int, axis: int, mode: int):
    if mode == 0:
        strides, step = [], size
        for d in reversed(shape):
            strides.append(step)
            step *= max(int(d), 1)
        return list(reversed(strides))
    strides, step = [0] * len(shape), size + 1
    for d in range(len(shape) - 1, -1, -1):
        strides[d] = 0 if (mode == 2 and d == axis) else step
        step *= max(int(shape[d]), 1)
    return strides


def lay_out(values: np.ndarray, strides, lead: int = 0):
    """Storage bytes (0xa5 elsewhere) holding `values` at the byte strides, `lead` bytes in; and
    the logical values read back (later writes win where a stride is 0)."""
    size = values.dtype.itemsize
    shape = values.shape
    count = int(np.prod(shape)) if len(shape) else 1
    span = (sum((d - 1) * s for d, s in zip(shape, strides)) + size) if count else 0
    storage = np.full(lead + span + 32, 0xA5, np.uint8)
    flat = values.reshape(-1)
    offsets = np.zeros(count, np.int64)
    if count:
        grids = np.indices(shape).reshape(len(shape), -1) if len(shape) else np.zeros((0, 1), np.int64)
        for axis, stride in enumerate(strides):
            offsets += grids[axis] * stride
    raw = flat.view(np.uint8).reshape(count, size) if count else np.zeros((0, size), np.uint8)
    for i in range(count):  # in logical order, so that later elements win
        storage[lead + offsets[i]:lead + offsets[i] + size] = raw[i]
    back = np.zeros(count, values.dtype)
    view = back.view(np.uint8).reshape(count, size) if count else back.view(np.uint8).reshape(0, size)
    for i in range(count):
        view[i] = storage[lead + offsets[i]:lead + offsets[i] + size]
    return storage, back.reshape(shape)


def reference_values(shape, size: int, boolean: bool = False) -> np.ndarray:
    count = int(np.prod(shape)) if len(shape) else 1
    i = np.arange(count, dtype=np.uint64)
    if boolean:
        return (i & np.uint64(1)).astype(np.uint8).reshape(shape)
    with np.errstate(over="ignore"):
        words = np.uint64(0x7FC000018123) + i * np.uint64(0x9E3779B1)
    return words.astype(WORDS[size]).reshape(shape)


def reference_indices(index_shape, extent: int, wide: bool) -> np.ndarray:
    count = int(np.prod(index_shape)) if len(index_shape) else 1
    ids = (np.arange(count, dtype=np.int64) * 3 + 1) % extent
    return ids.astype(np.int64 if wide else np.int32).reshape(index_shape)


def expected(values: np.ndarray, indices: np.ndarray, axis: int) -> np.ndarray:
    return np.take(values, indices.astype(np.int64), axis=axis)
