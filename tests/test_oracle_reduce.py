"""The oracle's Reduce over any axes, pinned without the GPU: the reference tests' known answers,
numpy brute force over random shapes, axis sets and permuted / padded / unaligned strides, and
agreement with the separately pinned last-axis routine."""
from __future__ import annotations

import itertools

import numpy as np
import pytest

from oracle import lib as orc

KINDS = {"sum": orc.SUM, "mean": orc.MEAN, "min": orc.MIN, "max": orc.MAX}


def numpy_reduce(kind, x64, axes, keep=False):
    axes = tuple(range(x64.ndim)) if axes is None else tuple(a % x64.ndim for a in axes)
    with np.errstate(invalid="ignore", divide="ignore"), np.testing.suppress_warnings() as sup:
        sup.filter(RuntimeWarning)
        if kind == "sum":
            return np.sum(x64, axis=axes, keepdims=keep)
        if kind == "mean":
            return np.mean(x64, axis=axes, keepdims=keep)  # NaN for an empty reduction
        fn = np.min if kind == "min" else np.max
        identity = np.inf if kind == "min" else -np.inf
        return fn(x64, axis=axes, keepdims=keep, initial=identity)  # NaN propagates in numpy too


def test_reference_known_answers():
    # tests/compute_provider_native/reduction_test.cc:46-80: every mode across the last axis
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    for kind, want in (("sum", [6, 15]), ("mean", [2, 5]), ("min", [1, 4]), ("max", [3, 6])):
        assert orc.reduce(KINDS[kind], orc.F32, x, x.shape, [1]).tolist() == want
    # :82-128: axes {0, 2} of [2, 2, 2], with and without kept dimensions
    x = np.arange(1, 9, dtype=np.float32).reshape(2, 2, 2)
    assert orc.reduce(orc.SUM, orc.F32, x, x.shape, [0, 2]).tolist() == [14, 22]
    kept = orc.reduce(orc.SUM, orc.F32, x, x.shape, [0, 2], keep_dimensions=True)
    assert kept.shape == (1, 2, 1) and kept.reshape(-1).tolist() == [14, 22]
    # :130-165: byte strides {10, 4} (rows not 4-byte aligned), a NaN among the values, all axes
    raw = np.zeros(18, np.uint8)
    for offset, value in zip((0, 4, 10, 14), (0.0, -0.0, 3.0, np.nan)):
        raw[offset:offset + 4] = np.frombuffer(np.float32(value).tobytes(), np.uint8)
    out = orc.reduce(orc.MIN, orc.F32, raw, [2, 2], None, [10, 4])
    assert out.shape == () and np.isnan(out)
    # :167-181: the minimum of zeros of both signs is -0
    zeros = np.zeros(37, np.float32)
    zeros[1] = zeros[19] = -0.0
    assert np.signbit(orc.reduce(orc.MIN, orc.F32, zeros, [37]))
    assert not np.signbit(orc.reduce(orc.MAX, orc.F32, zeros, [37]))
    # :183-222: an empty reduced extent writes 0, NaN, +inf, -inf
    empty = np.zeros((2, 0), np.float32)
    assert orc.reduce(orc.SUM, orc.F32, empty, [2, 0], [1]).tolist() == [0, 0]
    assert np.all(np.isnan(orc.reduce(orc.MEAN, orc.F32, empty, [2, 0], [1])))
    assert orc.reduce(orc.MIN, orc.F32, empty, [2, 0], [1]).tolist() == [np.inf, np.inf]
    assert orc.reduce(orc.MAX, orc.F32, empty, [2, 0], [1]).tolist() == [-np.inf, -np.inf]


@pytest.mark.parametrize("kind", list(KINDS))
def test_brute_force_every_axis_subset_dense_and_permuted(kind):
    rng = np.random.default_rng(41)
    shape = (3, 4, 2, 5)
    x = rng.normal(0, 2, shape).astype(np.float32)
    x[1, 2, 0, 3] = np.nan
    x[0, 0, 0, 0], x[0, 0, 0, 1] = 0.0, -0.0
    for count in range(1, 5):
        for axes in itertools.combinations(range(4), count):
            want = numpy_reduce(kind, x.astype(np.float64), axes)
            got = orc.reduce(KINDS[kind], orc.F32, x, shape, axes).astype(np.float64)
            assert got.shape == want.shape
            assert np.array_equal(np.isnan(got), np.isnan(want))
            ok = ~np.isnan(want)
            if kind in ("min", "max"):
                assert np.array_equal(got[ok], want[ok])
            else:
                assert np.allclose(got[ok], want[ok], rtol=1e-6, atol=1e-5)
            # the same logical tensor through permuted storage: strides of the transposed array
            for perm in ((3, 1, 0, 2), (1, 0, 3, 2)):
                stored = np.ascontiguousarray(np.transpose(x, perm))       # storage order
                strides = [0] * 4
                for position, axis in enumerate(perm):
                    strides[axis] = stored.strides[position]
                again = orc.reduce(KINDS[kind], orc.F32, stored, shape, axes, strides).astype(np.float64)
                assert np.array_equal(np.isnan(again), np.isnan(want))
                if kind in ("min", "max"):
                    assert np.array_equal(again[ok], want[ok])
                else:
                    assert np.allclose(again[ok], want[ok], rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("type_id", [orc.F32, orc.BF16, orc.F16], ids=["f32", "bf16", "f16"])
def test_agrees_with_the_last_axis_routine_and_rounds_once(type_id):
    rng = np.random.default_rng(42)
    x32 = rng.normal(0, 2, (6, 5, 33)).astype(np.float32)
    x = x32 if type_id == orc.F32 else orc.from_f32(type_id, x32)
    for kind in KINDS.values():
        a = orc.reduce(kind, type_id, x, x.shape, [-1])
        b = orc.reduce_last_axis(kind, type_id, x)
        assert a.tobytes() == b.tobytes()
    # narrow storage: f32 accumulation, one rounding at the end
    if type_id != orc.F32:
        wide = orc.to_f32(type_id, x)
        want = orc.from_f32(type_id, orc.reduce(orc.SUM, orc.F32, wide, wide.shape, [0, 2]))
        assert orc.reduce(orc.SUM, type_id, x, x.shape, [0, 2]).tobytes() == want.tobytes()


def test_unaligned_narrow_strides_and_padded_rows():
    rng = np.random.default_rng(43)
    values = orc.from_f32(orc.BF16, rng.normal(0, 1, (4, 6)).astype(np.float32))
    raw = np.zeros(4 * 15 + 2, np.uint8)          # rows 15 bytes apart, elements 2 bytes apart
    for r in range(4):
        raw[r * 15:r * 15 + 12] = values[r].view(np.uint8)
    for axes in ([0], [1], None):
        got = orc.reduce(orc.MAX, orc.BF16, raw, [4, 6], axes, [15, 2])
        want = orc.reduce(orc.MAX, orc.BF16, values, [4, 6], axes)
        assert got.tobytes() == want.tobytes()
