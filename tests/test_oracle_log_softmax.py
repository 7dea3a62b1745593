"""The oracle's LogSoftmax, pinned without the GPU: the reference tests' known answers and tail
cases, a float64 closed form, and consistency with the separately pinned softmax."""
from __future__ import annotations

import numpy as np

from oracle import lib as orc


def closed_form(x64):
    peak = x64.max(axis=-1, keepdims=True)
    return x64 - peak - np.log(np.exp(x64 - peak).sum(axis=-1, keepdims=True))


def test_reference_known_answers():
    # tests/compute_provider_native/transformer_test.cc:303-337 (axis 1 of [1, 3, 2] = these rows)
    rows = np.array([[1, 2, 3], [10, 20, 30]], np.float32)
    s0 = 3.0 + np.log(np.exp(-2.0) + np.exp(-1.0) + 1.0)
    s1 = 30.0 + np.log(np.exp(-20.0) + np.exp(-10.0) + 1.0)
    want = np.array([[1 - s0, 2 - s0, 3 - s0], [10 - s1, 20 - s1, 30 - s1]])
    got = orc.softmax(orc.F32, rows, log=True).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 4e-6 + 2e-7)


def test_reference_tail_cases_near_one_and_equal_maxima():
    # tests/compute_provider_cuda/tensor_test.cc:1168-1199: -20 everywhere but one, two or all zeros
    for type_id in (orc.F32, orc.BF16, orc.F16):
        for width in (129, 8193):
            x = np.full((3, width), -20.0, np.float32)
            x[0, width - 1] = 0
            x[1, 0] = x[1, width - 1] = 0
            x[2, :] = 0
            stored = x if type_id == orc.F32 else orc.from_f32(type_id, x)
            got = orc.softmax(type_id, stored, log=True)
            got = (got if type_id == orc.F32 else orc.to_f32(type_id, got)).astype(np.float64)
            for row, maxima in ((0, 1), (1, 2), (2, width)):
                partition = np.log(maxima) + np.log1p((width - maxima) * np.exp(-20.0) / maxima)
                want = x[row].astype(np.float64) - partition
                if type_id == orc.F32:
                    assert np.all(np.abs(got[row] - want) <= np.abs(want) * 4e-6 + 2e-7)
                else:
                    rounded = orc.to_f32(type_id, orc.from_f32(type_id, want.astype(np.float32))).astype(np.float64)
                    step = 2.0 ** (-7 if type_id == orc.BF16 else -10)
                    assert np.all(np.abs(got[row] - rounded) <= np.abs(rounded) * step)


def test_closed_form_masks_and_undefined_rows():
    rng = np.random.default_rng(81)
    x = rng.normal(0, 4, (9, 257)).astype(np.float32)
    got = orc.softmax(orc.F32, x, scale=0.5, log=True).astype(np.float64)
    want = closed_form(0.5 * x.astype(np.float64))
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6)
    # exp(log_softmax) is the (bit-exactly pinned) softmax within rounding
    soft = orc.softmax(orc.F32, x, scale=0.5).astype(np.float64)
    assert np.allclose(np.exp(got), soft, rtol=2e-5, atol=1e-12)
    # Boolean mask: masked columns are -inf, a fully masked row is NaN
    mask = rng.random((9, 257)) > 0.3
    mask[4, :] = False
    got = orc.softmax(orc.F32, x, mask_kind=orc.MASK_BOOLEAN, mask=mask.astype(np.uint8), log=True)
    assert np.all(np.isnan(got[4]))
    rows = [r for r in range(9) if r != 4]
    assert np.all(np.isneginf(got[rows][~mask[rows]]))
    masked = np.where(mask, x.astype(np.float64), -np.inf)
    with np.errstate(invalid="ignore"):
        want = closed_form(masked[rows])
    keep = mask[rows]
    assert np.all(np.abs(got[rows][keep] - want[keep]) <= 1e-5 * np.abs(want[keep]) + 1e-6)
    # NaN, +inf: the whole row is NaN; the first NaN is the maximum
    x[1, 7] = np.nan
    x[2, 9] = np.inf
    got = orc.softmax(orc.F32, x, log=True)
    assert np.all(np.isnan(got[1])) and np.all(np.isnan(got[2])) and not np.any(np.isnan(got[0]))
    assert np.all(np.isnan(orc.log_softmax_f32_row(np.array([-np.inf, -np.inf], np.float32))))
    assert orc.log_softmax_f32_row(np.array([3.0], np.float32)).tolist() == [0.0]


# ---- the scalar floor's own form (src/simd/math/activations.cc:320-336) ----------------------
import os

import pytest

from oracle import ref

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "scalar_floor_vectors.npz"))
needs_ref = pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (no reference tree)")
TAIL_WIDTHS = (129, 8193)


def same_bits_or_nan(got, want):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def tail_rows(width):
    x = np.full((3, width), -20.0, np.float32)
    x[0, width - 1] = 0
    x[1, 0] = x[1, width - 1] = 0
    x[2, :] = 0
    return x


def test_floor_form_golden_bit_exact():
    for n in (1, 7, 8, 9, 257, 4096):
        same_bits_or_nan(orc.log_softmax_floor_f32_row(GOLD[f"log_softmax_x_{n}"]), GOLD[f"log_softmax_y_{n}"])
    same_bits_or_nan(orc.log_softmax_floor_f32_row(GOLD["log_softmax_x_masked"]),
                     GOLD["log_softmax_y_masked_words"].view(np.float32))
    same_bits_or_nan(orc.log_softmax_floor_f32_row(GOLD["log_softmax_x_wide"]),
                     GOLD["log_softmax_y_wide_words"].view(np.float32))
    for width in TAIL_WIDTHS:
        for row, want in zip(tail_rows(width), GOLD[f"log_softmax_y_tails_{width}"]):
            same_bits_or_nan(orc.log_softmax_floor_f32_row(row), want)


@needs_ref
def test_floor_form_live_bit_exact_and_invalid_rows():
    rng = np.random.default_rng(83)
    for n in (1, 2, 3, 31, 64, 1000, 5000):
        for spread in (0.5, 3.0, 30.0):
            row = rng.normal(0, spread, n).astype(np.float32)
            same_bits_or_nan(orc.log_softmax_floor_f32_row(row), ref.log_softmax_f32(row))
            row[rng.random(n) < 0.3] = -np.inf
            same_bits_or_nan(orc.log_softmax_floor_f32_row(row), ref.log_softmax_f32(row))
    for bad in ([1.0, np.nan, 2.0], [1.0, np.inf], [-np.inf, -np.inf], [np.nan]):
        row = np.array(bad, np.float32)
        got = orc.log_softmax_floor_f32_row(row)
        assert np.all(np.isnan(got)) and np.all(np.isnan(ref.log_softmax_f32(row)))


def test_log1p_form_is_held_to_the_floor_form_at_the_reference_bound():
    """The kernel's form (maximum left out of an f32 sum, log1p) against the floor's form (double
    sum, log): 4e-6 relative + 2e-7, the bound of the reference's own LogSoftmax checks
    (tests/compute_provider_cuda/tensor_test.cc:75-84, 1168-1199); the same rows are invalid."""
    rng = np.random.default_rng(84)
    rows = [GOLD[f"log_softmax_x_{n}"] for n in (1, 7, 8, 9, 257, 4096)]
    rows += [GOLD["log_softmax_x_masked"], GOLD["log_softmax_x_wide"]]
    rows += [r for width in TAIL_WIDTHS for r in tail_rows(width)]
    rows += [rng.normal(0, s, n).astype(np.float32) for n in (5, 300, 4096, 20000) for s in (0.1, 4.0)]
    for row in rows:
        floor = orc.log_softmax_floor_f32_row(row).astype(np.float64)
        form = orc.log_softmax_f32_row(row).astype(np.float64)
        finite = np.isfinite(floor)
        assert np.array_equal(np.isneginf(floor), np.isneginf(form))
        assert np.all(np.abs(form[finite] - floor[finite]) <= np.abs(floor[finite]) * 4e-6 + 2e-7)
    # Rows of large magnitude: the floor rounds max + log(sum) to f32 at the magnitude of the
    # maximum (half a unit of 139 is 8e-6), which the log1p form does not; there the two agree
    # to the same relative bound taken on the largest operand of that subtraction.
    for n in (5, 300, 4096, 20000):
        row = rng.normal(0, 40.0, n).astype(np.float32)
        floor = orc.log_softmax_floor_f32_row(row).astype(np.float64)
        form = orc.log_softmax_f32_row(row).astype(np.float64)
        scale = np.maximum(np.abs(floor), float(np.abs(row).max()))
        assert np.all(np.abs(form - floor) <= scale * 4e-6 + 2e-7)
    for bad in ([1.0, np.nan, 2.0], [1.0, np.inf], [-np.inf, -np.inf], [np.nan]):
        row = np.array(bad, np.float32)
        assert np.all(np.isnan(orc.log_softmax_floor_f32_row(row))) and np.all(np.isnan(orc.log_softmax_f32_row(row)))
