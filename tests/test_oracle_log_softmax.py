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
