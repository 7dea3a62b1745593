"""The oracle's sampling operators.

Philox4x32-10 is pinned by the three known-answer vectors Random123 publishes for philox4x32_10
(kat_vectors: zero, all ones and the digits of pi) and by an array restatement of the independent
form the reference's tests carry (tests/compute_models/sampling_fixture.h:70-91); RandomBits by
that addressing over the fixture's identities, prefixes and row order (…:93-109,189-207).
Categorical is checked as the reference's fixture checks every backend (…:153-283,285-316): the
selected element has mass, the score is within 2e-5 + 2e-5 |s| of the float64 normaliser, a row
with one positive mass selects it, rows permute with their identities, asking for the score does
not change the draw, NaN / +Inf / all -Inf fail -- and, beyond the fixture, as the exact inverse
CDF of the row's 52-bit uniform in float64 and by the fixture's seven-sigma quality gate."""
from __future__ import annotations

import numpy as np
import pytest

from oracle import lib as orc

from sampling_support import fixture_identities, fixture_logits, inverse_cdf_bounds, philox_array, uniform_of

KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0), (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


def test_philox_known_answers():
    for counter, key, want in KAT:
        identity = [key[0], key[1], counter[2], counter[3]]
        assert list(orc.philox_block(identity, counter[0] | (counter[1] << 32))) == list(want)
        assert list(philox_array(np.array([counter], np.uint32), np.array([key], np.uint32))[0]) == list(want)


@pytest.mark.parametrize("rows", [0, 1, 17])
@pytest.mark.parametrize("count", [0, 1, 3, 4, 5, 17, 65])
def test_random_bits_addressing(rows, count):
    ids = fixture_identities(rows, 0xFFFFFFFFFFFFFFFF - 7)   # draw words that carry into the high half
    got = orc.random_bits(ids, count)
    assert got.shape == (rows, count)
    for j in range(count):
        counters = np.stack([np.full(rows, j // 4, np.uint32), np.zeros(rows, np.uint32), ids[:, 2], ids[:, 3]], axis=1)
        assert np.array_equal(got[:, j], philox_array(counters.reshape(rows, 4), ids[:, :2].reshape(rows, 2))[:, j % 4])
    assert np.array_equal(orc.random_bits(ids[::-1], count), got[::-1])          # rows are independent of their order
    if count > 3:
        assert np.array_equal(orc.random_bits(ids, count - 3), got[:, :count - 3])  # and prefixes of the word count


@pytest.mark.parametrize("type_id", [orc.F32, orc.F16, orc.BF16])
def test_categorical_fixture_journey(type_id):
    rows, width = 13, 17
    stored, values = fixture_logits(rows, width, type_id)
    ids = fixture_identities(rows, 0xFEDCBA9876543210)
    status, picked, scores = orc.categorical(type_id, stored, ids, scored=True)
    assert status == 0
    low, high, expected_scores = inverse_cdf_bounds(values, ids)
    for r in range(rows):
        assert np.isfinite(values[r, picked[r]])                     # never a masked element
        assert low[r] <= picked[r] <= high[r]
        assert abs(scores[r] - expected_scores[r, picked[r]]) <= 2e-5 + 2e-5 * abs(expected_scores[r, picked[r]])
    status, plain, none = orc.categorical(type_id, stored, ids)
    assert status == 0 and none is None and np.array_equal(plain, picked)
    status, reordered, _ = orc.categorical(type_id, stored[::-1].copy(), ids[::-1].copy(), scored=True)
    assert status == 0 and np.array_equal(reordered, picked[::-1])


def test_categorical_is_the_inverse_cdf_of_the_rows_uniform():
    rng = np.random.default_rng(5)
    rows, width = 200, 1000
    values = rng.normal(0, 3, (rows, width)).astype(np.float32)
    values[rng.random((rows, width)) < 0.2] = -np.inf
    ids = rng.integers(0, 1 << 32, (rows, 4), dtype=np.uint64).astype(np.uint32)
    status, picked, scores = orc.categorical(orc.F32, values, ids, scored=True)
    assert status == 0
    low, high, expected_scores = inverse_cdf_bounds(values, ids)
    assert ((low <= picked) & (picked <= high)).all()
    assert (low == high).mean() > 0.99                               # the bounds are sharp almost everywhere
    chosen = expected_scores[np.arange(rows), picked]
    assert np.all(np.abs(scores - chosen) <= 2e-5 + 2e-5 * np.abs(chosen))
    for r in range(0, rows, 37):                                     # the uniform is the 52-bit midpoint of words 0, 1
        words = orc.philox_block(ids[r], 0)
        assert orc.categorical_uniform(ids[r]) == uniform_of(words) and 0 < uniform_of(words) < 1


def test_categorical_one_positive_mass_and_large_offsets():
    width = 248320
    for rows in (1, 16):
        for step in (0, 1, 64):
            values = np.full((rows, width), -np.inf, np.float32)
            where = [(step * 7919 + r * 131) % width for r in range(rows)]
            for r, j in enumerate(where):
                values[r, j] = 1e20 if step % 2 else -1e20
            status, picked, scores = orc.categorical(orc.F32, values, fixture_identities(rows, step), scored=True)
            assert status == 0 and list(picked) == where and np.all(scores == 0)


def test_categorical_failures_write_nothing():
    ids = fixture_identities(3, 73)
    valid = np.full((3, 7), 0.25, np.float32)
    status, before, _ = orc.categorical(orc.F32, valid, ids, scored=True)
    assert status == 0
    for invalid in (np.inf, np.nan, -np.inf):
        bad = valid.copy()
        if invalid == -np.inf:
            bad[1, :] = -np.inf
        else:
            bad[1, 2] = invalid
        status, picked, scores = orc.categorical(orc.F32, bad, ids, scored=True)
        assert status == 1 and (picked == -1).all() and np.isnan(scores).all()
        status, after, _ = orc.categorical(orc.F32, valid, ids, scored=True)
        assert status == 0 and np.array_equal(after, before)         # no hidden generator state
    status, picked, _ = orc.categorical(orc.F32, np.zeros((0, 7), np.float32), np.zeros((0, 4), np.uint32))
    assert status == 0 and picked.shape == (0,)


@pytest.mark.parametrize("law", [[0, 0, 0, 0, 0, 0, 0], [-2, -1, 0, 1, 2, -0.5, 0.5],
                                 [-np.inf, -2, -np.inf, 0, 1, -np.inf, 0.5]])
def test_categorical_quality_gate(law):
    # tests/compute_models/sampling_fixture.h:285-316: 64 batches of 4096 rows, every bucket within seven sigma
    rows, batches = 4096, 64
    values = np.tile(np.array(law, np.float32), (rows, 1))
    buckets = np.zeros(7, np.int64)
    for batch in range(batches):
        status, picked, _ = orc.categorical(orc.F32, values, fixture_identities(rows, batch * rows))
        assert status == 0
        buckets += np.bincount(picked, minlength=7)
    count = rows * batches
    p = np.exp(np.array(law, np.float64))
    p /= p.sum()
    for j in range(7):
        if p[j] == 0:
            assert buckets[j] == 0
        else:
            assert count * p[j] >= 20
            assert abs(buckets[j] - count * p[j]) <= 7 * np.sqrt(count * p[j] * (1 - p[j])) + 8
