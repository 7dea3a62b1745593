"""Parity of RandomBits and Categorical (through the C ABI) with the CPU oracle.

RandomBits is bit-exact.  Categorical is held to what the reference holds every backend to
(tests/compute_models/sampling_fixture.h:153-316): the selected element has mass, the score is
within 2e-5 + 2e-5 |s| of the float64 normaliser, one positive mass is selected wherever it sits,
rows permute with their identities, asking for the score does not change the draw, invalid rows
fail the completion with InvalidArgument and leave no hidden state, the fixed-seed distribution
passes the seven-sigma gate -- and, because this route follows the CPU provider's inverse CDF, to
the oracle's index itself wherever the float64 CDF leaves no room for rounding."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import capi
from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, context, note
from sampling_support import fixture_identities, fixture_logits, inverse_cdf_bounds

pytestmark = pytest.mark.gpu

DT = hc.DataType
KINDS = {orc.F32: DT.kFloat32, orc.F16: DT.kFloat16, orc.BF16: DT.kBFloat16}


def on_device(raw: np.ndarray) -> torch.Tensor:
    flat = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    return torch.from_numpy(flat.copy()).to(DEVICE) if flat.size else torch.empty(16, dtype=torch.uint8, device=DEVICE)


def random_bits_on_device(ids: np.ndarray, count: int, lead: int = 0) -> np.ndarray:
    """`lead`: bytes the identities sit past a 256-byte boundary (the reference asks element alignment only)."""
    rows = ids.shape[0]
    prepared = hc.prepare(context(), hc.RandomBits(count), hc.TensorDesc.dense(DT.kUInt32, [rows, 4]))
    assert prepared.output_description() == hc.TensorDesc.dense(DT.kUInt32, [rows, count])
    assert prepared.workspace_requirement().size == 0
    assert prepared.dispatch_count() == (1 if rows * count else 0)
    source = on_device(np.concatenate([np.zeros(lead, np.uint8), np.ascontiguousarray(ids).view(np.uint8).reshape(-1)]))
    out = torch.full((rows * count * 4 + 16,), 0x5A, dtype=torch.uint8, device=DEVICE)
    prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream, [source.data_ptr() + lead], [out.data_ptr()])
    torch.cuda.synchronize()
    host = out.cpu().numpy()
    assert (host[rows * count * 4:] == 0x5A).all()
    return host[:rows * count * 4].copy().view(np.uint32).reshape(rows, count)


def test_random_bits_match_philox_word_for_word():
    for rows in (0, 1, 17):
        for count in (0, 1, 3, 4, 5, 17, 65):
            note(f"random bits rows={rows} count={count}")
            ids = fixture_identities(rows, 0xFFFFFFFFFFFFFFFF - 7)
            assert np.array_equal(random_bits_on_device(ids, count), orc.random_bits(ids, count))
            assert np.array_equal(random_bits_on_device(ids[::-1].copy(), count), orc.random_bits(ids, count)[::-1])
    note("random bits 4096 x 1024 and 333 x 1001")
    ids = np.random.default_rng(9).integers(0, 1 << 32, (4096, 4), dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(random_bits_on_device(ids, 1024), orc.random_bits(ids, 1024))
    assert np.array_equal(random_bits_on_device(ids[:333], 1001), orc.random_bits(ids[:333], 1001))
    assert np.array_equal(random_bits_on_device(ids[:333], 64, lead=4), orc.random_bits(ids[:333], 64))
    note("random bits, long rows (a block per row piece): 3 x 4100, 2 x 16388, 5 x 1024 past an odd lead, 66000 x 1024")
    assert np.array_equal(random_bits_on_device(ids[:3], 4100), orc.random_bits(ids[:3], 4100))
    assert np.array_equal(random_bits_on_device(ids[:2], 16388), orc.random_bits(ids[:2], 16388))
    assert np.array_equal(random_bits_on_device(ids[:5], 1024, lead=12), orc.random_bits(ids[:5], 1024))
    many = np.random.default_rng(10).integers(0, 1 << 32, (66000, 4), dtype=np.uint64).astype(np.uint32)   # more rows than grid.y holds
    assert np.array_equal(random_bits_on_device(many, 1024), orc.random_bits(many, 1024))


def categorical_on_device(type_id, stored: np.ndarray, ids: np.ndarray, scored: bool, static: bool = False):
    """(status code or 0, indices, scores or None)."""
    rows, width = stored.shape
    kind = KINDS[type_id]
    prepared = hc.prepare(context(), hc.Categorical(scored), hc.TensorDesc.dense(kind, [rows, width]),
                          hc.TensorDesc.dense(DT.kUInt32, [rows, 4]))
    outs = prepared.output_descriptions()
    assert outs[0] == hc.TensorDesc.dense(DT.kInt32, [rows]) and len(outs) == (2 if scored else 1)
    assert prepared.dispatch_count() == (2 if rows else 0)
    logits, keys = on_device(stored), on_device(ids)
    picked = torch.full((max(rows, 1),), -7, dtype=torch.int32, device=DEVICE)
    scores = torch.full((max(rows, 1),), float("nan"), dtype=torch.float32, device=DEVICE)
    need = prepared.workspace_requirement()
    workspace = torch.full((max(need.size, 1),), 0xFF, dtype=torch.uint8, device=DEVICE)   # stale contents must not matter
    stream = torch.cuda.current_stream().cuda_stream
    outputs = [picked.data_ptr(), scores.data_ptr()] if scored else [picked.data_ptr()]
    status = 0
    try:
        if static:
            invocation = prepared.create_invocation_without_workspace()
            invocation.submit_without_workspace(stream, [logits.data_ptr(), keys.data_ptr()], outputs)
        else:
            invocation = prepared.create_invocation(workspace.data_ptr(), need.size)
            invocation.submit(stream, [logits.data_ptr(), keys.data_ptr()], outputs)
        invocation.wait(stream, static_scratch=static)
    except hc.StatusError as error:
        status = int(error.code)
    torch.cuda.synchronize()
    return status, picked.cpu().numpy()[:rows], (scores.cpu().numpy()[:rows] if scored else None)


def check_against_float64(values, ids, picked, scores, oracle_picked):
    low, high, expected = inverse_cdf_bounds(values, ids, slack=1e-6)   # masses are good to about 2e-7
    rows = values.shape[0]
    assert ((0 <= picked) & (picked < values.shape[1])).all()
    assert np.isfinite(values[np.arange(rows), picked]).all()              # never a masked element
    assert ((low <= picked) & (picked <= high)).all()
    sharp = low == high
    assert np.array_equal(picked[sharp], oracle_picked[sharp])             # the oracle's index wherever rounding has no room
    if scores is not None:
        chosen = expected[np.arange(rows), picked]
        assert np.all(np.abs(scores - chosen) <= 2e-5 + 2e-5 * np.abs(chosen))
    return sharp.mean()


@pytest.mark.parametrize("type_id", [orc.F32, orc.F16, orc.BF16])
def test_categorical_fixture_journey(type_id):
    rows, width = 13, 17
    stored, values = fixture_logits(rows, width, type_id)
    ids = fixture_identities(rows, 0xFEDCBA9876543210)
    note(f"categorical journey type {type_id}")
    status, picked, scores = categorical_on_device(type_id, stored, ids, True)
    assert status == 0
    _, oracle_picked, _ = orc.categorical(type_id, stored, ids)
    check_against_float64(values, ids, picked, scores, oracle_picked)
    status, plain, _ = categorical_on_device(type_id, stored, ids, False)
    assert status == 0 and np.array_equal(plain, picked)                    # asking for the score does not change the draw
    status, reordered, _ = categorical_on_device(type_id, stored[::-1].copy(), ids[::-1].copy(), True)
    assert status == 0 and np.array_equal(reordered, picked[::-1])          # rows travel with their identities


@pytest.mark.parametrize("type_id,rows,width", [(orc.F32, 64, 151936), (orc.BF16, 32, 151936), (orc.F16, 300, 4096),
                                                (orc.F32, 500, 4099), (orc.BF16, 2000, 130), (orc.F32, 3, 1 << 20)])
def test_categorical_is_the_oracles_inverse_cdf(type_id, rows, width):
    note(f"categorical inverse cdf type {type_id} rows {rows} width {width}")
    rng = np.random.default_rng(rows + width)
    values = rng.normal(0, 3, (rows, width)).astype(np.float32)
    values[rng.random((rows, width)) < 0.1] = -np.inf
    stored = values if type_id == orc.F32 else orc.from_f32(type_id, values)
    values = values if type_id == orc.F32 else orc.to_f32(type_id, stored)
    ids = rng.integers(0, 1 << 32, (rows, 4), dtype=np.uint64).astype(np.uint32)
    status, picked, scores = categorical_on_device(type_id, stored, ids, True)
    assert status == 0
    oracle_status, oracle_picked, _ = orc.categorical(type_id, stored, ids)
    assert oracle_status == 0
    assert check_against_float64(values, ids, picked, scores, oracle_picked) > 0.9   # rows pinned to the oracle's index


def test_categorical_one_positive_mass_in_a_full_vocabulary():
    width = 248320
    for rows in (1, 16):
        for step in (0, 1, 2, 63, 64):
            note(f"categorical one mass rows {rows} step {step}")
            values = np.full((rows, width), -np.inf, np.float32)
            where = [(step * 7919 + r * 131) % width for r in range(rows)]
            for r, j in enumerate(where):
                values[r, j] = 1e20 if step % 2 else -1e20
            status, picked, scores = categorical_on_device(orc.F32, values, fixture_identities(rows, step), True)
            assert status == 0 and list(picked) == where and np.all(scores == 0)


@pytest.mark.parametrize("static", [False, True])
def test_categorical_failures_fail_the_completion_and_keep_no_state(static):
    ids = fixture_identities(3, 73)
    valid = np.full((3, 7), 0.25, np.float32)
    status, before, before_scores = categorical_on_device(orc.F32, valid, ids, True, static)
    assert status == 0
    for invalid in (np.inf, np.nan, -np.inf):
        note(f"categorical failure {invalid} static {static}")
        bad = valid.copy()
        if invalid == -np.inf:
            bad[1, :] = -np.inf
        else:
            bad[1, 2] = invalid
        status, picked, _ = categorical_on_device(orc.F32, bad, ids, True, static)
        assert status == capi.INVALID_ARGUMENT and picked[1] == -7          # the invalid row wrote nothing
        assert orc.categorical(orc.F32, bad, ids)[0] == 1
        status, after, after_scores = categorical_on_device(orc.F32, valid, ids, True, static)
        assert status == 0 and np.array_equal(after, before) and np.array_equal(after_scores, before_scores)
    note("categorical failure deep inside a wide row")
    wide = np.random.default_rng(4).normal(0, 1, (5, 20000)).astype(np.float32)
    wide[3, 17777] = np.nan
    assert categorical_on_device(orc.F32, wide, fixture_identities(5, 1), False, static)[0] == capi.INVALID_ARGUMENT
    status, picked, _ = categorical_on_device(orc.F32, np.zeros((0, 7), np.float32), np.zeros((0, 4), np.uint32), True, static)
    assert status == 0 and picked.shape == (0,)


@pytest.mark.parametrize("law", [[0, 0, 0, 0, 0, 0, 0], [-2, -1, 0, 1, 2, -0.5, 0.5],
                                 [-np.inf, -2, -np.inf, 0, 1, -np.inf, 0.5]])
def test_categorical_quality_gate(law):
    # tests/compute_models/sampling_fixture.h:285-316
    rows, batches = 4096, 64
    values = np.tile(np.array(law, np.float32), (rows, 1))
    buckets = np.zeros(7, np.int64)
    note(f"categorical quality law {law}")
    for batch in range(batches):
        ids = fixture_identities(rows, batch * rows)
        status, picked, _ = categorical_on_device(orc.F32, values, ids, False)
        assert status == 0
        assert np.array_equal(picked, orc.categorical(orc.F32, values, ids)[1])   # seven well separated masses: no room for rounding
        buckets += np.bincount(picked, minlength=7)
    count = rows * batches
    p = np.exp(np.array(law, np.float64))
    p /= p.sum()
    for j in range(7):
        if p[j] == 0:
            assert buckets[j] == 0
        else:
            assert abs(buckets[j] - count * p[j]) <= 7 * np.sqrt(count * p[j] * (1 - p[j])) + 8
