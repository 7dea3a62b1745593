"""Independent forms for the sampling tests: Philox4x32-10 over numpy arrays (the equations of
Random123's philox4x32_10 as the reference's fixture restates them, tests/compute_models/
sampling_fixture.h:70-91), the fixture's identities and logits (…:93-101,214-223) and the float64
inverse CDF of a row's uniform with the band of indices rounding can move the answer within."""
from __future__ import annotations

import numpy as np

from oracle import lib as orc


def philox_array(counters: np.ndarray, keys: np.ndarray) -> np.ndarray:
    """counters [n, 4], keys [n, 2] (uint32) -> [n, 4] words."""
    c = [counters[:, i].astype(np.uint64) for i in range(4)]
    k = [keys[:, i].astype(np.uint64) for i in range(2)]
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = c[0] * np.uint64(0xD2511F53)
        p1 = c[2] * np.uint64(0xCD9E8D57)
        c = [((p1 >> np.uint64(32)) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> np.uint64(32)) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + np.uint64(0x9E3779B9)) & mask, (k[1] + np.uint64(0xBB67AE85)) & mask]
    return np.stack(c, axis=1).astype(np.uint32)


def fixture_identities(rows: int, draw: int) -> np.ndarray:
    r = np.arange(rows, dtype=np.uint64)
    with np.errstate(over="ignore"):
        draws = np.uint64(draw) + r
    out = np.stack([(r * np.uint64(0x9E3779B9)) & np.uint64(0xFFFFFFFF),
                    np.uint64(0xFEDCBA98) ^ ((r * np.uint64(17)) & np.uint64(0xFFFFFFFF)),
                    draws & np.uint64(0xFFFFFFFF), draws >> np.uint64(32)], axis=1)
    return out.astype(np.uint32).reshape(rows, 4)


def fixture_logits(rows: int, width: int, type_id: int):
    """(storage, float32 values after the storage's rounding)."""
    r, j = np.meshgrid(np.arange(rows), np.arange(width), indexing="ij")
    values = (((r * 7 + j) % 11 - 5) * 0.25 + np.where(r % 3 == 0, 1024.0, -1024.0)).astype(np.float32)
    values[j % 5 == 0] = -np.inf
    if type_id == orc.F32:
        return values, values
    stored = orc.from_f32(type_id, values)
    return stored, orc.to_f32(type_id, stored)


def uniform_of(words) -> float:
    return (float(words[0]) * 2.0 ** 20 + float(int(words[1]) >> 12) + 0.5) * 2.0 ** -52


def inverse_cdf_bounds(values: np.ndarray, identities: np.ndarray, slack: float = 4e-6):
    """Per row the lowest and highest index an inverse-CDF draw of the row's uniform may return
    when every mass carries a relative error of up to `slack`, and the float64 log probability of
    every element.  values: float32 [rows, width] (the logical log-weights)."""
    rows, width = values.shape
    v = values.astype(np.float64)
    maximum = v.max(axis=1, keepdims=True)
    mass = np.exp(v - maximum)
    total = mass.sum(axis=1)
    scores = (v - maximum) - np.log(total)[:, None]
    cumulative = np.cumsum(mass, axis=1)
    low, high = np.zeros(rows, np.int64), np.zeros(rows, np.int64)
    for r in range(rows):
        block = philox_array(np.array([[0, 0, identities[r, 2], identities[r, 3]]], np.uint32),
                             np.array([identities[r, :2]], np.uint32))[0]
        threshold = total[r] * uniform_of(block)
        band = slack * total[r]
        positive = np.nonzero(mass[r] > 0)[0]
        first = np.searchsorted(cumulative[r], threshold - band, side="right")
        last = np.searchsorted(cumulative[r], threshold + band, side="right")
        # an index without mass is never returned: move to the neighbours that have some
        low[r] = positive[np.searchsorted(positive, min(first, width - 1), side="left").clip(0, positive.size - 1)]
        high[r] = positive[np.searchsorted(positive, min(last, width - 1), side="left").clip(0, positive.size - 1)]
    return low, high, scores
