"""The oracle's Q4_K / Q6_K decode against blocks built field by field in the packing direction
(tests/k_quant_support.py).  ggml itself is not in the reference tree: these tests pin the index
conventions and the arithmetic order of the restatement, not ggml's source."""
from __future__ import annotations

import numpy as np

from oracle import lib as orc

from k_quant_support import pack_q4_k, pack_q6_k, random_rows, values_q4_k, values_q6_k


def test_q4_k_every_scale_slot_and_nibble_position():
    for sub in range(8):                       # one sub-block at a time: its scale, its minimum, its nibbles
        scales, minima = np.zeros(8, int), np.zeros(8, int)
        scales[sub], minima[sub] = 37 + sub, 5 + 7 * sub
        quants = np.zeros((8, 32), int)
        quants[sub] = np.arange(32) % 16
        block = pack_q4_k(0.5, 0.25, scales, minima, quants)
        wide, narrow, sumsq = orc.k_quant_dequant(orc.Q4_K, block[None, :], 1, 256)
        want = np.zeros(256, np.float32)
        want[32 * sub:32 * sub + 32] = 0.5 * scales[sub] * (np.arange(32) % 16) - 0.25 * minima[sub]
        assert np.array_equal(wide[0], want)
        assert np.array_equal(narrow[0], orc.from_f32(orc.BF16, want))
        assert np.isclose(sumsq[0], np.sum(want.astype(np.float64) ** 2), rtol=1e-6)
    # six-bit extremes in every slot at once
    scales, minima = np.full(8, 63), np.arange(8) * 9
    quants = np.full((8, 32), 15)
    wide, _, _ = orc.k_quant_dequant(orc.Q4_K, pack_q4_k(1.0, 1.0, scales, minima, quants)[None, :], 1, 256)
    assert np.array_equal(wide[0].reshape(8, 32)[:, 0], 63.0 * 15 - minima)


def test_q6_k_every_scale_slot_and_bit_position():
    for sub in range(16):
        scales = np.zeros(16, int)
        scales[sub] = -100 + 13 * sub
        quants = np.full(256, 32)              # value 0 everywhere ...
        quants[16 * sub:16 * sub + 16] = [0, 1, 2, 3, 15, 16, 17, 31, 32, 33, 47, 48, 49, 62, 63, 21]
        block = pack_q6_k(0.25, scales, quants)
        wide, narrow, _ = orc.k_quant_dequant(orc.Q6_K, block[None, :], 1, 256)
        want = np.zeros(256, np.float32)
        want[16 * sub:16 * sub + 16] = 0.25 * scales[sub] * (quants[16 * sub:16 * sub + 16] - 32)
        assert np.array_equal(wide[0], want)
        assert np.array_equal(narrow[0], orc.from_f32(orc.BF16, want))


def test_random_blocks_rows_and_strides():
    rng = np.random.default_rng(1400)
    for kind, tag in ((orc.Q4_K, "q4_k"), (orc.Q6_K, "q6_k")):
        raw, want = random_rows(tag, rng, 5, 768)
        wide, narrow, sumsq = orc.k_quant_dequant(kind, raw, 5, 768)
        assert np.array_equal(wide, want)
        assert np.array_equal(narrow, orc.from_f32(orc.BF16, want))
        assert np.allclose(sumsq, np.sum(want.astype(np.float64) ** 2, axis=1), rtol=1e-5)
        padded = np.zeros((5, raw.shape[1] + 6), np.uint8)       # rows further apart than their blocks
        padded[:, :raw.shape[1]] = raw
        again, _, _ = orc.k_quant_dequant(kind, padded, 5, 768, row_stride=padded.shape[1])
        assert np.array_equal(again, want)
