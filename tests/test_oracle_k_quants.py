"""The oracle's Q4_K / Q6_K decode against blocks built field by field in the packing direction
(tests/k_quant_support.py), and against the two independent readings of these formats that the
reference tree holds (ggml's own source is not in it)."""
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


# ---- the reference's own independent decoders, restated array-wise over raw random bytes --------
# The reference tree holds two readings of these formats that do not go through ggml's code:
#   third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38  Q4_K as array operations (the ggml
#       dequantize_row_q4_K / get_scale_min_k4 sequence);
#   tests/compute_models/qwen27_original_nextn_reference.h:74-86 (q4_scale, q6_code), 119-127
#       (Q4_K group), 262-287 (expect_embedding: the bit-exact value each decoded element must have).
def random_raw_rows(rng, rows, blocks, size, scale_bytes):
    raw = rng.integers(0, 256, (rows, blocks, size), dtype=np.uint8)
    for at in scale_bytes:                    # keep the f16 fields finite (exponent below 31)
        raw[:, :, at] &= 0x3B
    return raw


def f16_field(raw, at):
    return (raw[..., at].astype(np.uint16) | (raw[..., at + 1].astype(np.uint16) << 8)).view(np.float16).astype(np.float32)


def rn_multiply(a, b):                        # one binary32 rounding of the exact product
    return (np.asarray(a, np.float64) * np.asarray(b, np.float64)).astype(np.float32)


def test_q4_k_against_the_array_form_in_the_reference_tree():
    rng = np.random.default_rng(1401)
    raw = random_raw_rows(rng, 6, 3, 144, (1, 3))
    field = raw.astype(np.uint32)
    scale_lo, min_lo, high = field[..., 4:8], field[..., 8:12], field[..., 12:16]
    scales = np.concatenate([scale_lo & 63, (high & 15) | ((scale_lo >> 6) << 4)], axis=-1)
    mins = np.concatenate([min_lo & 63, (high >> 4) | ((min_lo >> 6) << 4)], axis=-1)
    q = field[..., 16:144].reshape(6, 3, 4, 32)
    codes = np.stack([q & 15, q >> 4], axis=-2).reshape(6, 3, 8, 32)
    d = f16_field(raw, 0)[..., None] * scales.astype(np.float32)
    minimum = f16_field(raw, 2)[..., None] * mins.astype(np.float32)
    want = (d[..., None] * codes.astype(np.float32)).astype(np.float32) - minimum[..., None]
    wide, _, _ = orc.k_quant_dequant(orc.Q4_K, raw.reshape(6, -1), 6, 768)
    assert np.array_equal(wide.view(np.uint32), want.reshape(6, 768).astype(np.float32).view(np.uint32))


def test_q4_k_q6_k_q8_0_against_the_reference_tests_embedding_expectations():
    rng = np.random.default_rng(1402)
    column = np.arange(256)
    # Q6_K: code from its low nibble and two high bits; value = RN(RN(d * scale16) * code)
    raw = random_raw_rows(rng, 5, 2, 210, (209,))
    half, within = column // 128, column % 128
    lane, quarter = within % 32, within // 32
    low = raw[..., half * 64 + lane + (quarter % 2) * 32].astype(np.int32)
    top = raw[..., 128 + half * 32 + lane].astype(np.int32)
    code = (((low >> np.where(quarter >= 2, 4, 0)) & 15) | (((top >> (quarter * 2)) & 3) << 4)) - 32
    scale16 = raw[..., 192 + column // 16].view(np.int8).astype(np.float32)
    want = rn_multiply(rn_multiply(f16_field(raw, 208)[..., None], scale16), code.astype(np.float32))
    wide, _, _ = orc.k_quant_dequant(orc.Q6_K, raw.reshape(5, -1), 5, 512)
    assert np.array_equal(wide.view(np.uint32), want.reshape(5, 512).view(np.uint32))
    # Q4_K: float(d * (q * scale) + dmin * (-minimum)), the sum taken in double
    raw = random_raw_rows(rng, 5, 2, 144, (1, 3))
    group = column // 32
    b = raw.astype(np.int32)
    first = group < 4
    g_hi = np.where(first, 4, group)          # keeps the indices below in range for groups 0..3
    scale = np.where(first, b[..., 4 + np.minimum(group, 3)] & 63,
                     (b[..., 8 + g_hi] & 15) | ((b[..., g_hi] >> 6) << 4))
    minimum = np.where(first, b[..., 8 + np.minimum(group, 3)] & 63,
                       (b[..., 8 + g_hi] >> 4) | ((b[..., 4 + g_hi] >> 6) << 4))
    q = (b[..., 16 + (group // 2) * 32 + column % 32] >> np.where(group % 2 == 1, 4, 0)) & 15
    d, dmin = f16_field(raw, 0).astype(np.float64)[..., None], f16_field(raw, 2).astype(np.float64)[..., None]
    want = (d * (q * scale) + dmin * (-minimum)).astype(np.float32)
    wide, _, _ = orc.k_quant_dequant(orc.Q4_K, raw.reshape(5, -1), 5, 512)
    assert np.array_equal(wide.view(np.uint32), want.reshape(5, 512).view(np.uint32))
    # Q8_0: RN(d * code), exact
    raw = random_raw_rows(rng, 4, 8, 34, (1,))
    want = rn_multiply(f16_field(raw, 0)[..., None], raw[..., 2:].view(np.int8).astype(np.float32))
    got = orc.q8_0_dequant_f32(raw.reshape(4, -1), 4, 256)
    assert np.array_equal(got.view(np.uint32), want.reshape(4, 256).view(np.uint32))
