"""Builders of GGUF Q4_K / Q6_K blocks from their logical fields (the published block layouts,
written in the packing direction) and the values those fields stand for, for the tests."""
from __future__ import annotations

import numpy as np


def pack_q4_k(d: np.float16, dmin: np.float16, scales, minima, quants) -> np.ndarray:
    """scales, minima: 8 six-bit integers; quants: [8, 32] four-bit integers -> 144 bytes."""
    scales, minima = np.asarray(scales, np.uint8), np.asarray(minima, np.uint8)
    quants = np.asarray(quants, np.uint8).reshape(8, 32)
    block = np.zeros(144, np.uint8)
    block[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    block[2:4] = np.frombuffer(np.float16(dmin).tobytes(), np.uint8)
    packed = np.zeros(12, np.uint8)
    for j in range(4):                      # sub-blocks 0..3: low six bits of bytes j and j + 4
        packed[j] = scales[j] & 63
        packed[j + 4] = minima[j] & 63
    for j in range(4, 8):                   # sub-blocks 4..7: nibbles of byte j + 4, top bits above the first eight
        packed[j + 4] = (scales[j] & 0xF) | ((minima[j] & 0xF) << 4)
        packed[j - 4] |= (scales[j] >> 4) << 6
        packed[j] |= (minima[j] >> 4) << 6
    block[4:16] = packed
    for chunk in range(4):                  # 32 bytes hold sub-block 2c (low nibbles) and 2c + 1 (high nibbles)
        block[16 + 32 * chunk:16 + 32 * chunk + 32] = quants[2 * chunk] | (quants[2 * chunk + 1] << 4)
    return block


def values_q4_k(d, dmin, scales, minima, quants) -> np.ndarray:
    d, dmin = np.float32(np.float16(d)), np.float32(np.float16(dmin))
    out = np.empty((8, 32), np.float32)
    for j in range(8):
        step = np.float32(d * np.float32(scales[j]))
        offset = np.float32(dmin * np.float32(minima[j]))
        out[j] = (step * np.asarray(quants, np.float32).reshape(8, 32)[j]).astype(np.float32) - offset
    return out.reshape(256)


def pack_q6_k(d: np.float16, scales, quants) -> np.ndarray:
    """scales: 16 int8; quants: 256 six-bit integers (value = quant - 32) -> 210 bytes."""
    quants = np.asarray(quants, np.uint8).reshape(2, 4, 32)        # half, group of 32, position
    block = np.zeros(210, np.uint8)
    for half in range(2):
        low = quants[half] & 0xF
        high = quants[half] >> 4
        ql = np.zeros(64, np.uint8)
        ql[0:32] = low[0] | (low[2] << 4)
        ql[32:64] = low[1] | (low[3] << 4)
        qh = high[0] | (high[1] << 2) | (high[2] << 4) | (high[3] << 6)
        block[64 * half:64 * half + 64] = ql
        block[128 + 32 * half:128 + 32 * half + 32] = qh
    block[192:208] = np.asarray(scales, np.int8).view(np.uint8)
    block[208:210] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    return block


def values_q6_k(d, scales, quants) -> np.ndarray:
    d = np.float32(np.float16(d))
    scales = np.asarray(scales, np.int8)
    signed = np.asarray(quants, np.int32).reshape(16, 16) - 32      # sixteen sub-blocks of 16
    out = np.empty((16, 16), np.float32)
    for sub in range(16):
        step = np.float32(d * np.float32(scales[sub]))
        out[sub] = (step * signed[sub].astype(np.float32)).astype(np.float32)
    return out.reshape(256)


def random_rows(kind: str, rng, rows: int, k: int):
    """-> (bytes [rows, row_bytes], f32 values [rows, k]) of random blocks with finite scales."""
    blocks_per_row = k // 256
    size = 144 if kind == "q4_k" else 210
    raw = np.zeros((rows, blocks_per_row * size), np.uint8)
    values = np.zeros((rows, k), np.float32)
    for r in range(rows):
        for b in range(blocks_per_row):
            d = np.float16(rng.normal(0, 0.02))
            if kind == "q4_k":
                dmin = np.float16(rng.normal(0, 0.02))
                scales, minima = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
                quants = rng.integers(0, 16, (8, 32))
                raw[r, b * size:(b + 1) * size] = pack_q4_k(d, dmin, scales, minima, quants)
                values[r, b * 256:(b + 1) * 256] = values_q4_k(d, dmin, scales, minima, quants)
            else:
                scales = rng.integers(-128, 128, 16)
                quants = rng.integers(0, 64, 256)
                raw[r, b * size:(b + 1) * size] = pack_q6_k(d, scales, quants)
                values[r, b * 256:(b + 1) * 256] = values_q6_k(d, scales, quants)
    return raw, values
