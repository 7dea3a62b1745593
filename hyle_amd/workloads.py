"""Seeded synthetic inputs of the five benchmark configurations (numpy, PCG64).

The same bytes feed the GPU run, the parity tests and the CPU baseline.  Narrow floats are
produced as uint16 bit patterns with a vectorised RN-even rounding (finite inputs only).
Every generator takes the leading extent as a parameter so tests can ask for a slice of the
full shape.
"""
from __future__ import annotations

import numpy as np


def to_bf16_bits(values: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round to nearest even (finite values)."""
    u = np.ascontiguousarray(values, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def config1(rows: int = 4096, cols: int = 2048, seed: int = 0):
    """A[rows, cols] f32 ~ N(0,1); b[cols] f32 ~ U(-1,1); s = 0.5: C = (A + b) * s."""
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((rows, cols), dtype=np.float32)
    b = rng.uniform(-1.0, 1.0, cols).astype(np.float32)
    s = np.array([0.5], np.float32)
    return a, b, s


def config2(rows: int = 8192, hidden: int = 2048, seed: int = 1):
    """X[rows, hidden] bf16 = N(0,1) scaled per row by U(0.1, 10); w[hidden] bf16 ~ N(1, 0.1)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, hidden), dtype=np.float32)
    x *= rng.uniform(0.1, 10.0, (rows, 1)).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(hidden, dtype=np.float32)).astype(np.float32)
    return to_bf16_bits(x), to_bf16_bits(w)


def config3_swiglu(rows: int = 8192, hidden: int = 6144, seed: int = 2):
    """gate, up [rows, hidden] bf16 ~ N(0, 2)."""
    rng = np.random.default_rng(seed)
    gate = 2.0 * rng.standard_normal((rows, hidden), dtype=np.float32)
    up = 2.0 * rng.standard_normal((rows, hidden), dtype=np.float32)
    return to_bf16_bits(gate), to_bf16_bits(up)


def config3_residual(rows: int = 8192, hidden: int = 2048, seed: int = 2):
    """R, Y [rows, hidden] bf16 ~ N(0, 1): R += Y."""
    rng = np.random.default_rng(seed + 1000)
    r = rng.standard_normal((rows, hidden), dtype=np.float32)
    y = rng.standard_normal((rows, hidden), dtype=np.float32)
    return to_bf16_bits(r), to_bf16_bits(y)


def config4_softmax(heads: int = 32, seq: int = 4096, seed: int = 3):
    """S[heads, seq, seq] f32 ~ N(0, 3); causal Bool mask [seq, seq] (1 = keep)."""
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((heads, seq, seq), dtype=np.float32)
    s *= np.float32(3.0)
    mask = np.tril(np.ones((seq, seq), np.uint8))
    return s, mask


def config4_argmax(rows: int = 64, vocab: int = 151936, seed: int = 3):
    """logits[rows, vocab] f32 ~ N(0, 4) with a few planted exact ties of the row maximum."""
    rng = np.random.default_rng(seed + 1000)
    logits = rng.standard_normal((rows, vocab), dtype=np.float32)
    logits *= np.float32(4.0)
    for r in range(0, rows, 3):  # the maximum appears again later in the row, bit for bit
        top = int(np.argmax(logits[r]))
        later = int(rng.integers(top, vocab))
        logits[r, later] = logits[r, top]
        if r % 2 == 0 and top > 0:  # and once before it: the earlier index must win
            logits[r, int(rng.integers(0, top))] = logits[r, top]
    return logits


def config5(rows: int = 6144, k: int = 2048, seed: int = 4):
    """Q8_0 weight: rows x k/32 blocks {fp16 d ~ U(1e-3, 2e-2); int8 q ~ U[-127, 127]}.
    Returns the raw block bytes as uint8 [rows, k/32*34]."""
    rng = np.random.default_rng(seed)
    nb = k // 32
    d = rng.uniform(1e-3, 2e-2, (rows, nb)).astype(np.float16)
    q = rng.integers(-127, 128, (rows, nb, 32), dtype=np.int8)
    blocks = np.empty((rows, nb, 34), np.uint8)
    blocks[:, :, :2] = d.view(np.uint8).reshape(rows, nb, 2)
    blocks[:, :, 2:] = q.view(np.uint8)
    return blocks.reshape(rows, nb * 34)


# algorithmic bytes of the full shapes: the bytes an ideal implementation must move
ALGORITHMIC_BYTES = {
    "cfg1_broadcast_add_mul_f32": 4096 * 2048 * 4 * 2 + 2048 * 4,
    "cfg2_rmsnorm_bf16": 8192 * 2048 * 2 * 2 + 2048 * 2,
    "cfg3_swiglu_bf16": 3 * 8192 * 6144 * 2,
    "cfg3_residual_add_bf16": 3 * 8192 * 2048 * 2,
    "cfg4_softmax_f32_causal": 2 * 32 * 4096 * 4096 * 4 + 4096 * 4096,
    "cfg4_argmax_f32": 64 * 151936 * 4 + 64 * 4 + 64 * 4,
    "cfg5_q8_0_dequant_sumsq": 6144 * 64 * 34 + 6144 * 2048 * 2 + 6144 * 4,
}
