"""GGUF Q4_K / Q6_K rows -> bf16 + row sums of squares (through the C ABI) against the oracle:
bit-exact bf16 values, sums of squares within 1e-5 relative.  The blocks come from the field-wise
builders of tests/k_quant_support.py and from raw random bytes (any byte pattern is a valid block
as long as its f16 scales are finite)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, context, note, run
from k_quant_support import random_rows

pytestmark = pytest.mark.gpu

KINDS = {"q4_k": (orc.Q4_K, hc.GgufQuantizedType.kQ4K, 144), "q6_k": (orc.Q6_K, hc.GgufQuantizedType.kQ6K, 210)}


def dequant_on_device(tag, raw, rows, k, row_stride=None, offset=0):
    _, gguf, _ = KINDS[tag]
    storage = torch.from_numpy(np.ascontiguousarray(raw).reshape(-1)).to(DEVICE)
    desc = hc.TensorDesc.gguf_weight(gguf, hc.DataType.kBFloat16, k, rows, row_stride)
    out, sumsq = run(hc.GgufDequantSumSquares(), storage[offset:], descs=[desc])
    return out.contiguous().view(torch.int16).cpu().numpy().view(np.uint16), sumsq.cpu().numpy()


def sumsq_bar(got, wide):
    """Row sums of squares against the float64 sum of the oracle's exact f32 values: 1e-5 relative.
    (The oracle's own sequential f32 sum is a looser witness: 2048 heavy-tailed terms.)"""
    exact = np.sum(wide.astype(np.float64) ** 2, axis=1)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= 1e-5 * exact)


def finite_scales(tag, raw, block_bytes):
    """Random bytes with the f16 fields forced finite."""
    blocks = raw.reshape(-1, block_bytes)
    for at in ((1, 3) if tag == "q4_k" else (209,)):
        blocks[:, at] &= 0x3B            # exponent below all-ones, small magnitude
    return raw


@pytest.mark.parametrize("tag", ["q4_k", "q6_k"])
def test_k_quant_built_blocks_and_random_bytes(tag):
    kind, _, block_bytes = KINDS[tag]
    rng = np.random.default_rng(1500)
    for rows, k in ((1, 256), (3, 768), (5, 2048), (2, 2304), (4, 4096)):
        raw, values = random_rows(tag, rng, rows, k)
        note(f"{tag} built blocks [{rows}, {k}]")
        got, sumsq = dequant_on_device(tag, raw, rows, k)
        wide, want, want_sumsq = orc.k_quant_dequant(kind, raw, rows, k)
        assert np.array_equal(wide, values)                      # the oracle against the builders
        assert np.array_equal(got, want)
        sumsq_bar(sumsq, wide)
        assert np.allclose(want_sumsq, np.sum(wide.astype(np.float64) ** 2, axis=1), rtol=2e-4)
        note(f"{tag} random bytes [{rows}, {k}]")
        raw = finite_scales(tag, rng.integers(0, 256, (rows, k // 256 * block_bytes), dtype=np.uint8), block_bytes)
        got, sumsq = dequant_on_device(tag, raw, rows, k)
        wide, want, want_sumsq = orc.k_quant_dequant(kind, raw, rows, k)
        assert np.array_equal(got, want)
        sumsq_bar(sumsq, wide)


@pytest.mark.parametrize("tag", ["q4_k", "q6_k"])
def test_k_quant_padded_rows_and_odd_addresses(tag):
    kind, _, block_bytes = KINDS[tag]
    rng = np.random.default_rng(1501)
    rows, k = 6, 1024
    row_bytes = k // 256 * block_bytes
    raw = finite_scales(tag, rng.integers(0, 256, (rows, row_bytes), dtype=np.uint8), block_bytes)
    wide, want, want_sumsq = orc.k_quant_dequant(kind, raw, rows, k)
    for pad, offset in ((2, 0), (7, 0), (0, 1), (5, 3), (16, 2)):
        padded = np.zeros(offset + rows * (row_bytes + pad) + 8, np.uint8)
        for r in range(rows):
            start = offset + r * (row_bytes + pad)
            padded[start:start + row_bytes] = raw[r]
        note(f"{tag} rows {row_bytes + pad} bytes apart, tensor at byte {offset}")
        got, sumsq = dequant_on_device(tag, padded, rows, k, row_stride=row_bytes + pad, offset=offset)
        assert np.array_equal(got, want)
        sumsq_bar(sumsq, wide)


@pytest.mark.parametrize("tag", ["q4_k", "q6_k"])
def test_k_quant_whole_vector_rows(tag):
    """K a multiple of 2048 with base and row stride multiples of 16 takes the wave-per-row kernel
    (several spans per row, padded strides, a row count that leaves waves of the last block idle);
    the same rows 2 bytes off take the general one."""
    kind, _, block_bytes = KINDS[tag]
    rng = np.random.default_rng(1503)
    for rows, k in ((7, 2048), (13, 6144), (257, 4096)):
        row_bytes = k // 256 * block_bytes
        raw = finite_scales(tag, rng.integers(0, 256, (rows, row_bytes), dtype=np.uint8), block_bytes)
        wide, want, _ = orc.k_quant_dequant(kind, raw, rows, k)
        for pad, offset in ((0, 0), (16, 0), (48, 32), (16, 2)):
            padded = np.zeros(offset + rows * (row_bytes + pad) + 8, np.uint8)
            for r in range(rows):
                start = offset + r * (row_bytes + pad)
                padded[start:start + row_bytes] = raw[r]
            note(f"{tag} [{rows}, {k}] rows {row_bytes + pad} bytes apart, tensor at byte {offset}")
            got, sumsq = dequant_on_device(tag, padded, rows, k, row_stride=row_bytes + pad, offset=offset)
            assert np.array_equal(got, want)
            sumsq_bar(sumsq, wide)


def test_k_quant_schema_and_benchmark_shape():
    DT = hc.DataType
    desc = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ4K, DT.kBFloat16, 2048, 6144)
    values, sumsq = hc.infer_output_descriptions(hc.GgufDequantSumSquares(), [desc])
    assert values == hc.TensorDesc.dense(DT.kBFloat16, [6144, 2048]) and sumsq == hc.TensorDesc.dense(DT.kFloat32, [6144])
    assert hc.prepare(context(), hc.GgufDequantSumSquares(), desc).route_name() == "k-quant-dequant-rows"
    with pytest.raises(hc.StatusError):
        hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ6K, DT.kBFloat16, 2000, 8)
    rng = np.random.default_rng(1502)
    for tag in ("q4_k", "q6_k"):
        kind, _, block_bytes = KINDS[tag]
        raw = finite_scales(tag, rng.integers(0, 256, (6144, 8 * block_bytes), dtype=np.uint8), block_bytes)
        note(f"{tag} [6144, 2048]")
        got, sumsq = dequant_on_device(tag, raw, 6144, 2048)
        wide, want, want_sumsq = orc.k_quant_dequant(kind, raw, 6144, 2048)
        assert np.array_equal(got, want)
        sumsq_bar(sumsq, wide)
