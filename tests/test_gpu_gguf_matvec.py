"""y = MatMul(x, W) for GGUF weights (Q8_0, Q4_K, Q6_K) and up to 8 activation rows, through the
C ABI, against the oracle's float64 product of exactly decoded weights.

Bar: |got - exact| <= 1e-5 * sum_k |w x| for f32 activations (the f32 sum of K products in the
kernel's order); bf16 / f16 outputs within one unit in the last place of the rounded exact value
unless inside that same bound.  This is the product with exact weights (ActivationArithmetic.kExact);
the product as the reference's ggml route computes it (8-bit activation blocks, integer dots) is
the other arithmetic of the same operator and has its own test, test_gpu_gguf_matvec_q8.py.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, assert_narrow_ulp, context, host_values, note, run, to_device, to_host
from k_quant_support import random_rows

pytestmark = pytest.mark.gpu

KINDS = {"q8_0": (orc.Q8_0, hc.GgufQuantizedType.kQ8_0), "q4_k": (orc.Q4_K, hc.GgufQuantizedType.kQ4K),
         "q6_k": (orc.Q6_K, hc.GgufQuantizedType.kQ6K)}


def weights_for(tag, rng, rows, k):
    if tag != "q8_0":
        return random_rows(tag, rng, rows, k)[0]
    raw = rng.integers(0, 256, (rows, k // 32, 34), dtype=np.uint8)
    raw[:, :, :2] = rng.normal(0, 0.02, (rows, k // 32)).astype(np.float16).view(np.uint8).reshape(rows, k // 32, 2)
    return raw.reshape(rows, -1)


def check(tag, x_tag, raw, rows, k, x, row_stride=None, offset=0):
    kind, gguf = KINDS[tag]
    stored = host_values(x, x_tag)
    wide = stored if x_tag == "f32" else orc.to_f32(TYPES[x_tag][1], stored)
    storage = torch.from_numpy(np.ascontiguousarray(raw).reshape(-1)).to(DEVICE)
    descs = [hc.TensorDesc.gguf_weight(gguf, TYPES[x_tag][0], k, rows, row_stride),
             hc.TensorDesc.dense(TYPES[x_tag][0], list(x.shape))]
    (out,) = run(hc.GgufMatVec(), storage[offset:], to_device(stored, x_tag), descs=descs)
    assert list(out.shape) == ([rows] if x.ndim == 1 else [x.shape[0], rows])
    source = raw.reshape(-1)[offset:]
    exact, magnitude = orc.gguf_matvec(kind, source, rows, k, wide, row_stride)
    exact, magnitude = exact.reshape(out.shape), magnitude.reshape(out.shape)
    got = to_host(out)
    if x_tag == "f32":
        assert np.all(np.abs(got.astype(np.float64) - exact) <= 1e-5 * magnitude + 1e-30)
    else:
        oid = TYPES[x_tag][1]
        as_f32 = orc.to_f32(oid, got).astype(np.float64)
        settled = np.abs(as_f32 - exact) <= 1e-5 * magnitude
        want = orc.from_f32(oid, exact.astype(np.float32))
        assert_narrow_ulp(np.where(settled, want, got), want, x_tag)


@pytest.mark.parametrize("x_tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("tag", list(KINDS))
def test_matvec_shapes_and_batches(tag, x_tag):
    rng = np.random.default_rng(1700)
    for rows, k, m in ((1, 256, 1), (5, 512, 1), (67, 2048, 1), (9, 2304, 3), (130, 1024, 8), (3, 8192, 1), (6, 4096, 2)):
        raw = weights_for(tag, rng, rows, k)
        x = rng.normal(0, 1, (m, k) if m > 1 else (k,)).astype(np.float32)
        note(f"matvec {tag} x {x_tag} rows {rows} k {k} m {m}")
        check(tag, x_tag, raw, rows, k, x)


@pytest.mark.parametrize("tag", list(KINDS))
def test_matvec_padded_rows_and_odd_addresses(tag):
    rng = np.random.default_rng(1701)
    rows, k = 10, 1024
    raw = weights_for(tag, rng, rows, k)
    row_bytes = raw.shape[1]
    x = rng.normal(0, 1, (2, k)).astype(np.float32)
    for pad, offset in ((2, 0), (7, 1), (16, 2)):
        padded = np.zeros(offset + rows * (row_bytes + pad) + 8, np.uint8)
        for r in range(rows):
            start = offset + r * (row_bytes + pad)
            padded[start:start + row_bytes] = raw[r]
        note(f"matvec {tag} rows {row_bytes + pad} bytes apart, tensor at byte {offset}")
        check(tag, "f32", padded, rows, k, x, row_stride=row_bytes + pad, offset=offset)


@pytest.mark.parametrize("x_tag", ["f32", "bf16"])
@pytest.mark.parametrize("tag", ["q4_k", "q6_k", "q8_0"])
def test_matvec_single_token_forms(tag, x_tag):
    """One activation row over 2048 or 4096 values takes the x-in-registers kernel
    (rows read as whole 16-byte vectors and redistributed through LDS) when base and row stride
    are multiples of 16, the general kernel otherwise.  Enough rows that a wave walks several."""
    rng = np.random.default_rng(1703)
    for rows, k in ((21, 4096), (23001, 2048), (5200, 4096)):
        raw = weights_for(tag, rng, rows, k)
        note(f"matvec {tag} single token rows {rows} k {k} x {x_tag}")
        check(tag, x_tag, raw, rows, k, rng.normal(0, 1, k).astype(np.float32))
    rows, k = 300, 2048
    raw = weights_for(tag, rng, rows, k)
    row_bytes = raw.shape[1]
    x = rng.normal(0, 1, k).astype(np.float32)
    for pad, offset in ((16, 0), (32, 16), (2, 0), (6, 2), (16, 4), (3, 0), (0, 1)):
        padded = np.zeros(offset + rows * (row_bytes + pad) + 8, np.uint8)
        for r in range(rows):
            start = offset + r * (row_bytes + pad)
            padded[start:start + row_bytes] = raw[r]
        note(f"matvec {tag} single token rows {row_bytes + pad} bytes apart, tensor at byte {offset}")
        check(tag, x_tag, padded, rows, k, x, row_stride=row_bytes + pad, offset=offset)


@pytest.mark.parametrize("x_tag", ["f32", "bf16"])
@pytest.mark.parametrize("tag", ["q4_k", "q6_k", "q8_0"])
def test_matvec_single_token_long_rows(tag, x_tag):
    """One activation row over two to six whole 2048-value spans: a wave of the block per span, its
    activations in registers, the spans' shares added in LDS.  Row counts below, at and around the
    number of blocks of the grid (twelve waves per compute unit), blocks that take more than the
    four rows they keep in flight; seven spans take the kernel that stages the activations in LDS."""
    rng = np.random.default_rng(1704)
    for rows, k in ((2048, 6144), (3, 8192), (3100, 10240), (37, 12288), (7000, 4096), (1025, 6144), (4100, 8192),
                    (40, 14336)):
        raw = weights_for(tag, rng, rows, k)
        note(f"matvec {tag} long rows {rows} k {k} x {x_tag}")
        check(tag, x_tag, raw, rows, k, rng.normal(0, 1, k).astype(np.float32))


@pytest.mark.parametrize("tag", ["q4_k", "q6_k", "q8_0"])
def test_matvec_single_token_few_rows(tag):
    """Fewer rows than a wave keeps in flight, and row counts around a block's four waves."""
    rng = np.random.default_rng(1705)
    for k in (2048, 4096):
        x = rng.normal(0, 1, k).astype(np.float32)
        for rows in (1, 2, 3, 4, 5, 7, 9):
            raw = weights_for(tag, rng, rows, k)
            note(f"matvec {tag} single token rows {rows} k {k}")
            check(tag, "f32", raw, rows, k, x)


@pytest.mark.parametrize("x_tag", ["f32", "bf16"])
@pytest.mark.parametrize("tag", ["q4_k", "q6_k", "q8_0"])
def test_matvec_few_tokens_whole_spans(tag, x_tag):
    """Two to eight activation rows over rows of 2048 n values: each span is decoded once and
    multiplied against every activation row held in LDS; what does not fit there (eight rows of
    2048) takes the general kernel."""
    rng = np.random.default_rng(1706)
    for rows, k, m in ((300, 2048, 2), (3100, 2048, 4), (77, 2048, 6), (50, 4096, 3), (33, 6144, 2), (20, 2048, 8),
                       (1, 2048, 5)):
        raw = weights_for(tag, rng, rows, k)
        note(f"matvec {tag} x {x_tag} rows {rows} k {k} m {m}")
        check(tag, x_tag, raw, rows, k, rng.normal(0, 1, (m, k)).astype(np.float32))


def test_matvec_schema_admission_and_decode_shape():
    D, DT = hc.TensorDesc.dense, hc.DataType
    w = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ4K, DT.kBFloat16, 2048, 6144)
    assert hc.infer_output_descriptions(hc.GgufMatVec(), [w, D(DT.kBFloat16, [2048])]) == [D(DT.kBFloat16, [6144])]
    assert hc.infer_output_descriptions(hc.GgufMatVec(), [w, D(DT.kFloat32, [4, 2048])]) == [D(DT.kFloat32, [4, 6144])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.GgufMatVec(), [w, D(DT.kFloat32, [4, 1024])])
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.GgufMatVec(), w, D(DT.kFloat32, [9, 2048]))
    assert err.value.is_unimplemented()
    with pytest.raises(hc.StatusError) as err:        # the activations would not fit in LDS
        hc.prepare(context(), hc.GgufMatVec(),
                   hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ8_0, DT.kFloat32, 8192, 16), D(DT.kFloat32, [4, 8192]))
    assert err.value.is_unimplemented()
    assert hc.prepare(context(), hc.GgufMatVec(), w, D(DT.kBFloat16, [2048])).route_name() == "gguf-matvec-rows"
    rng = np.random.default_rng(1702)
    raw = weights_for("q4_k", rng, 512, 2048)
    note("matvec q4_k [512 x 2048] bf16")
    check("q4_k", "bf16", raw, 512, 2048, rng.normal(0, 1, 2048).astype(np.float32))
