"""y = MatMul(x, W) for GGUF weights with the activations quantised to ggml's 8-bit blocks first
(hc.ActivationArithmetic.kGgmlQ8), through the C ABI, against the oracle's restatement of what
the reference's ggml CPU route computes.

Bar: the reference's own.  Its tests accept a native result within
gamma(K / 4 + 65, 2^-24) * sum |terms| (plus the float64 centre's own error) of the exact value
of the integer-dot model (tests/compute_models/qwen27_original_nextn_reference.h:216-257;
tests/compute_models/dspark_original_shared_reference.h:219-262): `bound` below is that figure,
computed by the oracle.  bf16 / f16 outputs add the one rounding of the store.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, context, host_values, note, run, to_device, to_host
from k_quant_support import random_rows

pytestmark = pytest.mark.gpu

KINDS = {"q8_0": (orc.Q8_0, hc.GgufQuantizedType.kQ8_0), "q4_k": (orc.Q4_K, hc.GgufQuantizedType.kQ4K),
         "q6_k": (orc.Q6_K, hc.GgufQuantizedType.kQ6K)}
Q8 = hc.GgufMatVec(hc.ActivationArithmetic.kGgmlQ8)


def weights_for(tag, rng, rows, k):
    if tag != "q8_0":
        return random_rows(tag, rng, rows, k)[0]
    raw = rng.integers(0, 256, (rows, k // 32, 34), dtype=np.uint8)
    raw[:, :, :2] = rng.normal(0, 0.02, (rows, k // 32)).astype(np.float16).view(np.uint8).reshape(rows, k // 32, 2)
    return raw.reshape(rows, -1)


def raw_bytes_for(tag, rng, rows, k):
    """Uniformly random block bytes with finite f16 fields: every scale slot and bit pattern occurs."""
    size, per, fields = {"q8_0": (34, 32, (1,)), "q4_k": (144, 256, (1, 3)), "q6_k": (210, 256, (209,))}[tag]
    raw = rng.integers(0, 256, (rows, k // per, size), dtype=np.uint8)
    for at in fields:
        raw[:, :, at] &= 0x3B
    return raw.reshape(rows, -1)


def check(tag, x_tag, raw, rows, k, x, row_stride=None):
    kind, gguf = KINDS[tag]
    stored = host_values(x, x_tag)
    wide = stored if x_tag == "f32" else orc.to_f32(TYPES[x_tag][1], stored)
    storage = torch.from_numpy(np.ascontiguousarray(raw).reshape(-1)).to(DEVICE)
    descs = [hc.TensorDesc.gguf_weight(gguf, TYPES[x_tag][0], k, rows, row_stride),
             hc.TensorDesc.dense(TYPES[x_tag][0], list(x.shape))]
    (out,) = run(Q8, storage, to_device(stored, x_tag), descs=descs)
    assert list(out.shape) == ([rows] if x.ndim == 1 else [x.shape[0], rows])
    centre, bound = orc.gguf_matvec_q8(kind, raw.reshape(-1), rows, k, wide, row_stride)
    centre, bound = centre.reshape(out.shape), bound.reshape(out.shape)
    got = to_host(out)
    if x_tag != "f32":
        got = orc.to_f32(TYPES[x_tag][1], got)
        bound = bound + np.abs(centre) * 2.0 ** (-8 if x_tag == "bf16" else -11) + 1e-30
    error = np.abs(got.astype(np.float64) - centre)
    assert np.all(np.isfinite(got))
    worst = np.max(error / np.maximum(bound, 1e-300))
    assert worst <= 1.0, f"{tag} x {x_tag}: error is {worst:.3f} of the accepted bound"
    return worst


@pytest.mark.parametrize("x_tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("tag", list(KINDS))
def test_q8_route_shapes_and_batches(tag, x_tag):
    rng = np.random.default_rng(1800)
    for rows, k, m in ((1, 2048, 1), (67, 2048, 1), (130, 2048, 2), (9, 2048, 3), (33, 2048, 4), (21, 2048, 5),
                       (40, 2048, 8), (6, 4096, 1), (19, 4096, 2), (13, 4096, 4), (9000, 2048, 3), (5, 6144, 1),
                       (3, 12288, 1), (7, 8192, 1),
                       # one row, a wave per span: blocks with one row, with more than the four in flight, five and
                       # seven spans (the last parks its codes in LDS)
                       (9000, 2048, 1), (5000, 4096, 1), (1030, 6144, 1), (600, 10240, 1), (5, 14336, 1)):
        raw = weights_for(tag, rng, rows, k)
        x = rng.normal(0, 1.5, (m, k) if m > 1 else (k,)).astype(np.float32)
        note(f"q8 matvec {tag} x {x_tag} rows {rows} k {k} m {m}")
        check(tag, x_tag, raw, rows, k, x)


@pytest.mark.parametrize("tag", list(KINDS))
def test_q8_route_raw_bytes_zero_blocks_ties_and_padded_rows(tag):
    rng = np.random.default_rng(1801)
    rows, k = 50, 2048
    raw = raw_bytes_for(tag, rng, rows, k)
    x = rng.normal(0, 2, (4, k)).astype(np.float32)
    x[0, 256:512] = 0.0                        # an activation block of zeros
    x[1, :] = 0.0                              # a whole row of zeros
    x[2, 512:768] = np.where(np.arange(256) % 2 == 0, 1.25, -1.25)   # every magnitude equal: the first sign decides
    x[3, 1024:1056] = -3.0                     # a Q8_0 block whose every value is the (negative) maximum
    note(f"q8 matvec {tag}: raw bytes, zero blocks, equal magnitudes")
    check(tag, "f32", raw, rows, k, x)
    row_bytes = raw.shape[1]
    padded = np.zeros((rows, row_bytes + 48), np.uint8)
    padded[:, :row_bytes] = raw
    note(f"q8 matvec {tag}: rows 48 bytes further apart than their blocks")
    check(tag, "f32", padded, rows, k, x, row_stride=row_bytes + 48)


@pytest.mark.parametrize("tag,m", [("q6_k", 4), ("q4_k", 1), ("q4_k", 3), ("q4_k", 8), ("q8_0", 2)])
def test_q8_route_vocabulary_sized_weight(tag, m):
    rng = np.random.default_rng(1802)
    rows, k = 151936, 2048
    size, per = {"q8_0": (34, 32), "q4_k": (144, 256), "q6_k": (210, 256)}[tag]
    raw = raw_bytes_for(tag, rng, 4096, k)
    raw = np.tile(raw, (rows // 4096 + 1, 1))[:rows]          # 151936 rows out of 4096 distinct ones
    raw = raw.copy()
    raw[:, 5 * size:6 * size] = raw_bytes_for(tag, rng, rows, per).reshape(rows, size)   # and one block of its own each
    x = rng.normal(0, 1, (m, k) if m > 1 else (k,)).astype(np.float32)
    note(f"q8 matvec {tag} [2048 -> 151936] x {m}")
    check(tag, "f32", raw, rows, k, x)


def test_q8_route_declines_what_it_does_not_serve():
    ctx = context()
    weight = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ6K, hc.DataType.kFloat32, 1024, 16)
    with pytest.raises(hc.StatusError) as declined:
        hc.prepare(ctx, Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [1024]))
    assert declined.value.is_unimplemented()
    weight = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ6K, hc.DataType.kFloat32, 8192, 16)
    with pytest.raises(hc.StatusError) as declined:
        hc.prepare(ctx, Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [8, 8192]))
    assert declined.value.is_unimplemented()
