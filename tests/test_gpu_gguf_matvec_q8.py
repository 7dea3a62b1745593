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


def check(tag, x_tag, raw, rows, k, x, row_stride=None, byte_offset=0, kernel=None, x_offset=0):
    """byte_offset: the weight starts that many bytes into its (256-byte aligned) allocation;
    x_offset: the activations start that many elements into theirs;
    kernel: the launch shape the case is written for (a prefix of the label)."""
    kind, gguf = KINDS[tag]
    stored = host_values(x, x_tag)
    wide = stored if x_tag == "f32" else orc.to_f32(TYPES[x_tag][1], stored)
    flat = np.ascontiguousarray(raw).reshape(-1)
    if byte_offset:
        flat = np.concatenate([np.zeros(byte_offset, np.uint8), flat])
    storage = torch.from_numpy(flat).to(DEVICE)[byte_offset:]
    descs = [hc.TensorDesc.gguf_weight(gguf, TYPES[x_tag][0], k, rows, row_stride),
             hc.TensorDesc.dense(TYPES[x_tag][0], list(x.shape))]
    activations = to_device(stored, x_tag)
    if x_offset:
        padded = torch.zeros(activations.numel() + x_offset, dtype=activations.dtype, device=DEVICE)
        padded[x_offset:] = activations.reshape(-1)
        activations = padded[x_offset:].view(activations.shape)
    (out,) = run(Q8, storage, activations, descs=descs)
    if kernel is not None:
        assert hc.last_launch_variant().startswith(kernel), (hc.last_launch_variant(), kernel)
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
                       (9000, 2048, 1), (5000, 4096, 1), (1030, 6144, 1), (600, 10240, 1), (5, 14336, 1),
                       # several tokens whose codes leave no room for the quad kernel's row slots: the kernel that
                       # fetches the codes from LDS span by span, for two, four and eight tokens
                       (11, 18432, 2), (7, 20480, 2), (9, 12288, 3), (10, 8192, 5), (6, 6144, 7)):
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


def test_q8_route_the_reference_s_own_projection_shapes():
    """The shapes of the reference's Q8_0 / Q4_K projection cases
    (tests/compute_models/cpu_c5_gguf_inputs.h:231,237,259,287,314): none is a multiple of 2048 wide.
    The Q8_0 ones of 256 n values take the span kernel with a short last span (128 values: the kernel
    that walks a row block by block), the Q4_K one the matrix-unit kernel."""
    rng = np.random.default_rng(1803)
    for tag, k, rows in (("q8_0", 1024, 32768), ("q4_k", 5120, 10240), ("q8_0", 7168, 3072), ("q8_0", 17408, 5120),
                         ("q8_0", 128, 512)):
        raw = weights_for(tag, rng, rows, k)
        x = rng.normal(0, 1.5, (k,)).astype(np.float32)
        note(f"q8 matvec {tag} [{k} -> {rows}], one activation row")
        kernel = {1024: "gguf_matvec_q8_spans/q8_0/1-spans/short", 5120: "gguf_matvec_q8_tiles/q4_k/1-tokens",
                  7168: "gguf_matvec_q8_spans/q8_0/4-spans/short", 17408: "gguf_matvec_q8_spans/q8_0/9-spans/short",
                  128: "gguf_matvec_q8_blocks/q8_0/1-tokens"}[k]
        check(tag, "f32", raw, rows, k, x, kernel=kernel)


@pytest.mark.parametrize("x_tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("tag", list(KINDS))
def test_q8_route_any_whole_number_of_blocks_and_activation_rows(tag, x_tag):
    """K from one block up, not a multiple of 2048 (Q8_0 also not of 256: the last run of 256 values is
    short); 1 to 8 activation rows; more rows than waves, fewer rows than waves of a block."""
    rng = np.random.default_rng(1804)
    per = 32 if tag == "q8_0" else 256
    widths = (32, 96, 128, 480, 1024, 5120) if tag == "q8_0" else (256, 768, 1024, 2304, 5120)
    for k in widths:
        for rows, m in ((1, 1), (3, 2), (70, 1), (33, 3), (257, 4), (19, 5), (40, 8)):
            # uniformly random block bytes for the short rows (their products overflow f16: modest weights there)
            raw = raw_bytes_for(tag, rng, rows, k) if k <= 1024 and x_tag != "f16" else weights_for(tag, rng, rows, k)
            x = rng.normal(0, 1.5, (m, k) if m > 1 else (k,)).astype(np.float32)
            note(f"q8 matvec {tag} x {x_tag} rows {rows} k {k} (blocks of {per}) m {m}")
            label = {1: 1, 2: 2, 3: 4, 4: 4, 5: 8, 8: 8}[m]
            if tag == "q4_k" and k >= 1024:   # Q4_K rows of four blocks or more: the matrix unit, four activation rows a set
                check(tag, x_tag, raw, rows, k, x, kernel=f"gguf_matvec_q8_tiles/q4_k/{1 if m == 1 else (4 if m <= 4 else 8)}-tokens")
            elif tag == "q8_0" and k >= 1024 and m == 1:   # Q8_0 rows of 256 n values, one activation row: a short last span
                check(tag, x_tag, raw, rows, k, x, kernel=f"gguf_matvec_q8_spans/q8_0/{-(-k // 2048)}-spans/short")
            else:
                check(tag, x_tag, raw, rows, k, x, kernel=f"gguf_matvec_q8_blocks/{tag}/{label}-tokens")


@pytest.mark.parametrize("tag", list(KINDS))
def test_q8_route_rows_at_even_addresses_and_strides(tag):
    """Rows that start 2, 6 or 14 bytes off a 16-byte boundary (the weight inside its allocation, and a
    row stride that is not a multiple of 16), for K = 2048 too: those leave the span kernels for the
    block-walking one, and must give what the aligned launch gives."""
    rng = np.random.default_rng(1805)
    for k, rows, m in ((2048, 37, 1), (2048, 9, 4), (4096, 21, 2), (1280 if tag != "q8_0" else 1120, 50, 3)):
        raw = raw_bytes_for(tag, rng, rows, k)
        x = rng.normal(0, 2, (m, k) if m > 1 else (k,)).astype(np.float32)
        row_bytes = raw.shape[1]
        for byte_offset, pad in ((2, 0), (6, 2), (14, 10), (0, 6)):
            padded = np.zeros((rows, row_bytes + pad), np.uint8)
            padded[:, :row_bytes] = raw
            note(f"q8 matvec {tag} k {k} rows {rows} m {m}: weight {byte_offset} bytes off, rows {pad} bytes apart")
            check(tag, "f32", padded, rows, k, x, row_stride=row_bytes + pad, byte_offset=byte_offset,
                  kernel="gguf_matvec_q8_blocks/")
        for x_tag, x_offset in (("f32", 1), ("bf16", 3), ("f16", 1)):
            note(f"q8 matvec {tag} k {k} rows {rows} m {m}: {x_tag} activations {x_offset} elements off a 16-byte boundary")
            check(tag, x_tag, weights_for(tag, rng, rows, k), rows, k, x, x_offset=x_offset)


def test_q8_route_activation_rows_in_groups_when_their_codes_do_not_fit_together():
    """Eight activation rows of 17408 values need 8 x 19.6 KB of codes: they are served two at a
    time, four dispatches over the same weight."""
    rng = np.random.default_rng(1806)
    rows, k, m = 300, 17408, 8
    raw = weights_for("q8_0", rng, rows, k)
    x = rng.normal(0, 1.0, (m, k)).astype(np.float32)
    weight = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ8_0, hc.DataType.kFloat32, k, rows)
    prepared = hc.prepare(context(), Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [m, k]))
    assert prepared.dispatch_count() == 4
    note(f"q8 matvec q8_0 [{k} -> {rows}] x {m}: activation rows in groups of two")
    check("q8_0", "f32", raw, rows, k, x, kernel="gguf_matvec_q8_blocks/q8_0/2-tokens")   # four dispatches of one launch shape are one entry


def test_q8_route_declines_what_it_does_not_serve():
    ctx = context()
    # more than eight activation rows
    weight = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ6K, hc.DataType.kFloat32, 1024, 16)
    with pytest.raises(hc.StatusError) as declined:
        hc.prepare(ctx, Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [9, 1024]))
    assert declined.value.is_unimplemented()
    # one activation row's codes beyond a block's LDS
    weight = hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ8_0, hc.DataType.kFloat32, 65536, 4)
    with pytest.raises(hc.StatusError) as declined:
        hc.prepare(ctx, Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [65536]))
    assert declined.value.is_unimplemented()
    # what it now serves: widths that are whole blocks but no multiple of 2048, eight rows of 8192
    for gguf, k, m in ((hc.GgufQuantizedType.kQ6K, 1024, 1), (hc.GgufQuantizedType.kQ6K, 8192, 8),
                       (hc.GgufQuantizedType.kQ8_0, 32, 1)):
        weight = hc.TensorDesc.gguf_weight(gguf, hc.DataType.kFloat32, k, 16)
        hc.prepare(ctx, Q8, weight, hc.TensorDesc.dense(hc.DataType.kFloat32, [m, k] if m > 1 else [k]))


@pytest.mark.parametrize("x_tag", ["f32", "bf16", "f16"])
def test_q8_route_q4_k_sub_block_dots_on_the_matrix_unit(x_tag):
    """Q4_K with rows of whole 16-byte vectors: sixteen weight rows per wave, every 32-value sub-block
    dot from a 16 x 16 x 64 int8 matrix instruction.  Row counts around the wave's sixteen and the
    block's sixty-four, every scale slot and nibble pattern (raw bytes), activation blocks of zeros
    and of equal magnitudes, rows further apart than their blocks."""
    rng = np.random.default_rng(1810)
    k = 2048
    for rows in (1, 15, 16, 17, 31, 63, 64, 65, 200, 1037):
        raw = raw_bytes_for("q4_k", rng, rows, k)
        x = rng.normal(0, 2, k).astype(np.float32)
        if rows % 2:
            x[256:512] = 0.0
            x[512:768] = np.where(np.arange(256) % 2 == 0, 1.25, -1.25)
            x[1999] = 40.0
        note(f"q8 matvec q4_k tiles x {x_tag} rows {rows}")
        check("q4_k", x_tag, raw, rows, k, x, kernel="gguf_matvec_q8_tiles/q4_k/1-tokens")
    rows = 70
    raw = raw_bytes_for("q4_k", rng, rows, k)
    padded = np.zeros((rows, raw.shape[1] + 48), np.uint8)
    padded[:, :raw.shape[1]] = raw
    note(f"q8 matvec q4_k tiles x {x_tag}: rows 48 bytes further apart than their blocks")
    check("q4_k", x_tag, padded, rows, k, rng.normal(0, 1, k).astype(np.float32), row_stride=raw.shape[1] + 48,
          kernel="gguf_matvec_q8_tiles/q4_k/1-tokens")


@pytest.mark.parametrize("x_tag", ["f32", "bf16"])
def test_q8_route_q4_k_matrix_unit_widths_tokens_and_shared_tiles(x_tag):
    """Any whole number of blocks from four up (a last group of four that overlaps the one before),
    one to eight activation rows (one, or one or two sets of four), and few rows of many blocks,
    where two or four waves share a tile and add their shares."""
    rng = np.random.default_rng(1811)
    for rows, k, m in ((40, 1024, 1), (33, 1280, 1), (50, 1536, 2), (21, 1792, 3), (70, 2304, 1), (19, 3328, 4),
                       (48, 5120, 1), (130, 5120, 4), (35, 5120, 5), (20, 4096, 8), (600, 2048, 2), (90, 6144, 7),
                       (10240, 5120, 1), (2100, 7680, 1), (64, 16384, 1), (17, 9984, 2)):
        raw = raw_bytes_for("q4_k", rng, rows, k)
        x = rng.normal(0, 1.5, (m, k) if m > 1 else (k,)).astype(np.float32)
        if m > 1:
            x[m - 1, 256:512] = 0.0
        tokens = 1 if m == 1 else (4 if m <= 4 else 8)
        note(f"q8 matvec q4_k tiles x {x_tag} rows {rows} k {k} m {m}")
        check("q4_k", x_tag, raw, rows, k, x, kernel=f"gguf_matvec_q8_tiles/q4_k/{tokens}-tokens")
    note("q8 matvec q4_k: fewer than four blocks per row, an odd row stride and unaligned activations keep the block-walking kernel")
    raw = raw_bytes_for("q4_k", rng, 20, 768)
    check("q4_k", x_tag, raw, 20, 768, rng.normal(0, 1, 768).astype(np.float32), kernel="gguf_matvec_q8_blocks/q4_k/1-tokens")
    raw = raw_bytes_for("q4_k", rng, 20, 2048)
    padded = np.zeros((20, raw.shape[1] + 2), np.uint8)
    padded[:, :raw.shape[1]] = raw
    check("q4_k", x_tag, padded, 20, 2048, rng.normal(0, 1, 2048).astype(np.float32), row_stride=raw.shape[1] + 2,
          kernel="gguf_matvec_q8_blocks/q4_k/1-tokens")
    check("q4_k", x_tag, raw, 20, 2048, rng.normal(0, 1, 2048).astype(np.float32), x_offset=1,
          kernel="gguf_matvec_q8_blocks/q4_k/1-tokens")


@pytest.mark.parametrize("x_tag", ["f32", "bf16", "f16"])
def test_q8_route_q8_0_rows_with_a_short_last_span(x_tag):
    """Q8_0 rows of 256 n values (8 blocks are 17 whole vectors) take the span kernel, whose last wave
    then has 8 to 56 blocks: one to nine spans, the lanes past the row's end neither read past it nor
    add to it, every quant and scale pattern."""
    rng = np.random.default_rng(1812)
    for k in (1024, 1280, 2304, 3840, 5120, 7168, 9216, 10496, 12544, 14592, 17408, 18176):
        for rows in (1, 5, 70) if k != 7168 else (1, 5, 70, 3072):
            raw = raw_bytes_for("q8_0", rng, rows, k) if x_tag != "f16" else weights_for("q8_0", rng, rows, k)
            x = rng.normal(0, 1.5, k).astype(np.float32)
            if rows == 5:
                x[k - 256:] = 0.0            # the last activation blocks are zeros
                x[32:64] = -2.5              # a block whose every value is the (negative) maximum
            note(f"q8 matvec q8_0 short last span x {x_tag} rows {rows} k {k}")
            check("q8_0", x_tag, raw, rows, k, x, kernel=f"gguf_matvec_q8_spans/q8_0/{-(-k // 2048)}-spans/short")
    note("q8 matvec q8_0: more than nine spans, several activation rows and misplaced rows keep the block-walking kernel")
    raw = raw_bytes_for("q8_0", rng, 20, 18688)
    check("q8_0", x_tag, raw if x_tag != "f16" else weights_for("q8_0", rng, 20, 18688), 20, 18688,
          rng.normal(0, 1, 18688).astype(np.float32), kernel="gguf_matvec_q8_blocks/q8_0/1-tokens")
    raw = weights_for("q8_0", rng, 20, 5120)
    check("q8_0", x_tag, raw, 20, 5120, rng.normal(0, 1, (2, 5120)).astype(np.float32), kernel="gguf_matvec_q8_blocks/q8_0/2-tokens")
    check("q8_0", x_tag, raw, 20, 5120, rng.normal(0, 1, 5120).astype(np.float32), byte_offset=2, kernel="gguf_matvec_q8_blocks/q8_0/1-tokens")


def test_q8_route_q4_k_matrix_unit_seeded_random_shapes():
    """Forty seeded draws of (rows, blocks per row, activation rows, activation type, row padding):
    whatever combination of tile sharing, overlapped last group, token sets and quantising rounds they
    hit must agree with the oracle like the hand-picked cases."""
    rng = np.random.default_rng(1813)
    for case in range(40):
        blocks = int(rng.integers(4, 41))
        k = 256 * blocks
        m = int(rng.integers(1, 9))
        tokens = 1 if m == 1 else (4 if m <= 4 else 8)
        if (1 + tokens) * k + tokens * blocks * 36 + 1024 * max(tokens // 4, 1) > 65536:
            m, tokens = 1, 1                                   # the codes of more rows would not fit a block's LDS
        rows = int(rng.choice([1, 7, 16, 33, 64, 100, 257, 1000, 3000]))
        x_tag = ("f32", "bf16", "f16")[case % 3]
        pad = int(rng.choice([0, 16, 48]))
        raw = raw_bytes_for("q4_k", rng, rows, k) if x_tag != "f16" else weights_for("q4_k", rng, rows, k)
        padded = np.zeros((rows, raw.shape[1] + pad), np.uint8)
        padded[:, :raw.shape[1]] = raw
        x = rng.normal(0, 1.5, (m, k) if m > 1 else (k,)).astype(np.float32)
        note(f"q8 matvec q4_k tiles draw {case}: rows {rows} k {k} m {m} x {x_tag} pad {pad}")
        check("q4_k", x_tag, padded, rows, k, x, row_stride=raw.shape[1] + pad, kernel=f"gguf_matvec_q8_tiles/q4_k/{tokens}-tokens")
