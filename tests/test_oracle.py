"""Pins the CPU oracle (oracle/hyle_oracle.c) before anything is compared to it.

Three independent anchors per function:
  * the committed golden vectors (tests/golden/scalar_floor_vectors.npz: outputs of
    the reference's own scalar floor compiled from its sources);
  * the live reference scalar floor (oracle/_ref) where it was built;
  * what the mathematics fixes: float64 closed forms, IEEE identities, brute force,
    and the known-answer cases of the reference's own tests (cited per test).
"""
from __future__ import annotations

import math
import os

import numpy as np
import pytest

from oracle import lib as orc
from oracle import ref

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "scalar_floor_vectors.npz"))
needs_ref = pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (no reference tree)")


def f32(words):
    return np.asarray(words, np.uint32).view(np.float32)


def same_bits_or_nan32(got, want):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


# ---------------------------------------------------------------- codecs ---
def bf16_rne_independent(words: np.ndarray) -> np.ndarray:
    """RN-even by comparing distances to the two neighbouring bf16 values in float64."""
    words = words.astype(np.uint32)
    sign = words & 0x80000000
    mag = words & 0x7FFFFFFF
    lo = mag & 0xFFFF0000
    hi = lo + 0x10000
    x = mag.view(np.float32).astype(np.float64)
    lo_v = lo.view(np.float32).astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        # the neighbour above the largest finite bf16 is 2^128 for rounding purposes
        hi_v = np.where(hi >= 0x7F800000, 2.0 ** 128, hi.view(np.float32).astype(np.float64))
    below, above = x - lo_v, hi_v - x
    up = (above < below) | ((above == below) & (((lo >> 16) & 1) == 1))
    out = np.where(up, hi, lo)
    return ((out | sign) >> 16).astype(np.uint16)


def test_bf16_codec_closed_form_and_golden():
    words = GOLD["codec_f32_words"]
    got = orc.from_f32(orc.BF16, words.view(np.float32))
    assert np.array_equal(got, GOLD["codec_bf16_bits"])
    finite = (words & 0x7FFFFFFF) < 0x7F800000
    assert np.array_equal(got[finite], bf16_rne_independent(words[finite]))
    # inf keeps its pattern, NaN keeps the upper payload and gains bit 6
    # (include/hyle/simd/dtype.h:114-121)
    assert orc.f32_bits_to_bf16(0x7F800000) == 0x7F80
    assert orc.f32_bits_to_bf16(0xFF800000) == 0xFF80
    assert orc.f32_bits_to_bf16(0x7F800001) == 0x7FC0
    assert orc.f32_bits_to_bf16(0x7FA00000) == 0x7FE0
    assert orc.f32_bits_to_bf16(0xFF812345) == 0xFFC1
    # decode is a shift
    all16 = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(orc.to_f32(orc.BF16, all16).view(np.uint32), all16.astype(np.uint32) << 16)
    # every bf16 value survives a round trip
    back = orc.from_f32(orc.BF16, orc.to_f32(orc.BF16, all16))
    nan = (all16 & 0x7FFF) > 0x7F80
    assert np.array_equal(back[~nan], all16[~nan])
    assert np.array_equal(back[nan], all16[nan] | 0x40)


def test_f16_codec_against_ieee_and_golden():
    all16 = np.arange(65536, dtype=np.uint16)
    dec = orc.to_f32(orc.F16, all16)
    assert np.array_equal(dec.view(np.uint32), GOLD["codec_f16_all_to_f32_words"])
    same_bits_or_nan32(dec, all16.view(np.float16).astype(np.float32))  # numpy's IEEE binary16
    words = GOLD["codec_f32_words"]
    enc = orc.from_f32(orc.F16, words.view(np.float32))
    assert np.array_equal(enc, GOLD["codec_f16_bits"])
    vals = words.view(np.float32)
    ok = ~np.isnan(vals)
    with np.errstate(over="ignore"):
        assert np.array_equal(enc[ok], vals[ok].astype(np.float16).view(np.uint16))
    assert np.all((enc[~ok] & 0x7FFF) == 0x7FFF)  # NaN -> mantissa 0x3FF (dtype.h:72-74)
    back = orc.from_f32(orc.F16, dec)
    nan = (all16 & 0x7FFF) > 0x7C00
    assert np.array_equal(back[~nan], all16[~nan])


@needs_ref
def test_codecs_match_reference_floor_on_random_words():
    rng = np.random.default_rng(5)
    words = rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    vals = words.view(np.float32)
    assert np.array_equal(orc.from_f32(orc.BF16, vals), ref.f32_to_bf16(vals))
    assert np.array_equal(orc.from_f32(orc.F16, vals), ref.f32_to_f16(vals))


# ------------------------------------------------------- shapes/offsets ---
def test_broadcast_shape_numpy_rule():
    # src/compute_ops/operation.cc:249-278
    assert orc.broadcast_shape([4096, 2048], [2048]) == [4096, 2048]
    assert orc.broadcast_shape([2, 3], [3]) == [2, 3]
    assert orc.broadcast_shape([2, 1, 5], [7, 1]) == [2, 7, 5]
    assert orc.broadcast_shape([], [3]) == [3]
    assert orc.broadcast_shape([], []) == []
    assert orc.broadcast_shape([0, 3], [1]) == [0, 3]
    assert orc.broadcast_shape([2, 3], [4]) is None
    assert orc.broadcast_shape([1] * 9, [1]) is None
    rng = np.random.default_rng(0)
    for _ in range(200):
        a = [int(rng.choice([1, 2, 3, 5])) for _ in range(rng.integers(0, 5))]
        b = [int(rng.choice([1, 2, 3, 5])) for _ in range(rng.integers(0, 5))]
        try:
            want = list(np.broadcast_shapes(tuple(a), tuple(b)))
        except ValueError:
            want = None
        assert orc.broadcast_shape(a, b) == want


def test_broadcast_offsets_match_numpy_strides():
    # src/compute_provider_native/native_plan.h:135-174
    rng = np.random.default_rng(1)
    for _ in range(50):
        out_dims = [int(rng.integers(1, 5)) for _ in range(rng.integers(1, 5))]
        in_rank = int(rng.integers(0, len(out_dims) + 1))
        in_dims = [d if rng.random() < 0.6 else 1 for d in out_dims[len(out_dims) - in_rank:]]
        arr = np.arange(int(np.prod(in_dims, dtype=np.int64)), dtype=np.float32).reshape(in_dims)
        expanded = np.broadcast_to(arr, out_dims).reshape(-1)
        strides = orc.dense_strides(in_dims, orc.F32)
        for linear in range(expanded.size):
            off = orc.broadcast_byte_offset(in_dims, strides, out_dims, linear)
            assert arr.reshape(-1)[off // 4] == expanded[linear]
        assert orc.logical_byte_offset(out_dims, orc.dense_strides(out_dims, orc.F32), 3 % expanded.size) == \
            4 * (3 % expanded.size)


# -------------------------------------------------------------- binary ---
def test_binary_known_answers_from_reference_tests():
    # tests/compute_provider_native/elementwise_test.cc:532-565
    left = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    right = np.array([10, 20, 30], np.float32)
    assert np.array_equal(orc.binary(orc.ADD, orc.F32, left, right),
                          np.array([[11, 22, 33], [14, 25, 36]], np.float32))
    # tests/compute_provider_native/elementwise_test.cc:480-530
    l6 = np.array([-2.0, -0.0, 1.0, 4.0, 8.0, np.nan], np.float32)
    r6 = np.array([1.0, -3.0, 2.0, 0.5, -2.0, 7.0], np.float32)
    with np.errstate(invalid="ignore"):
        same_bits_or_nan32(orc.binary(orc.ADD, orc.F32, l6, r6), l6 + r6)
        same_bits_or_nan32(orc.binary(orc.SUBTRACT, orc.F32, l6, r6), l6 - r6)
        same_bits_or_nan32(orc.binary(orc.MULTIPLY, orc.F32, l6, r6), l6 * r6)
        same_bits_or_nan32(orc.binary(orc.DIVIDE, orc.F32, l6, r6), l6 / r6)
        same_bits_or_nan32(orc.binary(orc.MINIMUM, orc.F32, l6, r6), np.fmin(l6, r6))
        same_bits_or_nan32(orc.binary(orc.MAXIMUM, orc.F32, l6, r6), np.fmax(l6, r6))


def test_binary_is_ieee_and_chain_rounds_twice():
    rng = np.random.default_rng(2)
    a = rng.normal(0, 1, (37, 129)).astype(np.float32)
    b = rng.uniform(-1, 1, 129).astype(np.float32)
    s = np.array([0.5], np.float32)
    t = orc.binary(orc.ADD, orc.F32, a, b)
    assert np.array_equal(t, a + b)  # numpy float32 add is the IEEE closed form
    assert np.array_equal(orc.binary(orc.MULTIPLY, orc.F32, t, s), (a + b) * np.float32(0.5))
    assert np.array_equal(orc.binary_chain(orc.ADD, orc.MULTIPLY, orc.F32, a, b, s),
                          (a + b) * np.float32(0.5))
    # an fma would differ here: (x + y) rounded, then times z
    x = np.array([1.0], np.float32)
    y = np.array([2.0 ** -24], np.float32)
    z = np.array([3.0], np.float32)
    assert orc.binary_chain(orc.ADD, orc.MULTIPLY, orc.F32, x, y, z)[0] == np.float32(3.0)


def test_binary_narrow_rounds_once_per_op():
    # decode -> f32 op -> RN-even store (elementwise.cc:135-147); the bf16 sum of two
    # bf16 numbers is exact in f32 except for rare far-exponent cases, so compare with a
    # float64 sum rounded twice (f32 then bf16)
    rng = np.random.default_rng(3)
    a = orc.from_f32(orc.BF16, rng.normal(0, 1, 4097).astype(np.float32))
    b = orc.from_f32(orc.BF16, rng.normal(0, 1, 4097).astype(np.float32))
    got = orc.binary(orc.ADD, orc.BF16, a, b)
    want32 = (orc.to_f32(orc.BF16, a).astype(np.float64) + orc.to_f32(orc.BF16, b).astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, bf16_rne_independent(want32.view(np.uint32)))
    # chain through the storage type: intermediate is rounded to bf16
    c = orc.from_f32(orc.BF16, rng.normal(0, 1, 4097).astype(np.float32))
    step = orc.binary(orc.MULTIPLY, orc.BF16, got, c)
    assert np.array_equal(orc.binary_chain(orc.ADD, orc.MULTIPLY, orc.BF16, a, b, c), step)


def test_binary_strided_and_zero_stride_inputs():
    # a [3,4] view with a padded row stride, and a stride-0 broadcast row
    storage = np.arange(3 * 6, dtype=np.float32)
    dims, strides = [3, 4], [24, 4]
    row = np.array([100.0], np.float32)
    got = orc.binary_raw(orc.ADD, orc.F32, storage, dims, strides, row, [1, 1], [0, 0], [3, 4])
    want = storage.reshape(3, 6)[:, :4] + np.float32(100.0)
    assert np.array_equal(got, want)


# ---------------------------------------------------------- activations ---
def silu64(x):
    x = np.asarray(x, np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        out = x / (1.0 + np.exp(-x))
    out = np.where(np.isneginf(x), 0.0, out)
    return out


def test_silu_swiglu_golden_bit_exact():
    x, u = f32(GOLD["act_x_f32_words"]), f32(GOLD["act_u_f32_words"])
    same_bits_or_nan32(orc.silu(orc.F32, x), f32(GOLD["silu_f32_words"]))
    same_bits_or_nan32(orc.swiglu(orc.F32, x, u), f32(GOLD["swiglu_f32_words"]))
    for tid, tag in ((orc.BF16, "bf16"), (orc.F16, "f16")):
        xs, us = GOLD[f"act_x_{tag}"], GOLD[f"act_u_{tag}"]
        assert np.array_equal(orc.silu(tid, xs), GOLD[f"silu_{tag}"])
        assert np.array_equal(orc.swiglu(tid, xs, us), GOLD[f"swiglu_{tag}"])
    all_gate = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(orc.silu(orc.BF16, all_gate), GOLD["silu_bf16_all"])


def test_silu_closed_form_and_reference_test_cases():
    # tests/simd/math_test.cc:689-709: ramp inputs, tolerance |e|*8e-6 + 2e-6
    for n in (1, 7, 8, 9, 257):
        x = (-12.0 + 24.0 * np.arange(1, n + 1, dtype=np.float32) / np.float32(n + 1)).astype(np.float32)
        got = orc.silu(orc.F32, x).astype(np.float64)
        want = silu64(x)
        assert np.all(np.abs(got - want) <= np.abs(want) * 8e-6 + 2e-6)
    # tests/simd/math_test.cc:758-780: -inf -> 0, +inf -> +inf, NaN -> NaN
    sp = np.array([-np.inf, -0.0, 0.0, np.inf, np.nan, -2.0], np.float32)
    out = orc.silu(orc.F32, sp)
    assert out[0] == 0.0 and not np.signbit(out[0])
    assert out[3] == np.inf and np.isnan(out[4])
    assert abs(out[5] - (-2.0 / (1.0 + math.exp(2.0)))) < 1e-7
    # tests/simd/math_test.cc:1052-1097: split gated rows
    n = 259
    i = np.arange(n, dtype=np.float32)
    gate = (-9.0 + 18.0 * i / np.float32(n - 1)).astype(np.float32)
    value = (1.5 * np.cos(i * np.float32(0.11))).astype(np.float32)
    got = orc.swiglu(orc.F32, gate, value).astype(np.float64)
    want = silu64(gate) * value.astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 8e-6 + 2e-6)
    # packed halves: row = [gate | value] (elementwise.cc:192-208)
    packed = np.concatenate([gate[:256].reshape(2, 128), value[:256].reshape(2, 128)], axis=1)
    assert np.array_equal(orc.swiglu_packed(orc.F32, packed),
                          orc.swiglu(orc.F32, gate[:256], value[:256]).reshape(2, 128))


def test_swiglu_bf16_rounds_once():
    rng = np.random.default_rng(4)
    g = orc.from_f32(orc.BF16, rng.normal(0, 2, 5000).astype(np.float32))
    u = orc.from_f32(orc.BF16, rng.normal(0, 2, 5000).astype(np.float32))
    got = orc.swiglu(orc.BF16, g, u)
    wide = orc.swiglu(orc.F32, orc.to_f32(orc.BF16, g), orc.to_f32(orc.BF16, u))
    assert np.array_equal(got, orc.from_f32(orc.BF16, wide))
    # float64 closed form lands within one bf16 step
    want = silu64(orc.to_f32(orc.BF16, g)) * orc.to_f32(orc.BF16, u).astype(np.float64)
    err = np.abs(orc.to_f32(orc.BF16, got).astype(np.float64) - want)
    assert np.all(err <= np.abs(want) * 2.0 ** -8 + 1e-38)


@needs_ref
def test_activations_match_reference_floor_live():
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.normal(0, 4, 200000), rng.uniform(-110, 110, 50000)]).astype(np.float32)
    u = rng.normal(0, 2, x.size).astype(np.float32)
    same_bits_or_nan32(orc.silu(orc.F32, x), ref.silu(0, x))
    same_bits_or_nan32(orc.swiglu(orc.F32, x, u), ref.swiglu(0, x, u))
    xb, ub = orc.from_f32(orc.BF16, x), orc.from_f32(orc.BF16, u)
    assert np.array_equal(orc.swiglu(orc.BF16, xb, ub), ref.swiglu(2, xb, ub))
    xh, uh = orc.from_f32(orc.F16, x), orc.from_f32(orc.F16, u)
    assert np.array_equal(orc.swiglu(orc.F16, xh, uh), ref.swiglu(1, xh, uh))


# -------------------------------------------------------------- RMSNorm ---
def test_rms_norm_golden_bit_exact():
    for n in (1, 7, 127, 128, 129, 257, 2048):
        x, w = GOLD[f"rms_x_f32_{n}"], GOLD[f"rms_w_f32_{n}"]
        same_bits_or_nan32(orc.rms_norm(orc.F32, x, w, 1e-6), GOLD[f"rms_y_f32_{n}"])
        same_bits_or_nan32(orc.rms_norm(orc.F32, x, None, 1e-5), GOLD[f"rms_y_f32_nw_{n}"])
        assert np.array_equal(orc.rms_norm(orc.BF16, GOLD[f"rms_x_bf16_{n}"], GOLD[f"rms_w_bf16_{n}"], 1e-6),
                              GOLD[f"rms_y_bf16_{n}"])
        assert np.array_equal(orc.rms_norm(orc.F16, GOLD[f"rms_x_f16_{n}"], GOLD[f"rms_w_f16_{n}"], 1e-5),
                              GOLD[f"rms_y_f16_{n}"])


def test_rms_norm_closed_form_reference_generator():
    # tests/simd/math_test.cc:1168-1199
    n, eps = 257, 1e-5
    i = np.arange(n, dtype=np.float32)
    x = (3.0 * np.sin(i * np.float32(0.13)) + 0.25).astype(np.float32)
    w = (0.75 + 0.5 * i / np.float32(n)).astype(np.float32)
    inv = 1.0 / math.sqrt(float(np.sum(x.astype(np.float64) ** 2)) / n + eps)
    want = x.astype(np.float64) * inv * w.astype(np.float64)
    got = orc.rms_norm(orc.F32, x, w, eps).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 3e-5 + 3e-6)
    got_nw = orc.rms_norm(orc.F32, x, None, eps).astype(np.float64)
    assert np.all(np.abs(got_nw - x * inv) <= np.abs(x * inv) * 3e-5 + 3e-6)
    # a constant row of c normalises to c/sqrt(c^2+eps) * w exactly computable
    const = np.full(64, 2.0, np.float32)
    y = orc.rms_norm(orc.F32, const, None, 0.0)
    assert np.array_equal(y, np.ones(64, np.float32))


def test_rms_norm_bf16_domain_test_and_native_variant():
    # tests/compute_provider_native/normalization_test.cc:186-199 values, hidden set :315-323
    for hidden in (1, 127, 128, 129, 2048, 4096):
        rows = 3
        idx = np.arange(rows * hidden)
        vals = np.where(idx // hidden == 1, 2.0, ((idx % 97) - 48) / 16.0).astype(np.float32)
        scale = (1.001 + (np.arange(hidden) % 7) / 16.0).astype(np.float32)
        xb = orc.from_f32(orc.BF16, vals).reshape(rows, hidden)
        wb = orc.from_f32(orc.BF16, scale)
        for eps in (1e-5, 1e-6):
            floor = orc.rms_norm(orc.BF16, xb, wb, eps)
            native = orc.rms_norm(orc.BF16, xb, wb, eps, native=True)
            xf = orc.to_f32(orc.BF16, xb).astype(np.float64)
            wf = orc.to_f32(orc.BF16, wb).astype(np.float64)
            inv = 1.0 / np.sqrt(np.mean(xf * xf, axis=1, keepdims=True) + eps)
            want = xf * inv * wf
            for got in (floor, native):
                g = orc.to_f32(orc.BF16, got).astype(np.float64)
                # half_test::expect_near: relative 0.008 + one subnormal (half_test_support.h:107-121)
                rounded = orc.to_f32(orc.BF16, orc.from_f32(orc.BF16, want.astype(np.float32))).astype(np.float64)
                assert np.all(np.abs(g - rounded) <= np.abs(rounded) * 0.008 + 9.2e-41)
            # the two accumulation orders agree to one bf16 step
            d = np.abs(floor.astype(np.int32) - native.astype(np.int32))
            assert d.max() <= 1
        # f32 weight with bf16 input (operation.cc:492-505)
        mixed = orc.rms_norm(orc.BF16, xb, scale, 1e-6, weight_type=orc.F32)
        assert mixed.shape == xb.shape


@needs_ref
def test_rms_norm_matches_reference_floor_live():
    rng = np.random.default_rng(7)
    for n in (3, 64, 1000, 2048, 6144):
        x = (rng.normal(0, 1, n) * rng.uniform(0.1, 10)).astype(np.float32)
        w = rng.normal(1, 0.1, n).astype(np.float32)
        same_bits_or_nan32(orc.rms_norm(orc.F32, x, w, 1e-6), ref.rms_norm_row(0, x, w, 1e-6))
        xb, wb = orc.from_f32(orc.BF16, x), orc.from_f32(orc.BF16, w)
        assert np.array_equal(orc.rms_norm(orc.BF16, xb, wb, 1e-6), ref.rms_norm_row(2, xb, wb, 1e-6))


# ------------------------------------------- every unary kind, gated forms ---
ABS, NEG, EXP, LOG, SQRT, RSQRT, TANH, SIGMOID, RELU, GELU, GELU_TANH, SILU, SOFTPLUS = range(13)


def test_unary_and_gated_golden_bit_exact():
    x, u = f32(GOLD["more_x_f32_words"]), f32(GOLD["more_u_f32_words"])
    for name, kind in (("gelu", GELU), ("gelu_tanh", GELU_TANH), ("sigmoid", SIGMOID), ("relu", RELU)):
        same_bits_or_nan32(orc.unary(kind, orc.F32, x), f32(GOLD[f"{name}_f32_words"]))
    same_bits_or_nan32(orc.gated(1, orc.F32, x, u), f32(GOLD["geglu_f32_words"]))
    same_bits_or_nan32(orc.gated(2, orc.F32, x, u), f32(GOLD["geglu_tanh_f32_words"]))
    for tag, type_id in (("bf16", orc.BF16), ("f16", orc.F16)):
        assert np.array_equal(orc.unary(GELU, type_id, GOLD[f"more_x_{tag}"]), GOLD[f"gelu_{tag}"])
        assert np.array_equal(orc.unary(GELU_TANH, type_id, GOLD[f"more_x_{tag}"]), GOLD[f"gelu_tanh_{tag}"])
    assert np.array_equal(orc.gated(1, orc.BF16, GOLD["more_x_bf16"], GOLD["more_u_bf16"]), GOLD["geglu_bf16"])
    assert np.array_equal(orc.gated(2, orc.BF16, GOLD["more_x_bf16"], GOLD["more_u_bf16"]), GOLD["geglu_tanh_bf16"])
    # activation 0 is the SwiGLU already pinned above
    assert np.array_equal(orc.gated(0, orc.BF16, GOLD["act_x_bf16"], GOLD["act_u_bf16"]), GOLD["swiglu_bf16"])
    assert np.array_equal(orc.unary(SILU, orc.BF16, GOLD["act_x_bf16"]), GOLD["silu_bf16"])


def test_unary_closed_forms_and_reference_test_values():
    rng = np.random.default_rng(41)
    x = np.concatenate([rng.normal(0, 3, 4000), rng.uniform(-80, 80, 1000)]).astype(np.float32)
    pos = np.abs(x) + np.float32(1e-3)
    x64, pos64 = x.astype(np.float64), pos.astype(np.float64)
    # exact kinds
    assert np.array_equal(orc.unary(ABS, orc.F32, x), np.abs(x))
    assert np.array_equal(orc.unary(NEG, orc.F32, x), -x)
    assert np.array_equal(orc.unary(SQRT, orc.F32, pos), np.sqrt(pos))          # correctly rounded both sides
    assert np.array_equal(orc.unary(RELU, orc.F32, x), np.maximum(x, np.float32(0)))
    # libm kinds against float64, a few units in the last place
    def close(got, want, rel=4e-7):
        got = got.astype(np.float64)
        assert np.all(np.abs(got - want) <= rel * np.abs(want) + 1e-45)
    with np.errstate(over="ignore"):
        close(orc.unary(EXP, orc.F32, x), np.exp(x64).astype(np.float32).astype(np.float64))
        close(orc.unary(LOG, orc.F32, pos), np.log(pos64))
        close(orc.unary(RSQRT, orc.F32, pos), 1.0 / np.sqrt(pos64))
        close(orc.unary(TANH, orc.F32, x), np.tanh(x64))
        close(orc.unary(SIGMOID, orc.F32, x), 1.0 / (1.0 + np.exp(-x64)), rel=1e-6)
        close(orc.unary(SOFTPLUS, orc.F32, x), np.log1p(np.exp(x64)), rel=2e-7)
        inner = 0.79788456080286535588 * x64 * (1 + 0.044715 * x64 * x64)
        # 1 + tanh(.) cancels for negative arguments in f32, as in the reference's own formula
        got = orc.unary(GELU_TANH, orc.F32, x[:4000]).astype(np.float64)
        want = (0.5 * x64 * (1 + np.tanh(inner)))[:4000]
        assert np.all(np.abs(got - want) <= 2e-6 * np.abs(want) + 2e-7 * np.abs(x64[:4000]))
    # special values of the scalar forms
    inf, nan = np.float32(np.inf), np.float32(np.nan)
    for kind in (GELU, GELU_TANH, SILU):
        got = orc.unary(kind, orc.F32, np.array([-inf, inf, nan, 0.0, -0.0], np.float32))
        assert got[0] == 0 and not np.signbit(got[0]) and got[1] == inf and np.isnan(got[2]) and got[3] == 0
    assert np.isnan(orc.unary(RELU, orc.F32, np.array([nan], np.float32))[0])
    relu_zero = orc.unary(RELU, orc.F32, np.array([-0.0, -1.0], np.float32))
    assert not np.signbit(relu_zero).any() and (relu_zero == 0).all()
    assert np.isnan(orc.unary(SIGMOID, orc.F32, np.array([nan], np.float32))[0])
    assert orc.unary(SIGMOID, orc.F32, np.array([-inf, inf], np.float32)).tolist() == [0.0, 1.0]
    assert orc.unary(SOFTPLUS, orc.F32, np.array([-inf, 100.0, inf], np.float32)).tolist() == [0.0, 100.0, np.inf]
    # tests/compute_provider_native/elementwise_test.cc:127-178: seven values, every kind, 3e-4 relative
    values = np.array([-2.0, -0.0, 0.25, 0.5, 1.0, 2.0, 4.0], np.float32)
    v64 = values.astype(np.float64)
    from math import erf
    with np.errstate(divide="ignore", invalid="ignore"):
        expected = {ABS: np.abs(v64), NEG: -v64, EXP: np.exp(v64), LOG: np.log(v64), SQRT: np.sqrt(v64),
                    RSQRT: 1 / np.sqrt(v64), TANH: np.tanh(v64), SIGMOID: 1 / (1 + np.exp(-v64)),
                    RELU: np.maximum(v64, 0), GELU: np.array([0.5 * v * (1 + erf(v * 0.7071067811865476)) for v in v64]),
                    SILU: v64 / (1 + np.exp(-v64)), SOFTPLUS: np.log1p(np.exp(v64))}
    for kind, want in expected.items():
        got = orc.unary(kind, orc.F32, values).astype(np.float64)
        for g, w in zip(got, want):
            if np.isnan(w):
                assert np.isnan(g)
            elif np.isinf(w):
                assert g == w
            else:
                assert abs(g - w) <= abs(w) * 3e-4 + 3e-6
    # narrow storage: decode, apply, round once
    xb = orc.from_f32(orc.BF16, x[:2000])
    for kind in (EXP, TANH, SOFTPLUS, NEG, ABS):
        want = orc.from_f32(orc.BF16, orc.unary(kind, orc.F32, orc.to_f32(orc.BF16, xb)))
        assert np.array_equal(orc.unary(kind, orc.BF16, xb), want)


@needs_ref
def test_unary_and_gated_match_reference_floor_live():
    rng = np.random.default_rng(42)
    x = np.concatenate([rng.normal(0, 3, 20000), rng.uniform(-100, 100, 5000)]).astype(np.float32)
    u = rng.normal(0, 2, x.size).astype(np.float32)
    for name, kind in (("gelu", GELU), ("gelu_tanh", GELU_TANH), ("sigmoid", SIGMOID), ("relu", RELU)):
        same_bits_or_nan32(orc.unary(kind, orc.F32, x), ref.activation(name, 0, x))
    same_bits_or_nan32(orc.gated(1, orc.F32, x, u), ref.gated("geglu", 0, x, u))
    same_bits_or_nan32(orc.gated(2, orc.F32, x, u), ref.gated("geglu_tanh", 0, x, u))
    all16 = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    for type_id in (orc.BF16, orc.F16):
        assert np.array_equal(orc.unary(GELU, type_id, all16), ref.activation("gelu", type_id, all16))
        assert np.array_equal(orc.unary(GELU_TANH, type_id, all16), ref.activation("gelu_tanh", type_id, all16))


# ------------------------------------------------------------ layer norm ---
def test_layer_norm_golden_bit_exact():
    for n in (1, 7, 127, 128, 129, 257, 2048):
        x, s, b = GOLD[f"ln_x_f32_{n}"], GOLD[f"ln_s_f32_{n}"], GOLD[f"ln_b_f32_{n}"]
        same_bits_or_nan32(orc.layer_norm(orc.F32, x, s, b, 1e-5), GOLD[f"ln_y_f32_{n}"])
        same_bits_or_nan32(orc.layer_norm(orc.F32, x, None, None, 1e-6), GOLD[f"ln_y_f32_plain_{n}"])
        for tag, type_id in (("bf16", orc.BF16), ("f16", orc.F16)):
            got = orc.layer_norm(type_id, GOLD[f"ln_x_{tag}_{n}"], GOLD[f"ln_s_{tag}_{n}"], GOLD[f"ln_b_{tag}_{n}"], 1e-5)
            assert np.array_equal(got, GOLD[f"ln_y_{tag}_{n}"])


def test_layer_norm_closed_form_and_reference_test_cases():
    # tests/simd/math_test.cc:1168-1231: generator row, affine and plain, constant row -> zeros
    n, eps = 257, 1e-5
    i = np.arange(n, dtype=np.float32)
    x = (3.0 * np.sin(i * np.float32(0.13)) + 0.25).astype(np.float32)
    w = (0.75 + 0.5 * i / np.float32(n)).astype(np.float32)
    b = (0.125 * np.cos(i * np.float32(0.07))).astype(np.float32)
    x64 = x.astype(np.float64)
    inv = 1.0 / math.sqrt(float(np.mean((x64 - x64.mean()) ** 2)) + eps)
    want = (x64 - x64.mean()) * inv * w + b
    got = orc.layer_norm(orc.F32, x, w, b, eps).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 3e-5 + 3e-6)
    plain = orc.layer_norm(orc.F32, x, None, None, eps).astype(np.float64)
    assert np.all(np.abs(plain - (x64 - x64.mean()) * inv) <= np.abs((x64 - x64.mean()) * inv) * 3e-5 + 3e-6)
    assert np.array_equal(orc.layer_norm(orc.F32, np.full(17, 3.0, np.float32), None, None, eps), np.zeros(17, np.float32))
    # tests/compute_provider_native/normalization_test.cc:69-127: plain, scale only, affine (2e-5 absolute)
    values = np.array([[1, 2, 3], [2, 4, 6]], np.float32)
    scale, bias = np.array([2, 3, 4], np.float32), np.array([10, 20, 30], np.float32)
    first = 1.0 / math.sqrt(2.0 / 3.0 + 1e-5)
    second = 2.0 / math.sqrt(8.0 / 3.0 + 1e-5)
    normalized = np.array([[-first, 0, first], [-second, 0, second]])
    assert np.all(np.abs(orc.layer_norm(orc.F32, values, None, None, 1e-5) - normalized) <= 2e-5)
    assert np.all(np.abs(orc.layer_norm(orc.F32, values, scale, None, 1e-5) - normalized * scale) <= 2e-5)
    assert np.all(np.abs(orc.layer_norm(orc.F32, values, scale, bias, 1e-5) - (normalized * scale + bias)) <= 2e-5)
    # shift invariance up to rounding: adding a constant that is exact in f32 leaves the result
    shifted = orc.layer_norm(orc.F32, (x + np.float32(64.0)).astype(np.float32), None, None, eps).astype(np.float64)
    assert np.all(np.abs(shifted - plain) <= 2e-4)
    # narrow inputs with f32 parameters round once
    xb = orc.from_f32(orc.BF16, x)
    mixed = orc.layer_norm(orc.BF16, xb, w, b, eps, param_type=orc.F32)
    xf = orc.to_f32(orc.BF16, xb).astype(np.float64)
    inv_b = 1.0 / math.sqrt(float(np.mean((xf - xf.mean()) ** 2)) + eps)
    want_b = orc.from_f32(orc.BF16, ((xf - xf.mean()) * inv_b * w + b).astype(np.float32))
    assert np.abs(mixed.astype(np.int32) - want_b.astype(np.int32)).max() <= 1


@needs_ref
def test_layer_norm_matches_reference_floor_live():
    rng = np.random.default_rng(8)
    for n in (3, 64, 1000, 2048, 6144):
        x = (rng.normal(0.3, 1, n) * rng.uniform(0.1, 10)).astype(np.float32)
        s, b = rng.normal(1, 0.1, n).astype(np.float32), rng.normal(0, 0.5, n).astype(np.float32)
        same_bits_or_nan32(orc.layer_norm(orc.F32, x, s, b, 1e-5), ref.layer_norm_row(0, x, s, b, 1e-5))
        same_bits_or_nan32(orc.layer_norm(orc.F32, x, None, None, 1e-5), ref.layer_norm_row(0, x, None, None, 1e-5))
        for type_id in (orc.BF16, orc.F16):
            xn, sn, bn = orc.from_f32(type_id, x), orc.from_f32(type_id, s), orc.from_f32(type_id, b)
            assert np.array_equal(orc.layer_norm(type_id, xn, sn, bn, 1e-5), ref.layer_norm_row(type_id, xn, sn, bn, 1e-5))


# -------------------------------------------------------------- softmax ---
def softmax64(x):
    x = np.asarray(x, np.float64)
    e = np.exp(x - np.max(x))
    return e / e.sum()


def test_softmax_golden_bit_exact():
    for n in (1, 7, 8, 9, 257, 4096):
        same_bits_or_nan32(orc.softmax_f32_row(GOLD[f"softmax_x_{n}"]), GOLD[f"softmax_y_{n}"])
    same_bits_or_nan32(orc.softmax_f32_row(GOLD["softmax_x_masked"]), GOLD["softmax_y_masked"])
    same_bits_or_nan32(orc.softmax_f32_row(GOLD["softmax_x_wide"]), f32(GOLD["softmax_y_wide_words"]))


def test_softmax_reference_test_cases():
    # tests/simd/math_test.cc:1268-1311
    for n in (1, 7, 8, 9, 257, 4096):
        i = np.arange(n, dtype=np.float32)
        x = (np.sin(i * np.float32(0.7)) * np.float32(9.0) + np.cos(i * np.float32(0.13))).astype(np.float32)
        got = orc.softmax_f32_row(x)
        assert np.all(np.abs(got.astype(np.float64) - softmax64(x)) <= 2e-6)
        assert abs(float(got.astype(np.float64).sum()) - 1.0) <= 2e-5
    # tests/simd/math_test.cc:1314-1337
    inf = np.inf
    m = orc.softmax_f32_row(np.array([0.0, -inf, -1.0, -inf], np.float32))
    assert m[1] == 0.0 and m[3] == 0.0 and abs(float(m[0]) + float(m[2]) - 1.0) <= 2e-6
    for row in ([0.0, np.nan, -1.0, 2.0], [0.0, inf, -1.0, 2.0], [-inf] * 4):
        assert np.all(np.isnan(orc.softmax_f32_row(np.array(row, np.float32))))


def test_softmax_masks_scale_and_broadcast():
    # tests/compute_provider_native/transformer_test.cc:259-301 (scale 0.5, bool mask {1,0,1} over [1,3])
    vals = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    mask = np.array([[1, 0, 1]], np.uint8)
    got = orc.softmax(orc.F32, vals, scale=0.5, mask_kind=orc.MASK_BOOLEAN, mask=mask)
    want = np.stack([softmax64([0.5, -np.inf, 1.5]), softmax64([2.0, -np.inf, 3.0])])
    assert np.all(np.abs(got - want) <= 2e-6) and got[0, 1] == 0.0 and got[1, 1] == 0.0
    # tests/compute_provider_native/transformer_test.cc:337-387 (additive -inf, all-masked -> NaN)
    add = np.array([[0, -np.inf, -1]], np.float32)
    got = orc.softmax(orc.F32, vals, mask_kind=orc.MASK_ADDITIVE, mask=add)
    want = np.stack([softmax64([1, -np.inf, 2]), softmax64([4, -np.inf, 5])])
    assert np.all(np.abs(got - want) <= 2e-6)
    allm = np.full((1, 3), -np.inf, np.float32)
    assert np.all(np.isnan(orc.softmax(orc.F32, vals, mask_kind=orc.MASK_ADDITIVE, mask=allm)))
    # causal mask broadcast over heads equals per-row prefix softmax
    rng = np.random.default_rng(8)
    s = rng.normal(0, 3, (3, 16, 16)).astype(np.float32)
    causal = np.tril(np.ones((16, 16), np.uint8))
    got = orc.softmax(orc.F32, s, mask_kind=orc.MASK_BOOLEAN, mask=causal)
    for h in range(3):
        for q in range(16):
            assert np.all(np.abs(got[h, q, :q + 1] - softmax64(s[h, q, :q + 1])) <= 2e-6)
            assert np.all(got[h, q, q + 1:] == 0.0)


@needs_ref
def test_softmax_matches_reference_floor_live():
    rng = np.random.default_rng(9)
    for n in (5, 64, 1023, 4096, 151936):
        x = rng.normal(0, 3, n).astype(np.float32)
        same_bits_or_nan32(orc.softmax_f32_row(x), ref.softmax_f32(x))


# ---------------------------------------------------- reductions/argmax ---
def test_reduce_last_axis_nan_and_identities():
    # src/compute_provider_native/reduction.cc:24-47
    rng = np.random.default_rng(10)
    x = rng.normal(0, 1, (7, 300)).astype(np.float32)
    assert np.array_equal(orc.reduce_last_axis(orc.MAX, orc.F32, x), x.max(axis=1))
    assert np.array_equal(orc.reduce_last_axis(orc.MIN, orc.F32, x), x.min(axis=1))
    s = orc.reduce_last_axis(orc.SUM, orc.F32, x).astype(np.float64)
    assert np.all(np.abs(s - x.astype(np.float64).sum(axis=1)) <= 1e-4)
    m = orc.reduce_last_axis(orc.MEAN, orc.F32, x).astype(np.float64)
    assert np.all(np.abs(m - x.astype(np.float64).mean(axis=1)) <= 1e-6)
    x[2, 17] = np.nan
    assert np.isnan(orc.reduce_last_axis(orc.MAX, orc.F32, x)[2])
    assert np.isnan(orc.reduce_last_axis(orc.MIN, orc.F32, x)[2])
    # tests/simd/search_test.cc:196-206: max of signed zeros is +0, min is -0, in any order
    for zeros in ([0.0, -0.0, -1.0], [-0.0, 0.0, -1.0]):
        assert not np.signbit(orc.reduce_last_axis(orc.MAX, orc.F32, np.array([zeros], np.float32))[0])
    for zeros in ([0.0, -0.0, 1.0], [-0.0, 0.0, 1.0]):
        assert np.signbit(orc.reduce_last_axis(orc.MIN, orc.F32, np.array([zeros], np.float32))[0])
    empty = np.empty((2, 0), np.float32)
    assert np.all(orc.reduce_last_axis(orc.MAX, orc.F32, empty) == -np.inf)
    assert np.all(orc.reduce_last_axis(orc.MIN, orc.F32, empty) == np.inf)
    assert np.all(np.isnan(orc.reduce_last_axis(orc.MEAN, orc.F32, empty)))


def test_argmax_known_answers_from_reference_tests():
    # tests/simd/search_test.cc:166-186
    data = np.full(513, 4.0, np.float32)
    data[[9, 301]] = -17.0
    data[[13, 477]] = 29.0
    assert orc.index_of_max(data) == 13
    assert orc.topk1(data[None, :])[1][0] == 13
    data[[71, 402]] = np.nan
    assert orc.index_of_max(data) == 71           # simd rule: first NaN wins
    v, i = orc.topk1(data[None, :])               # TopK rule: NaN ranks last
    assert i[0] == 13 and v[0] == 29.0
    # tests/simd/search_test.cc:189-213: signed zeros tie, lowest index
    z = np.zeros(37, np.float32)
    z[[1, 19]] = -0.0
    assert orc.index_of_max(z) == 0 and orc.topk1(z[None, :])[1][0] == 0
    nz = np.full(5, -0.0, np.float32)
    nz[3] = 0.0
    assert orc.topk1(nz[None, :])[1][0] == 0      # -0 == +0
    assert orc.topk1(np.full((1, 4), np.nan, np.float32))[1][0] == 0
    # brute force
    rng = np.random.default_rng(11)
    for _ in range(200):
        row = rng.integers(-3, 4, rng.integers(1, 40)).astype(np.float32)
        assert orc.topk1(row[None, :])[1][0] == int(np.argmax(row))
        assert orc.index_of_max(row) == int(np.argmax(row))


# ----------------------------------------------------------------- Q8_0 ---
def make_q8(rng, rows, k):
    nb = k // 32
    d = rng.uniform(1e-3, 2e-2, (rows, nb)).astype(np.float16)
    q = rng.integers(-127, 128, (rows, nb, 32), dtype=np.int8)
    blocks = np.empty((rows, nb, 34), np.uint8)
    blocks[:, :, :2] = d.view(np.uint8).reshape(rows, nb, 2)
    blocks[:, :, 2:] = q.view(np.uint8)
    return blocks.reshape(rows, nb * 34), d, q


def test_q8_0_layout_and_exact_product():
    # src/compute_ops/low_precision.cc:28-29: 32 elements / 34 bytes
    rng = np.random.default_rng(12)
    rows, k = 5, 256
    blocks, d, q = make_q8(rng, rows, k)
    out, sumsq, sumsq_r = orc.q8_0_dequant_bf16(blocks, rows, k)
    # independent evaluation in float64: the product of an 8-bit and an 11-bit
    # significand is exact in float64 and in float32 alike
    y64 = q.astype(np.float64) * d.astype(np.float64)[:, :, None]
    y32 = y64.astype(np.float32)
    assert np.array_equal(y32.astype(np.float64), y64)            # exact in f32
    assert np.array_equal(orc.q8_0_dequant_f32(blocks, rows, k), y32.reshape(rows, k))
    assert np.array_equal(out, bf16_rne_independent(y32.view(np.uint32)).reshape(rows, k))
    want = (y64 ** 2).reshape(rows, k).sum(axis=1)
    assert np.all(np.abs(sumsq - want) <= 1e-5 * want)
    yr = orc.to_f32(orc.BF16, out).astype(np.float64)
    assert np.all(np.abs(sumsq_r - (yr ** 2).sum(axis=1)) <= 1e-5 * (yr ** 2).sum(axis=1))
    # row stride larger than the packed row
    padded = np.zeros((rows, blocks.shape[1] + 6), np.uint8)
    padded[:, :blocks.shape[1]] = blocks
    out2, _, _ = orc.q8_0_dequant_bf16(padded, rows, k, row_stride=padded.shape[1])
    assert np.array_equal(out2, out)


def test_q8_0_every_scale_times_every_quant():
    # all 65536 fp16 scale patterns x all 256 int8 values, against float64 -> f32 -> bf16
    scales = np.arange(65536, dtype=np.uint16)
    quants = np.arange(-128, 128, dtype=np.int8)
    d64 = scales.view(np.float16).astype(np.float64)
    for start in range(0, 256, 32):
        q = quants[start:start + 32]
        blocks = np.empty((65536, 34), np.uint8)
        blocks[:, :2] = scales.view(np.uint8).reshape(-1, 2)
        blocks[:, 2:] = q.view(np.uint8)[None, :]
        out, _, _ = orc.q8_0_dequant_bf16(blocks, 65536, 32)
        with np.errstate(invalid="ignore", over="ignore"):
            y32 = (d64[:, None] * q.astype(np.float64)[None, :]).astype(np.float32)
        ok = np.isfinite(y32)
        assert np.array_equal(out[ok], bf16_rne_independent(y32.view(np.uint32))[ok])
        nan = np.isnan(y32)
        assert np.all((out[nan] & 0x7FFF) > 0x7F80)


# ---- Cast / Copy ------------------------------------------------------------------------------
def test_cast_known_answers_from_reference_tests():
    # tests/compute_provider_native/cast_test.cc:139-143 (f32 -> f16 bit patterns)
    got = orc.cast(orc.F32, orc.F16, np.array([0.0, 1.0, -2.0, 0.5, 65504.0], np.float32), [5])
    assert got.tolist() == [0x0000, 0x3C00, 0xC000, 0x3800, 0x7BFF]
    # :177-183 (f16 [2,2] with byte strides {5,2} -> f32)
    physical = np.zeros(9, np.uint8)
    for bits, offset in zip((0x3C00, 0x4000, 0x4200, 0x4400), (0, 2, 5, 7)):
        physical[offset:offset + 2] = np.frombuffer(np.uint16(bits).tobytes(), np.uint8)
    got = orc.cast(orc.F16, orc.F32, physical, [2, 2], [5, 2])
    assert got.tolist() == [[1.0, 2.0], [3.0, 4.0]]
    # :232-247 (int32 -> f32 on both sides of the 2^24 ties and the 2^31 carry), dense and with
    # the odd byte strides {51, 5} of the reference test
    values = np.array([0, 1, -1, 129279, 16777215, 16777216, 16777217, 16777219, -16777217, -16777219,
                       2147483520, 2147483583, 2147483584, 2**31 - 1, -2**31, -2**31 + 1], np.int64).astype(np.int32)
    expected = [0x00000000, 0x3F800000, 0xBF800000, 0x47FC7F80, 0x4B7FFFFF, 0x4B800000, 0x4B800000, 0x4B800002,
                0xCB800000, 0xCB800002, 0x4EFFFFFF, 0x4EFFFFFF, 0x4F000000, 0x4F000000, 0xCF000000, 0xCF000000]
    assert orc.cast(orc.I32, orc.F32, values, [2, 8]).view(np.uint32).reshape(-1).tolist() == expected
    physical = np.full(51 + 7 * 5 + 4, 0x5A, np.uint8)
    for i, v in enumerate(values):
        offset = (i // 8) * 51 + (i % 8) * 5
        physical[offset:offset + 4] = np.frombuffer(np.int32(v).tobytes(), np.uint8)
    assert orc.cast(orc.I32, orc.F32, physical, [2, 8], [51, 5]).view(np.uint32).reshape(-1).tolist() == expected
    # :389-396 (truth keeps signed zeros false, subnormals / inf / NaN true; Bool -> float is 1 or 0)
    for type_id, words, one, dtype in (
            (orc.F32, [0, 0x80000000, 1, 0x80000001, 0x3F800000, 0xBF800000, 0x7F800000, 0x7FC00001], 0x3F800000, np.uint32),
            (orc.F16, [0, 0x8000, 1, 0x8001, 0x3C00, 0xBC00, 0x7C00, 0x7E01], 0x3C00, np.uint16),
            (orc.BF16, [0, 0x8000, 1, 0x8001, 0x3F80, 0xBF80, 0x7F80, 0x7FC1], 0x3F80, np.uint16)):
        assert orc.cast(type_id, orc.BOOL, np.array(words, dtype), [2, 4]).reshape(-1).tolist() == [0, 0, 1, 1, 1, 1, 1, 1]
        boolean = np.array([0, 1, 2, 255, 1, 0, 0, 1], np.uint8)
        got = orc.cast(orc.BOOL, type_id, boolean, [2, 4]).view(dtype).reshape(-1).tolist()
        assert got == [one if b else 0 for b in boolean]
    # :296-301: the reverse pair is not defined
    with pytest.raises(ValueError):
        orc.cast(orc.F32, orc.I32, np.zeros(4, np.float32), [4])


def test_cast_matches_independent_conversions():
    rng = np.random.default_rng(31)
    # int32 -> f32: numpy converts with round-to-nearest-even
    ints = np.concatenate([rng.integers(-2**31, 2**31, 200000, dtype=np.int64),
                           (1 << np.arange(31, dtype=np.int64)), (1 << np.arange(31, dtype=np.int64)) + 1,
                           -(1 << np.arange(32, dtype=np.int64)), (1 << np.arange(1, 32, dtype=np.int64)) - 1]).astype(np.int32)
    assert np.array_equal(orc.cast(orc.I32, orc.F32, ints, [ints.size]).view(np.uint32),
                          ints.astype(np.float32).view(np.uint32))
    # float -> float: decode to f32 and encode once, i.e. the pinned codecs; f16 -> f32 -> bf16 etc.
    words = rng.integers(0, 1 << 32, 300000, dtype=np.uint64).astype(np.uint32)
    finite = f32(words)
    via_f16 = orc.cast(orc.F32, orc.F16, finite, [finite.size])
    assert np.array_equal(via_f16, orc.from_f32(orc.F16, finite))
    same_bits_or_nan32(orc.cast(orc.F16, orc.F32, via_f16, [via_f16.size]), via_f16.view(np.float16).astype(np.float32))
    via_bf16 = orc.cast(orc.F32, orc.BF16, finite, [finite.size])
    numbers = ~np.isnan(finite)
    assert np.array_equal(via_bf16[numbers], bf16_rne_independent(words[numbers]))
    assert np.array_equal(orc.cast(orc.BF16, orc.F32, via_bf16, [via_bf16.size]).view(np.uint32), via_bf16.astype(np.uint32) << 16)
    halves = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(orc.cast(orc.F16, orc.BF16, halves, [halves.size]),
                          orc.from_f32(orc.BF16, orc.to_f32(orc.F16, halves)))
    assert np.array_equal(orc.cast(orc.BF16, orc.F16, halves, [halves.size]),
                          orc.from_f32(orc.F16, orc.to_f32(orc.BF16, halves)))
    # equal types keep the bytes (Copy), NaN payloads included, through any strides
    grid = rng.integers(0, 1 << 16, (6, 10), dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(orc.cast(orc.BF16, orc.BF16, grid, [6, 5], [20, 4]), grid[:, ::2])
    assert np.array_equal(orc.cast(orc.F32, orc.F32, words, [1000]).view(np.uint32), words[:1000])
