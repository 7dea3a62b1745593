"""The oracle's restatement of MatMul over a GGUF weight as the reference's ggml CPU route computes
it (8-bit activation blocks, integer block dot products), pinned without the GPU: the activation
codecs against array-wise restatements of the forms the reference's tests hold
(tests/compute_models/dspark_original_shared_reference.h:147-185 for Q8_0,
tests/compute_models/qwen27_original_nextn_reference.h:144-167 for Q8_K), hand-worked blocks, and
the centre against a float64 product of independently decoded weights."""
from __future__ import annotations

import numpy as np

from oracle import lib as orc

from k_quant_support import random_rows


def rn(value64):
    return np.asarray(value64, np.float64).astype(np.float32)


def q8_0_array_form(x):
    blocks = np.asarray(x, np.float32).reshape(-1, 32)
    maximum = np.abs(blocks).max(axis=1)
    live = maximum > 0
    safe = np.where(live, maximum, 1).astype(np.float64)
    divisor = rn(safe / 127.0)
    scale = np.where(live, divisor.astype(np.float16).astype(np.float32), 0).astype(np.float32)
    reciprocal = rn(127.0 / safe)
    scaled = rn(blocks.astype(np.float64) * reciprocal[:, None].astype(np.float64))
    codes = np.where(live[:, None], np.rint(scaled.astype(np.float64)), 0).astype(np.int8)
    return codes.reshape(-1), scale


def q8_k_array_form(x):
    blocks = np.asarray(x, np.float32).reshape(-1, 256)
    first = np.argmax(np.abs(blocks), axis=1)          # argmax returns the first of equal magnitudes
    maximum = blocks[np.arange(len(blocks)), first]
    live = maximum != 0
    safe = np.where(live, maximum, 1).astype(np.float64)
    inverse = rn(-127.0 / safe)
    stored = np.where(live, rn(1.0 / inverse.astype(np.float64)), 0).astype(np.float32)
    scaled = rn(blocks.astype(np.float64) * inverse[:, None].astype(np.float64))
    codes = np.where(live[:, None], np.minimum(127, np.rint(scaled.astype(np.float64))), 0).astype(np.int8)
    return codes.reshape(-1), stored


def activations(rng, k):
    x = rng.normal(0, 1.5, k).astype(np.float32)
    x[rng.random(k) < 0.05] = 0.0
    return x


def test_q8_0_activation_blocks_follow_the_reference_tests_form():
    rng = np.random.default_rng(1500)
    x = activations(rng, 32 * 40)
    x[64:96] = 0.0                                     # an all-zero block: scale 0, codes 0
    x[96:128] = np.float32(1.0)                        # every value the maximum
    x[128] = -7.5                                      # a negative maximum
    codes, scales = orc.quantize_q8_0(x)
    want_codes, want_scales = q8_0_array_form(x)
    assert np.array_equal(codes, want_codes) and np.array_equal(scales.view(np.uint32), want_scales.view(np.uint32))
    assert scales[2] == 0 and not codes[64:96].any()
    assert np.all(codes[96:128] == 127) and scales[3] == np.float32(np.float16(np.float32(1.0) / np.float32(127.0)))
    assert codes[128] == -127
    assert np.array_equal(scales, scales.astype(np.float16).astype(np.float32))      # an f16 value
    # each value is reproduced to half a step (plus the f16 rounding of the stored scale)
    back = np.repeat(scales, 32).astype(np.float64) * codes
    step = np.repeat(scales, 32).astype(np.float64)
    assert np.all(np.abs(back - x) <= 0.5 * step * (1 + 1e-6) + np.abs(x) * 2.0 ** -11)


def test_q8_k_activation_blocks_follow_the_reference_tests_form():
    rng = np.random.default_rng(1501)
    x = activations(rng, 256 * 12)
    x[256:512] = 0.0
    x[512], x[513] = 3.25, -3.25                       # equal magnitudes: the first one's sign decides
    x[514:768] *= 0.1
    x[768], x[769] = -3.25, 3.25
    x[770:1024] *= 0.1
    codes, scales = orc.quantize_q8_k(x)
    want_codes, want_scales = q8_k_array_form(x)
    assert np.array_equal(codes, want_codes) and np.array_equal(scales.view(np.uint32), want_scales.view(np.uint32))
    assert scales[1] == 0 and not codes[256:512].any()
    assert codes[512] == -127 and codes[513] == 127 and scales[2] < 0
    assert codes[768] == -127 and codes[769] == 127 and scales[3] > 0
    back = np.repeat(scales, 256).astype(np.float64) * codes
    step = np.abs(np.repeat(scales, 256).astype(np.float64))
    assert np.all(np.abs(back - x) <= 0.5 * step * (1 + 1e-6))


def test_hand_worked_q8_0_block():
    block = np.zeros(34, np.uint8)
    block[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    block[2:] = np.arange(1, 33, dtype=np.int8).view(np.uint8)
    x = np.ones(32, np.float32)
    centre, bound = orc.gguf_matvec_q8(orc.Q8_0, block[None, :], 1, 32, x)
    a_scale = float(np.float32(np.float16(np.float32(1.0) / np.float32(127.0))))
    assert centre[0, 0] == 0.5 * a_scale * 127 * 528   # exact in double
    assert 0 < bound[0, 0] < 1e-4 * abs(centre[0, 0])


def independent_weights(kind, raw, rows, k):
    """float64 weights of random raw rows, decoded through the checked f32 decoders (each value
    is within one f32 rounding of the exact product of its fields)."""
    if kind == orc.Q8_0:
        return orc.q8_0_dequant_f32(raw, rows, k).astype(np.float64)
    return orc.k_quant_dequant(kind, raw, rows, k)[0].astype(np.float64)


def test_centre_is_the_product_with_the_dequantised_activations_and_the_bound_has_its_scale():
    rng = np.random.default_rng(1502)
    k, rows, m = 2048, 9, 3
    x = np.stack([activations(rng, k) for _ in range(m)])
    for kind, tag in ((orc.Q4_K, "q4_k"), (orc.Q6_K, "q6_k"), (orc.Q8_0, None)):
        if tag is None:
            raw = rng.integers(0, 256, (rows, k // 32, 34), dtype=np.uint8)
            raw[:, :, 1] &= 0x3B
            raw = raw.reshape(rows, -1)
        else:
            raw, _ = random_rows(tag, rng, rows, k)
        weights = independent_weights(kind, raw, rows, k)
        centre, bound = orc.gguf_matvec_q8(kind, raw, rows, k, x)
        for i in range(m):
            if kind == orc.Q8_0:
                codes, scales = orc.quantize_q8_0(x[i])
                a = np.repeat(scales, 32).astype(np.float64) * codes
            else:
                codes, scales = orc.quantize_q8_k(x[i])
                a = np.repeat(scales, 256).astype(np.float64) * codes
            want = weights @ a
            size = np.abs(weights) @ np.abs(a)
            assert np.all(np.abs(centre[i] - want) <= 1e-6 * size)
            # the bound: (k / 4 + 65) f32 roundings of the summed magnitudes.  For Q4_K the two
            # components d * sc * q and dmin * m are bounded apart, so the sum of their
            # magnitudes exceeds the magnitude of the decoded weights.
            roundings = (k / 4 + 65) * 2.0 ** -24
            assert np.all(bound[i] >= roundings * size * (1 - 1e-3))
            if kind != orc.Q4_K:
                assert np.all(bound[i] <= roundings * size * 1.01 + 1e-12)
            # and the quantised product is close to the exact one: half a step per activation
            exact = weights @ x[i].astype(np.float64)
            step = np.repeat(np.abs(scales), 32 if kind == orc.Q8_0 else 256).astype(np.float64)
            slack = np.abs(weights) @ (0.5 * step * (1 + 1e-6) + np.abs(x[i]) * 2.0 ** -11)
            assert np.all(np.abs(centre[i] - exact) <= slack)
