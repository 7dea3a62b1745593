"""Parity of LayerNorm (through the C ABI) with the CPU oracle, and the equivalence the Qwen
graph's norm recipe relies on (cast -> RMSNorm -> cast equals one RMSNorm over narrow storage).

Bars: <= 1 unit in the last place for bf16/f16 outputs; for f32 outputs 1e-5 relative plus an
absolute floor of 2e-6 (normalised values are O(1); an element next to the row mean has no
significant digits left after the subtraction, so a purely relative bar is meaningless there).
Known answers first (tests/compute_provider_native/normalization_test.cc:69-170,
tests/simd/math_test.cc:1168-1231), then every route and parameter form over edge widths.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import (DEVICE, TYPES, assert_close_f32, assert_narrow_ulp, context, host_values, note, run,
                         to_device, to_host)

pytestmark = pytest.mark.gpu


def layer_bar(got, want, tag, bias=None):
    if tag == "f32":
        # the reference's mean is a running f32 sum, whose error bound grows with the row
        # length; beyond 4096 columns the floor grows with it (width / 4096)
        # and where fma(normalised * scale, bias) nearly cancels, the result carries the product's error
        width = want.shape[-1]
        floor = 2e-6 * max(1.0, width / 4096.0)
        if bias is not None:
            floor = floor + 1e-5 * float(np.abs(bias).max())
        assert_close_f32(got, want, rel=1e-5, abs_floor=floor)
    else:
        # one unit in the last place, except next to the row mean: there the subtraction leaves
        # an absolute error of the order of the f32 floor above, which is many units of a tiny
        # narrow value; those elements are held to that absolute floor instead
        oid = TYPES[tag][1]
        width = want.shape[-1]
        g, w = orc.to_f32(oid, got).astype(np.float64), orc.to_f32(oid, want).astype(np.float64)
        floor = 2e-6 * max(1.0, width / 4096.0)
        if bias is not None:
            # fma(normalised * scale, bias): where the two nearly cancel, the result carries the product's
            # error (the inverse deviation's: running against tree sums of `width` squares), not its own
            shift = bias if bias.dtype == np.float32 else orc.to_f32(oid, bias)   # f32 parameters, or the input's own type
            floor = floor + 1e-5 * max(1.0, width / 4096.0) * np.abs(shift.astype(np.float64))
        near_mean = np.abs(g - w) <= floor
        assert np.array_equal(np.isnan(g), np.isnan(w))
        assert_narrow_ulp(np.where(near_mean, want, got), want, tag)


def test_layer_norm_reference_known_answers():
    note("LayerNorm [2,3]: plain, scale only, affine (normalization_test.cc:69-127)")
    values = np.array([[1, 2, 3], [2, 4, 6]], np.float32)
    scale, bias = np.array([2, 3, 4], np.float32), np.array([10, 20, 30], np.float32)
    first = 1.0 / np.sqrt(2.0 / 3.0 + 1e-5)
    second = 2.0 / np.sqrt(8.0 / 3.0 + 1e-5)
    normalized = np.array([[-first, 0, first], [-second, 0, second]])
    op = hc.LayerNorm(epsilon=1e-5)
    x, s, b = to_device(values, "f32"), to_device(scale, "f32"), to_device(bias, "f32")
    (out,) = run(op, x)
    assert np.all(np.abs(to_host(out) - normalized) <= 2e-5)
    (out,) = run(op, x, s)
    assert np.all(np.abs(to_host(out) - normalized * scale) <= 2e-5)
    (out,) = run(op, x, s, b)
    assert np.all(np.abs(to_host(out) - (normalized * scale + bias)) <= 2e-5)
    note("LayerNorm in place over its input (normalization_test.cc:129-148)")
    prepared = hc.prepare(context(), op, hc.TensorDesc.dense(hc.DataType.kFloat32, [2, 3]))
    assert prepared.alias_support(0, 0)
    run(op, x, outputs=[x])
    assert np.all(np.abs(to_host(x) - normalized) <= 2e-5)
    note("LayerNorm of a constant row is zero (math_test.cc:1226-1231); empty last dimension is a no-op")
    (out,) = run(op, to_device(np.full((1, 17), 3.0, np.float32), "f32"))
    assert np.array_equal(to_host(out), np.zeros((1, 17), np.float32))
    empty = hc.prepare(context(), op, hc.TensorDesc.dense(hc.DataType.kFloat32, [4, 0]))
    assert empty.dispatch_count() == 0


@pytest.mark.parametrize("tag,param_tag", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16")])
def test_layer_norm_every_route_and_parameter_form(tag, param_tag):
    oid, pid = TYPES[tag][1], TYPES[param_tag][1]
    rng = np.random.default_rng(500)
    for rows, width in ((3, 1), (5, 8), (4, 24), (7, 127), (6, 128), (5, 129), (9, 512), (33, 1024), (17, 2048),
                        (5, 4096), (3, 9000), (2, 20000), (2, 70000)):
        x = host_values((rng.normal(0.4, 1, (rows, width)) * rng.uniform(0.1, 10, (rows, 1))).astype(np.float32), tag)
        scale = host_values(rng.normal(1, 0.1, width).astype(np.float32), param_tag)
        bias = host_values(rng.normal(0, 0.5, width).astype(np.float32), param_tag)
        dx, ds, db = to_device(x, tag), to_device(scale, param_tag), to_device(bias, param_tag)
        for eps in (1e-5, 1e-6):
            op = hc.LayerNorm(epsilon=eps)
            note(f"LayerNorm {tag} (params {param_tag}) [{rows}, {width}] eps {eps}: plain, scale, affine")
            if tag == param_tag:
                (out,) = run(op, dx)
                layer_bar(to_host(out), orc.layer_norm(oid, x, None, None, eps), tag)
            (out,) = run(op, dx, ds)
            layer_bar(to_host(out), orc.layer_norm(oid, x, scale, None, eps, param_type=pid), tag)
            (out,) = run(op, dx, ds, db)
            layer_bar(to_host(out), orc.layer_norm(oid, x, scale, bias, eps, param_type=pid), tag)
    note(f"LayerNorm {tag}: misaligned base pointer takes the element route")
    x = host_values(rng.normal(0, 2, (4, 1001)).astype(np.float32), tag)
    flat = to_device(np.concatenate([x.reshape(-1)[:1], x.reshape(-1)]), tag)
    view = flat[1:].view(4, 1001)
    (out,) = run(hc.LayerNorm(), view)
    layer_bar(to_host(out), orc.layer_norm(oid, x, None, None, 1e-5), tag)


def test_layer_norm_schema_errors_and_declines():
    ctx = context()
    D, DT = hc.TensorDesc.dense, hc.DataType
    with pytest.raises(hc.StatusError) as err:  # scale must match the last dimension
        hc.prepare(ctx, hc.LayerNorm(), D(DT.kFloat32, [4, 64]), D(DT.kFloat32, [32]))
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.LayerNorm(), D(DT.kFloat32, [4, 64]), D(DT.kFloat32, [64]), D(DT.kFloat32, [63]))
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.LayerNorm(epsilon=-1.0), D(DT.kFloat32, [4, 64]))
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:  # half accumulation is not served
        hc.prepare(ctx, hc.LayerNorm(accumulation_type=DT.kFloat16), D(DT.kFloat16, [4, 64]))
    assert err.value.is_unimplemented()
    with pytest.raises(hc.StatusError) as err:  # strided input: left to another provider
        hc.prepare(ctx, hc.LayerNorm(), hc.TensorDesc.strided_bytes(DT.kFloat32, [4, 64], [512, 4]))
    assert err.value.is_unimplemented()


@pytest.mark.parametrize("tag,param_tag", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16")])
def test_layer_norm_launches_that_cover_the_tensor_exactly(tag, param_tag):
    """64 rows of every width that fills a launch shape's lanes with whole vectors (sub-wave groups of 8 to
    32 lanes, then 64, 128 or 256 lanes with up to eight vectors each): the kernels that mask nothing (the
    other test's row counts and widths leave lanes or rows over), in all three parameter forms; 4096 and
    8192 vectors are past them."""
    oid, pid = TYPES[tag][1], TYPES[param_tag][1]
    rng = np.random.default_rng(502)
    per_vector = 4 if tag == "f32" else 8
    for vectors in (8, 16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 576, 640, 768, 896, 1024, 1280, 1536, 1792, 2048, 4096, 8192):
        rows, width = 64, vectors * per_vector
        x = host_values((rng.normal(-0.3, 1, (rows, width)) * rng.uniform(0.1, 10, (rows, 1))).astype(np.float32), tag)
        scale = host_values(rng.normal(1, 0.1, width).astype(np.float32), param_tag)
        bias = host_values(rng.normal(0, 0.5, width).astype(np.float32), param_tag)
        dx, ds, db = to_device(x, tag), to_device(scale, param_tag), to_device(bias, param_tag)
        op = hc.LayerNorm(epsilon=1e-6)
        note(f"LayerNorm {tag} (params {param_tag}) [{rows}, {width}] exact cover: plain, scale, affine")
        if tag == param_tag:
            (out,) = run(op, dx)
            layer_bar(to_host(out), orc.layer_norm(oid, x, None, None, 1e-6), tag)
        (out,) = run(op, dx, ds)
        layer_bar(to_host(out), orc.layer_norm(oid, x, scale, None, 1e-6, param_type=pid), tag)
        (out,) = run(op, dx, ds, db)
        layer_bar(to_host(out), orc.layer_norm(oid, x, scale, bias, 1e-6, param_type=pid), tag, bias=bias)


def test_layer_norm_bench_shape_and_shift_invariance():
    rng = np.random.default_rng(501)
    x = (rng.normal(0, 1, (8192, 2048)) * rng.uniform(0.1, 10, (8192, 1))).astype(np.float32)
    xb = orc.from_f32(orc.BF16, x)
    scale = orc.from_f32(orc.BF16, rng.normal(1, 0.1, 2048).astype(np.float32))
    bias = orc.from_f32(orc.BF16, rng.normal(0, 0.5, 2048).astype(np.float32))
    note("LayerNorm bf16 [8192, 2048] affine, full comparison")
    (out,) = run(hc.LayerNorm(epsilon=1e-6), to_device(xb, "bf16"), to_device(scale, "bf16"), to_device(bias, "bf16"))
    layer_bar(to_host(out), orc.layer_norm(orc.BF16, xb, scale, bias, 1e-6), "bf16")
    note("LayerNorm f32: rows have mean 0 and variance 1 - eps/(var+eps) (size-independent property)")
    (plain,) = run(hc.LayerNorm(epsilon=1e-6), to_device(x, "f32"))
    mean = plain.mean(dim=-1, dtype=torch.float64)
    second = (plain.double() ** 2).mean(dim=-1)
    assert float(mean.abs().max()) <= 1e-5
    var = torch.from_numpy(x).double().var(dim=-1, unbiased=False).to(DEVICE)
    assert float((second - var / (var + 1e-6)).abs().max()) <= 1e-4


def test_cast_norm_cast_equals_one_norm_over_narrow_storage():
    # engine/models/qwen35/graph_builder.cc:492-499: norm = cast(RmsNorm(cast(x, f32), f32 scale), type).
    # The f32 RMSNorm rounds (x * inv) * w to f32 and the cast rounds that to bf16; RMSNorm over bf16
    # storage with f32 parameters forms the same f32 product and rounds it once to bf16.  Only the
    # order of the sum of squares differs between the two launches.
    rng = np.random.default_rng(502)
    x = orc.from_f32(orc.BF16, (rng.normal(0, 1, (4096, 2048)) * rng.uniform(0.1, 10, (4096, 1))).astype(np.float32))
    w = rng.normal(1, 0.1, 2048).astype(np.float32)
    dx, dw = to_device(x, "bf16"), to_device(w, "f32")
    note("three launches: Cast bf16 -> f32, RmsNorm f32, Cast f32 -> bf16")
    (wide,) = run(hc.Cast(hc.DataType.kFloat32), dx)
    (normed,) = run(hc.RmsNorm(epsilon=1e-6), wide, dw)
    (chain,) = run(hc.Cast(hc.DataType.kBFloat16), normed)
    note("one launch: RmsNorm over bf16 storage with f32 parameters")
    (fused,) = run(hc.RmsNorm(epsilon=1e-6), dx, dw)
    differing = assert_narrow_ulp(to_host(fused), to_host(chain), "bf16")
    assert differing <= x.size // 1000  # the summation orders agree on all but a few roundings
    assert_narrow_ulp(to_host(fused), orc.rms_norm(orc.BF16, x, w, 1e-6, weight_type=orc.F32), "bf16")
