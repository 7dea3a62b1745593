"""Parity of every Unary kind and of the GELU gates (through the C ABI) with the CPU oracle.

Bars: bit-exact for abs, neg, relu and sqrt; 1e-5 relative for the other f32 results (the
transcendental kinds go through different but equally accurate exp / log / tanh / erf routines;
results below the smallest normal f32 are compared absolutely); <= 1 unit in the last place for
bf16 / f16 outputs.  Where a formula cancels in f32 (1 + tanh(.) and 1 + erf(.) for negative
arguments, log near 1) the bar carries the absolute term that the cancellation leaves, as the
reference's own test does (tests/compute_provider_native/elementwise_test.cc:120-128:
3e-4 relative + 3e-6).
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import (DEVICE, TYPES, assert_bits_equal, assert_close_f32, assert_narrow_ulp, context, host_values,
                         note, run, to_device, to_host)

pytestmark = pytest.mark.gpu

UK = hc.UnaryKind
EXACT = {UK.kAbs, UK.kNeg, UK.kRelu, UK.kSqrt}
CANCELLING = {UK.kGelu, UK.kGeluTanh, UK.kLog}


def domain(kind, rng, count):
    x = np.concatenate([rng.normal(0, 3, count - 40), rng.uniform(-100, 100, 24),
                        [0.0, -0.0, 1.0, -1.0, 1e-30, -1e-30, 1e-42, 88.0, -88.0, 104.0, -104.0, 20.0, -20.0,
                         np.inf, -np.inf, np.nan]]).astype(np.float32)
    if kind in (UK.kLog, UK.kSqrt, UK.kRsqrt):
        x[:count - 40] = np.abs(x[:count - 40]) + np.float32(1e-3)
    return x


def unary_bar(kind, got, want, x, tag):
    if kind in EXACT:
        # bit-exact; a NaN matches a NaN whatever its sign and payload
        assert_bits_equal(got, want) if tag == "f32" else assert_narrow_ulp(got, want, tag, ulps=0)
    elif tag == "f32":
        if kind in CANCELLING:
            finite = np.isfinite(want) & np.isfinite(x)
            assert np.array_equal(np.isnan(got), np.isnan(want))
            assert np.array_equal(got[~finite & ~np.isnan(want)], want[~finite & ~np.isnan(want)])
            scale = np.abs(x[finite]).astype(np.float64) if kind != UK.kLog else np.ones(int(finite.sum()))
            err = np.abs(got[finite].astype(np.float64) - want[finite].astype(np.float64))
            assert np.all(err <= 1e-5 * np.abs(want[finite].astype(np.float64)) + 3e-7 * scale)
        else:
            assert_close_f32(got, want, rel=1e-5, abs_floor=1.2e-38)
    else:
        if kind in CANCELLING:
            oid = TYPES[tag][1]
            g, w = orc.to_f32(oid, got).astype(np.float64), orc.to_f32(oid, want).astype(np.float64)
            scale = np.abs(orc.to_f32(oid, x)).astype(np.float64) if kind != UK.kLog else 1.0
            with np.errstate(invalid="ignore"):
                settled = np.abs(g - w) <= 3e-7 * scale
            assert_narrow_ulp(np.where(settled, want, got), want, tag)
        else:
            assert_narrow_ulp(got, want, tag)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("kind", list(UK), ids=lambda k: k.name[1:])
def test_unary_every_kind_edge_counts_and_specials(kind, tag):
    oid = TYPES[tag][1]
    rng = np.random.default_rng(600 + int(kind))
    for count in (1, 7, 129, 4099, 1 << 18):
        x = host_values(domain(kind, rng, max(count, 41))[-count:] if count < 41 else domain(kind, rng, count), tag)
        note(f"unary {kind.name} {tag} {count} elements")
        (out,) = run(hc.Unary(kind), to_device(x, tag))
        unary_bar(kind, to_host(out), orc.unary(int(kind), oid, x), x, tag)
    note(f"unary {kind.name} {tag}: strided view and in place")
    base = to_device(host_values(domain(kind, rng, 6 * 80).reshape(6, 80), tag), tag)
    view = base[:, 8:72:2]
    (out,) = run(hc.Unary(kind), view)
    unary_bar(kind, to_host(out), orc.unary(int(kind), oid, to_host(view.contiguous())), to_host(view.contiguous()), tag)
    x = host_values(domain(kind, rng, 4096), tag)
    data = to_device(x, tag)
    run(hc.Unary(kind), data, outputs=[data])
    unary_bar(kind, to_host(data), orc.unary(int(kind), oid, x), x, tag)


def test_unary_reference_known_values():
    # tests/compute_provider_native/elementwise_test.cc:127-178: seven values, every kind
    values = np.array([-2.0, -0.0, 0.25, 0.5, 1.0, 2.0, 4.0], np.float32)
    for kind in UK:
        note(f"unary {kind.name}: the reference test's seven values")
        (out,) = run(hc.Unary(kind), to_device(values, "f32"))
        got, want = to_host(out).astype(np.float64), orc.unary(int(kind), orc.F32, values).astype(np.float64)
        for g, w in zip(got, want):
            if np.isnan(w):
                assert np.isnan(g)
            elif np.isinf(w):
                assert g == w
            else:
                assert abs(g - w) <= abs(w) * 3e-4 + 3e-6
    note("integer Unary passes the schema but is declined")
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.Unary(UK.kAbs), hc.TensorDesc.dense(hc.DataType.kInt32, [8]))
    assert err.value.is_unimplemented()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.Unary(UK.kExp), hc.TensorDesc.dense(hc.DataType.kInt32, [8]))
    assert err.value.is_invalid_argument()


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("activation", [hc.GatedActivationKind.kGelu, hc.GatedActivationKind.kGeluTanh],
                         ids=lambda a: a.name[1:])
def test_gated_gelu_separate_and_packed(activation, tag):
    oid = TYPES[tag][1]
    rng = np.random.default_rng(700 + int(activation))
    kind = UK.kGelu if activation == hc.GatedActivationKind.kGelu else UK.kGeluTanh
    for rows, hidden in ((1, 8), (3, 64), (5, 129), (4, 1000), (16, 6144)):
        gate = rng.normal(0, 2, (rows, hidden)).astype(np.float32)
        gate[0, :5] = [-np.inf, np.inf, np.nan, -0.0, -30.0][:min(5, hidden)]
        gate, up = host_values(gate, tag), host_values(rng.normal(0, 2, (rows, hidden)).astype(np.float32), tag)
        want = orc.gated(int(activation), oid, gate, up)
        # the gate's cancellation error scales with |gate * up|
        scale = np.abs(orc.to_f32(oid, gate) if tag != "f32" else gate) * np.abs(orc.to_f32(oid, up) if tag != "f32" else up)
        note(f"gated {activation.name} {tag} [{rows}, {hidden}] separate inputs")
        (out,) = run(hc.GatedActivation(activation, hc.GatedInputKind.kSeparate), to_device(gate, tag), to_device(up, tag))
        check_gated(to_host(out), want, scale, tag)
        note(f"gated {activation.name} {tag} [{rows}, {2 * hidden}] packed halves")
        packed = np.concatenate([gate, up], axis=1)
        (out,) = run(hc.GatedActivation(activation, hc.GatedInputKind.kPackedHalves), to_device(packed, tag))
        check_gated(to_host(out), want, scale, tag)
    assert kind in CANCELLING


def check_gated(got, want, scale, tag):
    if tag == "f32":
        finite = np.isfinite(want) & np.isfinite(scale)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~finite & ~np.isnan(want)], want[~finite & ~np.isnan(want)])
        err = np.abs(got[finite].astype(np.float64) - want[finite].astype(np.float64))
        assert np.all(err <= 1e-5 * np.abs(want[finite].astype(np.float64)) + 3e-7 * scale[finite])
    else:
        oid = TYPES[tag][1]
        g, w = orc.to_f32(oid, got).astype(np.float64), orc.to_f32(oid, want).astype(np.float64)
        with np.errstate(invalid="ignore"):
            settled = np.abs(g - w) <= 3e-7 * scale
        assert_narrow_ulp(np.where(settled, want, got), want, tag)
