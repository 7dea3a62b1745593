"""Parity of LogSoftmax (through the C ABI) with the CPU oracle.

Bars: f32 within 4e-6 relative + 2e-7 absolute of the oracle, the reference's own bound for this
operator (tests/compute_provider_cuda/tensor_test.cc:75-84); bf16 / f16 within one unit in the
last place; -inf (masked columns) and NaN (undefined rows) in the same places.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, assert_narrow_ulp, context, host_values, note, run, to_device, to_host

pytestmark = pytest.mark.gpu

LOG = hc.SoftmaxKind.kLogSoftmax


def log_bar(got, want, tag):
    if tag != "f32":
        assert_narrow_ulp(got, want, tag)
        return
    assert got.shape == want.shape
    assert np.array_equal(np.isnan(got), np.isnan(want)), "NaN positions differ"
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]), "masked columns differ"
    ok = ~(np.isnan(want) | inf)
    g, w = got[ok].astype(np.float64), want[ok].astype(np.float64)
    assert np.all(np.abs(g - w) <= np.abs(w) * 4e-6 + 2e-7)


def test_log_softmax_reference_known_answers_and_non_trailing_axis():
    # tests/compute_provider_native/transformer_test.cc:303-337: axis 1 of [1, 3, 2]
    values = np.array([1, 10, 2, 20, 3, 30], np.float32).reshape(1, 3, 2)
    note("log-softmax over axis 1 of [1, 3, 2]")
    (out,) = run(hc.Softmax(axis=1, kind=LOG), to_device(values, "f32"))
    s0 = 3.0 + np.log(np.exp(-2.0) + np.exp(-1.0) + 1.0)
    s1 = 30.0 + np.log(np.exp(-20.0) + np.exp(-10.0) + 1.0)
    want = np.array([1 - s0, 10 - s1, 2 - s0, 20 - s1, 3 - s0, 30 - s1]).reshape(1, 3, 2)
    got = to_host(out).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 4e-6 + 2e-7)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_log_softmax_keeps_near_one_tails_and_counts_equal_maxima(tag):
    # tests/compute_provider_cuda/tensor_test.cc:1168-1199
    oid = TYPES[tag][1]
    for width in (129, 8193, 4096):
        x = np.full((3, width), -20.0, np.float32)
        x[0, width - 1] = 0
        x[1, 0] = x[1, width - 1] = 0
        x[2, :] = 0
        stored = host_values(x, tag)
        note(f"log-softmax tails {tag} width {width}, in place")
        data = to_device(stored, tag)
        run(hc.Softmax(kind=LOG), data, outputs=[data])
        got = to_host(data)
        log_bar(got, orc.softmax(oid, stored, log=True), tag)
        wide = (got if tag == "f32" else orc.to_f32(oid, got)).astype(np.float64)
        for row, maxima in ((0, 1), (1, 2), (2, width)):
            partition = np.log(maxima) + np.log1p((width - maxima) * np.exp(-20.0) / maxima)
            want = x[row].astype(np.float64) - partition
            if tag == "f32":
                assert np.all(np.abs(wide[row] - want) <= np.abs(want) * 4e-6 + 2e-7)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_log_softmax_widths_masks_every_route(tag):
    oid = TYPES[tag][1]
    rng = np.random.default_rng(1206)
    for heads, q, width in ((2, 3, 8), (1, 5, 24), (2, 8, 136), (2, 16, 512), (2, 8, 4096), (1, 4, 9000),
                            (1, 2, 70000), (2, 3, 129)):
        x = host_values(rng.normal(0, 3, (heads, q, width)).astype(np.float32), tag)
        keep = (rng.random((q, width)) < 0.7).astype(np.uint8)
        keep[:, 0] = 1
        if q > 2:
            keep[2, :] = 0  # a fully masked row -> NaN for every head
        note(f"log-softmax {tag} {heads}x{q}x{width} no mask")
        (out,) = run(hc.Softmax(kind=LOG), to_device(x, tag))
        log_bar(to_host(out), orc.softmax(oid, x, log=True), tag)
        note(f"log-softmax {tag} {heads}x{q}x{width} Bool mask broadcast over heads, scale 0.125")
        dmask = torch.from_numpy(keep).to(DEVICE).view(torch.bool)
        (out,) = run(hc.Softmax(scale=0.125, kind=LOG, mask=hc.MaskKind.kBoolean), to_device(x, tag), dmask)
        log_bar(to_host(out), orc.softmax(oid, x, scale=0.125, mask_kind=orc.MASK_BOOLEAN, mask=keep, log=True), tag)
        note(f"log-softmax {tag} {heads}x{q}x{width} additive mask [heads,1,width]")
        add = host_values(np.where(rng.random((heads, 1, width)) < 0.2, -np.inf, rng.normal(0, 1, (heads, 1, width))
                                   ).astype(np.float32), tag)
        add[..., 0] = 0
        (out,) = run(hc.Softmax(kind=LOG, mask=hc.MaskKind.kAdditive), to_device(x, tag), to_device(add, tag))
        log_bar(to_host(out), orc.softmax(oid, x, mask_kind=orc.MASK_ADDITIVE, mask=add, log=True), tag)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_log_softmax_unmasked_launches_that_cover_the_tensor_exactly(tag):
    """The logarithmic form over the same exact launch shapes as the softmax test: 32 unmasked rows of
    every width with a shape of its own, undefined rows (NaN, +inf, only -inf) and -inf elements (-inf out)."""
    oid = TYPES[tag][1]
    rng = np.random.default_rng(1207)
    per_vector = 4 if tag == "f32" else 8
    for vectors in (16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1280, 1536, 1792, 2048):
        rows, width = 32, vectors * per_vector
        values = rng.normal(0, 3, (rows, width)).astype(np.float32)
        values[3, 5] = np.nan
        values[4, width - 1] = np.inf
        values[5, :] = -np.inf
        values[6, ::3] = -np.inf
        values[7, 1::2] = values[7, 0]            # many equal maxima or equal values
        x = host_values(values, tag)
        note(f"log-softmax {tag} [{rows}, {width}] unmasked")
        (out,) = run(hc.Softmax(kind=LOG), to_device(x, tag))
        log_bar(to_host(out), orc.softmax(oid, x, log=True), tag)


def test_log_softmax_other_axes_views_and_undefined_rows():
    rng = np.random.default_rng(1207)
    for tag in ("f32", "bf16"):
        oid = TYPES[tag][1]
        x = host_values(rng.normal(0, 2, (4, 129, 3)).astype(np.float32), tag)
        for axis in (0, 1):
            note(f"log-softmax {tag} axis {axis} of [4, 129, 3]")
            (out,) = run(hc.Softmax(axis=axis, kind=LOG), to_device(x, tag))
            moved = np.ascontiguousarray(np.moveaxis(x, axis, -1))
            want = np.moveaxis(orc.softmax(oid, moved, log=True), -1, axis)
            log_bar(to_host(out), np.ascontiguousarray(want), tag)
        note(f"log-softmax {tag} strided view")
        base = to_device(x, tag)
        view = base[::2, 5:100, :].transpose(1, 2)
        (out,) = run(hc.Softmax(kind=LOG), view)
        log_bar(to_host(out), orc.softmax(oid, to_host(view.contiguous()), log=True), tag)
    inf = np.inf
    rows = np.array([[0.0, -inf, -1.0, -inf], [0.0, np.nan, -1.0, 2.0], [0.0, inf, -1.0, 2.0], [-inf] * 4], np.float32)
    note("log-softmax masked / undefined rows")
    (out,) = run(hc.Softmax(kind=LOG), to_device(rows, "f32"))
    got = to_host(out)
    log_bar(got, orc.softmax(orc.F32, rows, log=True), "f32")
    assert np.isneginf(got[0, 1]) and np.isneginf(got[0, 3]) and np.isnan(got[1:]).all()


def test_log_softmax_against_the_scalar_floor_golden_rows():
    """The floor's own outputs (src/simd/math/activations.cc:320-336, committed as data) at the
    reference's bound for this operator."""
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "scalar_floor_vectors.npz"))
    cases = [(gold[f"log_softmax_x_{n}"], gold[f"log_softmax_y_{n}"]) for n in (1, 7, 8, 9, 257, 4096)]
    cases.append((gold["log_softmax_x_masked"], gold["log_softmax_y_masked_words"].view(np.float32)))
    for x, want in cases:
        note(f"log-softmax floor golden row n={x.size}")
        (out,) = run(hc.Softmax(kind=LOG), to_device(x[None, :], "f32"))
        log_bar(to_host(out)[0], want, "f32")
