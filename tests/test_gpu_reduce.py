"""Parity of Reduce over any axes (through the C ABI) with the CPU oracle.

Bars: minimum and maximum are bit-exact (any NaN matches any NaN; the sign of a zero result
counts).  Sums and means may be taken in any order (include/hyle/compute/operation.h:314-318;
the reference's CUDA kernel adds thread-strided partial sums, reduction_kernel.cu:92-113), so
they are compared with the float64 value of the same reduction: 1e-5 relative plus the rounding
a different order can leave, 2e-7 * sum(|x|) per result (sum(|x|) / count for a mean); bf16 / f16
results are within one unit in the last place of the oracle unless inside that same bound.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, assert_bits_equal, assert_narrow_ulp, context, host_values, note, run, to_device, to_host

pytestmark = pytest.mark.gpu

RK = hc.ReductionKind
ORACLE_KIND = {RK.kSum: orc.SUM, RK.kMean: orc.MEAN, RK.kMinimum: orc.MIN, RK.kMaximum: orc.MAX}
F32ACC = hc.DataType.kFloat32


def route_of(operation, desc) -> str:
    return hc.prepare(context(), operation, desc).route_name()


def check(kind, tag, got, x_storage, dims, axes, byte_strides=None):
    """got: device result (storage representation).  x_storage: the input's bytes as stored."""
    oid = TYPES[tag][1]
    want = orc.reduce(ORACLE_KIND[kind], oid, x_storage, dims, axes, byte_strides)
    assert got.shape == want.shape, (got.shape, want.shape)
    got, want = np.atleast_1d(got), np.atleast_1d(want)
    if kind in (RK.kMinimum, RK.kMaximum):
        assert_bits_equal(got, want) if tag == "f32" else assert_narrow_ulp(got, want, tag, ulps=0)
        return
    # float64 value of the same reduction, from the oracle's own walk over f32 copies
    size = 4 if tag == "f32" else 2
    rank = len(dims)
    strides = byte_strides
    if strides is None:
        strides, step = [], size
        for d in reversed(dims):
            strides.insert(0, step)
            step *= d
    raw = np.ascontiguousarray(x_storage).view(np.uint8).reshape(-1)
    index = np.zeros(dims, np.int64)
    for a in range(rank):
        shape = [1] * rank
        shape[a] = dims[a]
        index = index + (np.arange(dims[a], dtype=np.int64) * strides[a]).reshape(shape)
    flat = index.reshape(-1)
    gathered = np.zeros((flat.size, size), np.uint8)
    for b in range(size):
        gathered[:, b] = raw[flat + b]
    values = gathered.reshape(-1).view(np.float32 if tag == "f32" else np.uint16).reshape(dims)
    x64 = (values if tag == "f32" else orc.to_f32(oid, values)).astype(np.float64)
    selected = tuple(range(rank)) if axes is None else tuple(a % rank for a in axes)
    count = int(np.prod([dims[a] for a in selected])) if selected else 1
    with np.errstate(invalid="ignore", over="ignore"):
        exact = np.sum(x64, axis=selected)
        spread = np.sum(np.abs(x64), axis=selected)
        if kind == RK.kMean:
            exact, spread = (exact / count, spread / count) if count else (np.full_like(exact, np.nan), spread)
    exact, spread = np.atleast_1d(exact), np.atleast_1d(spread)
    g = (got if tag == "f32" else orc.to_f32(oid, got)).astype(np.float64).reshape(exact.shape)
    got, want = got.reshape(exact.shape), want.reshape(exact.shape)
    nan = np.isnan(exact)
    assert np.array_equal(np.isnan(g), nan), "NaN positions differ"
    inf = np.isinf(exact) & ~nan
    assert np.array_equal(g[inf], exact[inf])
    ok = ~(nan | inf)
    bound = 1e-5 * np.abs(exact[ok]) + 2e-7 * spread[ok]
    if tag == "f32":
        assert np.all(np.abs(g[ok] - exact[ok]) <= bound + 1e-37)
    else:
        settled = np.zeros(g.shape, bool)
        settled[ok] = np.abs(g[ok] - exact[ok]) <= bound
        assert_narrow_ulp(np.where(settled | ~ok, want, got), want, tag)


def values_for(rng, dims, tag, plant=True):
    x = rng.normal(0, 2, dims).astype(np.float32)
    if plant and x.size > 16:
        flat = x.reshape(-1)
        flat[3] = np.nan
        flat[5], flat[6] = 0.0, -0.0
        flat[-2] = np.inf
    return host_values(x, tag)


CASES = [
    # dims, axes, expected route
    ([5, 7], [-1], "reduce-rows"),
    ([3, 5, 7], None, "reduce-rows"),
    ([6, 4096], [1], "reduce-rows"),
    ([2, 3, 1024], [1, 2], "reduce-rows"),
    ([3, 300000], [-1], "reduce-row-tiles"),
    ([1 << 20], None, "reduce-row-tiles"),
    ([1000, 64], [0], "reduce-columns"),
    ([4, 300, 96], [1], "reduce-columns"),
    ([100, 7], [0], "reduce-columns"),
    ([9, 1, 33, 5], [2], "reduce-columns"),
    ([70000, 8], [0], "reduce-column-segments"),
    ([2, 9000, 24], [1], "reduce-column-segments"),
    ([5000, 3], [0], "reduce-columns"),
    ([300000, 3], [0], "reduce-column-segments"),
    ([4, 5, 6], [0, 2], "reduce-strided"),
    ([3, 4, 5, 6], [1, 3], "reduce-strided"),
    ([17], [0], "reduce-rows"),
    ([4, 1, 6], [1], "reduce-columns"),
]


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("dims,axes,route", CASES, ids=[f"{'x'.join(map(str, d))}-{a}" for d, a, _ in CASES])
def test_reduce_every_kind_over_dense_inputs(dims, axes, route, tag):
    rng = np.random.default_rng(900 + len(dims) * 7 + (0 if axes is None else len(axes)))
    dtype = TYPES[tag][0]
    for kind in RK:
        x = values_for(rng, dims, tag, plant=kind in (RK.kMinimum, RK.kMaximum) or dims[0] % 2 == 1)
        operation = hc.Reduce(kind, hc.Axes.all() if axes is None else hc.Axes.from_(axes), accumulation_type=F32ACC)
        assert route_of(operation, hc.TensorDesc.dense(dtype, dims)) == route
        note(f"reduce {kind.name} {tag} {dims} axes {axes} ({route})")
        (out,) = run(operation, to_device(x, tag))
        check(kind, tag, to_host(out), x, dims, axes)
    note(f"reduce keep_dimensions {tag} {dims} axes {axes}")
    keep = hc.Reduce(RK.kMaximum, hc.Axes.all() if axes is None else hc.Axes.from_(axes), True, F32ACC)
    (kept,) = run(keep, to_device(x, tag))
    selected = range(len(dims)) if axes is None else [a % len(dims) for a in axes]
    assert list(kept.shape) == [1 if a in selected else d for a, d in enumerate(dims)]
    assert np.array_equal(to_host(kept).reshape(-1), to_host(out).reshape(-1), equal_nan=True) or tag != "f32"


def test_reduce_reference_known_answers_on_device():
    # tests/compute_provider_native/reduction_test.cc:46-128
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    for kind, want in ((RK.kSum, [6, 15]), (RK.kMean, [2, 5]), (RK.kMinimum, [1, 4]), (RK.kMaximum, [3, 6])):
        note(f"reduce known answers {kind.name}")
        (out,) = run(hc.Reduce(kind, hc.Axes.from_([1])), to_device(x, "f32"))
        assert to_host(out).tolist() == want
    x = np.arange(1, 9, dtype=np.float32).reshape(2, 2, 2)
    (out,) = run(hc.Reduce(RK.kSum, hc.Axes.from_([0, 2])), to_device(x, "f32"))
    assert to_host(out).tolist() == [14, 22]
    (out,) = run(hc.Reduce(RK.kSum, hc.Axes.from_([0, 2]), keep_dimensions=True), to_device(x, "f32"))
    assert list(out.shape) == [1, 2, 1] and to_host(out).reshape(-1).tolist() == [14, 22]
    # :167-181 the minimum of zeros of both signs is -0; the maximum is +0
    zeros = np.zeros(37, np.float32)
    zeros[1] = zeros[19] = -0.0
    (out,) = run(hc.Reduce(RK.kMinimum), to_device(zeros, "f32"))
    assert np.signbit(to_host(out))
    (out,) = run(hc.Reduce(RK.kMaximum), to_device(zeros, "f32"))
    assert not np.signbit(to_host(out)) and to_host(out) == 0


def test_reduce_unaligned_byte_strides_and_views():
    # tests/compute_provider_native/reduction_test.cc:130-165: strides {10, 4}, NaN, all axes
    raw = np.zeros(18 + 6, np.uint8)
    for offset, value in zip((0, 4, 10, 14), (0.0, -0.0, 3.0, np.nan)):
        raw[offset:offset + 4] = np.frombuffer(np.float32(value).tobytes(), np.uint8)
    desc = hc.TensorDesc.strided_bytes(hc.DataType.kFloat32, [2, 2], [10, 4])
    note("reduce f32 strides {10, 4} minimum over all axes")
    (out,) = run(hc.Reduce(RK.kMinimum), torch.from_numpy(raw).to(DEVICE), descs=[desc])
    assert np.isnan(to_host(out))
    rng = np.random.default_rng(950)
    for tag in ("f32", "bf16", "f16"):
        size = 4 if tag == "f32" else 2
        # rows 5 elements + 3 bytes apart, elements dense: a bytewise walk
        dims = [6, 40]
        values = values_for(rng, dims, tag)
        row_bytes = dims[1] * size + 3
        raw = np.zeros(dims[0] * row_bytes + 8, np.uint8)
        for r in range(dims[0]):
            raw[r * row_bytes:r * row_bytes + dims[1] * size] = values[r].view(np.uint8)
        desc = hc.TensorDesc.strided_bytes(TYPES[tag][0], dims, [row_bytes, size])
        for kind in RK:
            for axes in ([0], [1], None):
                note(f"reduce {kind.name} {tag} odd row stride axes {axes}")
                operation = hc.Reduce(kind, hc.Axes.all() if axes is None else hc.Axes.from_(axes), accumulation_type=F32ACC)
                (out,) = run(operation, torch.from_numpy(raw).to(DEVICE), descs=[desc])
                check(kind, tag, to_host(out), raw, dims, axes, [row_bytes, size])
        # torch views: a transposed and a stepped slice
        base = to_device(values_for(rng, [12, 10, 8], tag), tag)
        for view, axes in ((base.transpose(0, 2), [0]), (base[::2, 1:9, ::3], [1, 2]), (base.permute(1, 2, 0), [-1])):
            note(f"reduce sum {tag} view {tuple(view.shape)} strides {view.stride()} axes {axes}")
            (out,) = run(hc.Reduce(RK.kSum, hc.Axes.from_(axes), accumulation_type=F32ACC), view)
            dense = to_host(view.contiguous())
            check(RK.kSum, tag, to_host(out), dense, list(view.shape), axes)


def test_reduce_empty_extents_and_single_elements():
    # tests/compute_provider_native/reduction_test.cc:183-222
    for tag in ("f32", "bf16"):
        empty = torch.empty((2, 0), dtype=TYPES[tag][2], device=DEVICE)
        for kind, want in ((RK.kSum, 0.0), (RK.kMean, np.nan), (RK.kMinimum, np.inf), (RK.kMaximum, -np.inf)):
            note(f"reduce {kind.name} {tag} over an empty extent")
            (out,) = run(hc.Reduce(kind, hc.Axes.from_([1]), accumulation_type=F32ACC), empty)
            got = out.float().cpu().numpy()
            assert got.shape == (2,)
            assert np.all(np.isnan(got)) if np.isnan(want) else np.all(got == want)
        note(f"reduce {tag}: no output elements")
        (out,) = run(hc.Reduce(RK.kSum, hc.Axes.from_([1]), accumulation_type=F32ACC),
                     torch.empty((0, 5), dtype=TYPES[tag][2], device=DEVICE))
        assert list(out.shape) == [0]
    note("reduce: rank 0 and extent-1 axes")
    scalar = torch.tensor(3.5, device=DEVICE)
    (out,) = run(hc.Reduce(RK.kMean), scalar)
    assert out.shape == () and float(out) == 3.5
    x = to_device(np.arange(12, dtype=np.float32).reshape(3, 1, 4), "f32")
    (out,) = run(hc.Reduce(RK.kSum, hc.Axes.from_([1])), x)
    assert to_host(out).tolist() == np.arange(12, dtype=np.float32).reshape(3, 4).tolist()


def test_reduce_schema_and_admission():
    D, DT = hc.TensorDesc.dense, hc.DataType
    x = D(DT.kFloat32, [4, 5, 6])
    assert hc.infer_output_descriptions(hc.Reduce(), [x]) == [D(DT.kFloat32, [])]
    assert hc.infer_output_descriptions(hc.Reduce(RK.kSum, hc.Axes.from_([0, -1])), [x]) == [D(DT.kFloat32, [5])]
    assert hc.infer_output_descriptions(hc.Reduce(RK.kSum, hc.Axes.from_([0, -1]), True), [x]) == [D(DT.kFloat32, [1, 5, 1])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Reduce(RK.kSum, hc.Axes.from_([0, -3])), [x])
    assert err.value.is_invalid_argument()          # duplicate
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Reduce(RK.kSum, hc.Axes.from_([3])), [x])
    assert err.value.is_out_of_range()
    with pytest.raises(hc.StatusError) as err:
        hc.Axes.from_([])
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.Axes.from_([8])
    assert err.value.is_out_of_range()
    # narrow storage needs the f32 accumulation spelled out; integers are declined
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.Reduce(RK.kSum), D(DT.kBFloat16, [4, 8]))
    assert err.value.is_unimplemented()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.Reduce(RK.kSum), D(DT.kInt32, [4, 8]))
    assert err.value.is_unimplemented()
    # Reduce never aliases its input
    prepared = hc.prepare(context(), hc.Reduce(RK.kSum, hc.Axes.from_([1]), True), D(DT.kFloat32, [4, 1]))
    assert not prepared.alias_support(0, 0)


def test_reduce_benchmark_shapes():
    rng = np.random.default_rng(960)
    for tag, dims, axes in (("bf16", [8192, 2048], [-1]), ("bf16", [8192, 2048], [0]), ("f32", [4096, 4096], None)):
        x = host_values(rng.normal(0, 1, dims).astype(np.float32), tag)
        for kind in (RK.kSum, RK.kMaximum):
            note(f"reduce {kind.name} {tag} {dims} axes {axes}")
            operation = hc.Reduce(kind, hc.Axes.all() if axes is None else hc.Axes.from_(axes), accumulation_type=F32ACC)
            (out,) = run(operation, to_device(x, tag))
            check(kind, tag, to_host(out), x, dims, axes)
