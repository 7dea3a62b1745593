"""Parity of TopK(count = k) (through the C ABI) with the CPU oracle: bit-exact values (copies of
the source bits) and indices, in the reference's order (numbers before NaNs, best first, equal
numbers and NaNs by index; tests/compute_route_vulkan/topk_test_support.h:62-76)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, context, host_values, note, run, to_device, to_host

pytestmark = pytest.mark.gpu


def tied_values(rng, dims, tag):
    """Few distinct values (ties everywhere), NaNs, zeros of both signs, infinities."""
    x = (rng.integers(-40, 41, dims) / 8).astype(np.float32)
    flat = x.reshape(-1)
    n = flat.size
    flat[rng.integers(0, n, max(1, n // 11))] = np.nan
    flat[rng.integers(0, n, max(1, n // 13))] = -0.0
    flat[rng.integers(0, n, max(1, n // 17))] = 0.0
    flat[rng.integers(0, n, max(1, n // 50))] = np.inf
    flat[rng.integers(0, n, max(1, n // 50))] = -np.inf
    return host_values(x, tag)


def check(tag, stored, dims, count, axis, largest, outputs, byte_strides=None):
    values, indices = outputs
    want_values, want_indices = orc.topk(TYPES[tag][1], stored, dims, count, axis, largest, byte_strides)
    got_values, got_indices = to_host(values), to_host(indices)
    assert got_indices.shape == want_indices.shape and got_indices.dtype == np.int32
    assert np.array_equal(got_indices, want_indices)
    bits = np.uint32 if tag == "f32" else np.uint16
    assert np.array_equal(got_values.view(bits), want_values.view(bits))


CASES = [
    # dims, axis, counts
    ([5, 37], -1, (1, 2, 18, 37)),
    ([3, 2048], -1, (1, 7, 64, 1024)),
    ([4, 2049], -1, (2, 33)),
    ([2, 5000], -1, (5, 512)),
    ([6, 9, 16], 1, (1, 4, 9)),
    ([50, 3, 4], 0, (1, 3, 50)),
    ([300], 0, (1, 10, 300)),
    ([2, 3, 40, 5], 2, (8,)),
    ([1, 70001], -1, (3, 256, 1000)),
    ([2, 300000], -1, (1, 100)),
]


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("dims,axis,counts", CASES, ids=[f"{'x'.join(map(str, d))}-axis{a}" for d, a, _ in CASES])
def test_topk_dense_inputs_both_directions(dims, axis, counts, tag):
    rng = np.random.default_rng(1100 + len(dims) + dims[0])
    stored = tied_values(rng, dims, tag)
    for count in counts:
        for largest in (True, False):
            note(f"topk {tag} {dims} axis {axis} count {count} largest {largest}")
            outputs = run(hc.TopK(count=count, axis=axis, largest=largest), to_device(stored, tag))
            check(tag, stored, dims, count, axis, largest, outputs)


def test_topk_reference_special_rows():
    # tests/graph_route_cuda/topk_test.cc:458-476, also with count > 1
    width = 8193
    rows = []
    bits = np.full(width, 0xFF800000, np.uint32)
    bits[0], bits[1], bits[2] = 0x7FC12345, 0x80000000, 0
    rows.append(bits)
    rows.append((0x7FC03000 + np.arange(width)).astype(np.uint32))
    bits = np.full(width, 0xBF800000, np.uint32)
    bits[5] = bits[width - 1] = 0x40A00000
    rows.append(bits)
    x = np.stack(rows).view(np.float32)
    for count, expected in ((1, [[1], [0], [5]]), (3, [[1, 2, 3], [0, 1, 2], [5, width - 1, 0]])):
        note(f"topk special rows count {count}")
        values, indices = run(hc.TopK(count=count), to_device(x, "f32"))
        assert to_host(indices).tolist() == expected
        check("f32", x, [3, width], count, -1, True, (values, indices))


def test_topk_views_and_unaligned_strides():
    rng = np.random.default_rng(1150)
    for tag in ("f32", "bf16"):
        base = to_device(tied_values(rng, [12, 40, 6], tag), tag)
        for view, axis, count in ((base.transpose(0, 2), 1, 5), (base[::2, 3:35, ::2], 1, 9), (base.permute(2, 0, 1), -1, 40)):
            note(f"topk {tag} view {tuple(view.shape)} strides {view.stride()} axis {axis} count {count}")
            outputs = run(hc.TopK(count=count, axis=axis), view)
            check(tag, to_host(view.contiguous()), list(view.shape), count, axis, True, outputs)
        size = 4 if tag == "f32" else 2
        dims = [5, 300]
        values = tied_values(rng, dims, tag)
        row_bytes = dims[1] * size + 3                    # rows start at odd addresses
        raw = np.zeros(dims[0] * row_bytes + 8, np.uint8)
        for r in range(dims[0]):
            raw[r * row_bytes:r * row_bytes + dims[1] * size] = values[r].view(np.uint8)
        desc = hc.TensorDesc.strided_bytes(TYPES[tag][0], dims, [row_bytes, size])
        for axis, count in ((1, 17), (0, 2)):
            note(f"topk {tag} odd row stride axis {axis} count {count}")
            outputs = run(hc.TopK(count=count, axis=axis, largest=False), torch.from_numpy(raw).to(DEVICE), descs=[desc])
            check(tag, raw, dims, count, axis, False, outputs, [row_bytes, size])


def test_topk_when_the_first_bound_admits_every_key():
    """One thread of a block holds only hopeless values, so the bound taken from the per-thread
    maxima lets (nearly) every key through and the block has to find the exact k-th key."""
    rng = np.random.default_rng(1155)
    for tag, group in (("f32", 4), ("bf16", 8), ("f32", 1)):
        width = 20000 if group > 1 else 19999          # the odd width takes the element-wise loads
        x = rng.normal(0, 1, (3, width)).astype(np.float32)
        columns = np.arange(width)
        x[:, (columns // group) % 256 == 0] = -1000.0 - rng.random(int(((columns // group) % 256 == 0).sum()), dtype=np.float32)
        stored = host_values(x, tag)
        for count in (256, 200):
            for largest in (True, False):
                note(f"topk exact-search path {tag} width {width} count {count} largest {largest}")
                data = stored if largest else host_values(-x, tag)
                outputs = run(hc.TopK(count=count, largest=largest), to_device(data, tag))
                check(tag, data, [3, width], count, -1, largest, outputs)


def test_topk_mostly_distinct_values_take_the_float_bound():
    """Unordered, mostly distinct values: a tile's bound comes from the threads' float maxima and
    only the few elements that reach it become keys; the lists of the tiles meet in the ranking
    dispatch.  Winners that are zeros of either sign or infinities, NaNs among the losers, rows
    whose last tile is short, more lists than one wave can sample, and two ranking stages."""
    rng = np.random.default_rng(1158)
    shapes = (([4, 151936], (64, 8, 256)),      # 19 tiles; count 256 merges in two stages
              ([3, 20000], (100, 64)),           # 3 tiles, the last one short
              ([2, 600000], (4, 33)),            # 74 tiles: more lists than one wave samples
              ([5, 8192], (64,)),                # exactly one tile: the select dispatch writes the outputs
              ([2, 8200], (17,)))                # a last tile of 8 elements, fewer than count
    for tag in ("f32", "bf16", "f16"):
        for dims, counts in shapes:
            base = rng.normal(0, 2, dims).astype(np.float32)
            for largest in (True, False):
                sign = -1.0 if largest else 1.0
                x = base.copy()
                x[0] = sign * (np.abs(x[0]) + 1.0)                       # zeros are the best values of row 0
                spots = rng.choice(dims[1], 24, replace=False)
                x[0, spots[:12]] = 0.0
                x[0, spots[12:]] = -0.0
                x[1, rng.choice(dims[1], dims[1] // 50, replace=False)] = np.nan
                x[1, rng.choice(dims[1], 5, replace=False)] = -sign * np.inf
                x[-1, rng.choice(dims[1], 3, replace=False)] = sign * np.inf
                stored = host_values(x, tag)
                device = to_device(stored, tag)
                for count in counts:
                    note(f"topk float-bound path {tag} {dims} count {count} largest {largest}")
                    outputs = run(hc.TopK(count=count, largest=largest), device)
                    check(tag, stored, dims, count, -1, largest, outputs)


def test_topk_vocabulary_shape_count_64():
    rng = np.random.default_rng(1160)
    x = rng.normal(0, 3, (64, 151936)).astype(np.float32)
    x[3, 100] = x[3, 150000] = 50.0
    x[5, ::7] = np.nan
    note("topk f32 [64, 151936] count 64")
    outputs = run(hc.TopK(count=64), to_device(x, "f32"))
    check("f32", x, [64, 151936], 64, -1, True, outputs)


def test_topk_schema_and_admission():
    D, DT = hc.TensorDesc.dense, hc.DataType
    x = D(DT.kFloat32, [4, 5000])
    values, indices = hc.infer_output_descriptions(hc.TopK(count=7, axis=0 - 1), [x])
    assert values == D(DT.kFloat32, [4, 7]) and indices == D(DT.kInt32, [4, 7])
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.TopK(count=5001), [x])
    assert err.value.is_out_of_range()
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(context(), hc.TopK(count=2), D(DT.kUInt8, [4, 50]))
    assert err.value.is_unimplemented()
    assert hc.prepare(context(), hc.TopK(count=1025), x).route_name() == "topk-sorted-tiles"
    assert hc.prepare(context(), hc.TopK(count=1), D(DT.kInt32, [4, 5000])).route_name() == "topk-select-tiles"
    wide = hc.prepare(context(), hc.TopK(count=8), x)
    assert wide.route_name() == "topk-select-tiles" and wide.workspace_requirement().size == 0
    assert hc.prepare(context(), hc.TopK(count=8), D(DT.kFloat32, [4, 50000])).workspace_requirement().size > 0
    assert hc.prepare(context(), hc.TopK(count=300), x).route_name() == "topk-sorted-tiles"
    assert hc.prepare(context(), hc.TopK(count=1), x).route_name() == "argmax-tiles"
    assert hc.prepare(context(), hc.TopK(count=1, largest=False), x).route_name() == "topk-select-tiles"
    note("topk count 0 writes nothing")
    values, indices = run(hc.TopK(count=0), torch.zeros((3, 9), device=DEVICE))
    assert list(values.shape) == [3, 0] and list(indices.shape) == [3, 0]


def test_topk_counts_above_1024_merge_sorted_runs():
    """Counts the selection and single-tile sorts do not reach: whole sorted tiles, merged as runs."""
    rng = np.random.default_rng(1170)
    for tag, dims, counts in (("f32", [3, 5000], (1025, 2048, 3000, 5000)), ("bf16", [2, 70001], (1500, 4097)),
                              ("f32", [1, 300000], (2049, 20000)), ("f16", [5, 2049], (2049,)),
                              ("f32", [2, 4100, 3], (4000,))):
        stored = tied_values(rng, dims, tag)
        axis = 1 if len(dims) == 3 else -1
        for count in counts:
            for largest in (True, False):
                note(f"topk runs {tag} {dims} count {count} largest {largest}")
                outputs = run(hc.TopK(count=count, axis=axis, largest=largest), to_device(stored, tag))
                check(tag, stored, dims, count, axis, largest, outputs)
    note("topk runs: distinct values, every key kept")
    x = rng.permutation(40000).astype(np.float32).reshape(2, 20000)
    values, indices = run(hc.TopK(count=20000), to_device(x, "f32"))
    assert np.array_equal(to_host(values), -np.sort(-x, axis=1))
    assert np.array_equal(np.take_along_axis(x, to_host(indices).astype(np.int64), 1), to_host(values))


def test_topk_int32_keys():
    """include/hyle/compute/providers/cuda.h:108-121 admits I32: signed integer order, lowest index
    among equals, the extremes included."""
    rng = np.random.default_rng(1171)
    cases = (([4, 37], -1, (1, 5, 37)), ([3, 5000], -1, (1, 64, 300, 2000)), ([6, 9, 16], 1, (4,)), ([2, 70001], -1, (64, 1000)))
    for dims, axis, counts in cases:
        x = rng.integers(-50, 51, dims).astype(np.int32)                 # ties everywhere
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, 5)] = np.iinfo(np.int32).min
        flat[rng.integers(0, flat.size, 5)] = np.iinfo(np.int32).max
        flat[rng.integers(0, flat.size, 7)] = rng.integers(-2**31, 2**31, 7)   # beyond what a float tells apart
        for count in counts:
            for largest in (True, False):
                note(f"topk int32 {dims} axis {axis} count {count} largest {largest}")
                values, indices = run(hc.TopK(count=count, axis=axis, largest=largest), torch.from_numpy(x).to(DEVICE))
                want_values, want_indices = orc.topk(orc.I32, x, dims, count, axis, largest)
                assert np.array_equal(to_host(indices), want_indices)
                assert np.array_equal(to_host(values), want_values)
                order = np.argsort(-x.astype(np.int64) if largest else x.astype(np.int64), axis=axis, kind="stable")
                assert np.array_equal(np.take(order, range(count), axis=axis), want_indices)   # the oracle against numpy


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_topk_rows_at_odd_addresses_on_every_route(tag):
    """Byte strides that leave elements unaligned (src/compute_provider_native/cast.cc:113-116 allows
    them) are read byte by byte: the select route with one tile, with lists, and with two rounds of
    list merges; the sorting route with one tile, with merged lists (one and two rounds), and with
    whole sorted runs."""
    rng = np.random.default_rng(1190)
    size = 4 if tag == "f32" else 2
    for dims, count in (([3, 5000], 17), ([2, 20000], 40), ([2, 140000], 256), ([5, 300], 280), ([2, 5000], 300),
                        ([2, 5000], 1000), ([2, 5000], 1500)):
        values = tied_values(rng, dims, tag)
        row_bytes = dims[1] * size + 3
        raw = np.zeros(dims[0] * row_bytes + 8, np.uint8)
        for r in range(dims[0]):
            raw[r * row_bytes:r * row_bytes + dims[1] * size] = values[r].view(np.uint8)
        desc = hc.TensorDesc.strided_bytes(TYPES[tag][0], dims, [row_bytes, size])
        note(f"topk {tag} {dims} rows {row_bytes} bytes apart, count {count}")
        outputs = run(hc.TopK(count=count), torch.from_numpy(raw).to(DEVICE), descs=[desc])
        check(tag, raw, dims, count, 1, True, outputs, [row_bytes, size])
