"""Parity of Fill and Select (through the C ABI) with the CPU oracle: bit-exact, storage only.

The first case is the reference route test's own (tests/compute_route_vulkan/tensor_test.cc:255-283:
alternating flags, NaN-payload and odd-byte scalars); the masked residual with a rank-0 zero branch
is the shape tests/graph_route_cuda/tensor_test.cc:73-82 builds.  Then broadcast and strided
operands, pointers off the 16-byte grid, writing over a branch in place, and benchmark-sized
tensors checked against the oracle in full."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, context, note, run

pytestmark = pytest.mark.gpu

DT = hc.DataType
# hyle DataType -> (oracle type id of the same width, numpy word type)
KINDS = {
    DT.kBool: (orc.BOOL, np.uint8), DT.kUInt8: (orc.BOOL, np.uint8), DT.kInt8: (orc.BOOL, np.uint8),
    DT.kFloat16: (orc.F16, np.uint16), DT.kBFloat16: (orc.BF16, np.uint16),
    DT.kFloat32: (orc.F32, np.uint32), DT.kInt32: (orc.I32, np.uint32),
}
SCALAR_BITS = {1: 0xE3, 2: 0xFFC3, 4: 0xFFC00003}


def device_bytes(raw: np.ndarray, lead: int = 0) -> torch.Tensor:
    """The array's bytes on the device, `lead` bytes past a 256-byte aligned address."""
    flat = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    holder = torch.empty(flat.size + lead + 16, dtype=torch.uint8, device=DEVICE)
    view = holder[lead:lead + flat.size]
    view.copy_(torch.from_numpy(flat.copy()))
    return view


def random_words(rng, dtype, shape):
    return rng.integers(0, int(np.iinfo(dtype).max) + 1, shape, dtype=np.uint64).astype(dtype)


def fill_on_device(kind: DT, dims, bits: int, lead: int = 0) -> np.ndarray:
    dtype = KINDS[kind][1]
    count = int(np.prod(dims)) if len(dims) else 1
    out = torch.full((count * np.dtype(dtype).itemsize + lead + 32,), 0x5A, dtype=torch.uint8, device=DEVICE)
    target = out[lead:lead + count * np.dtype(dtype).itemsize]
    run(hc.Fill(tuple(dims), kind, hc.ScalarValue.from_bits(kind, bits)), outputs=[target])
    host = out.cpu().numpy()
    assert (host[:lead] == 0x5A).all() and (host[lead + target.numel():] == 0x5A).all(), "Fill wrote outside its output"
    return host[lead:lead + target.numel()].view(dtype).reshape(dims)


def select_on_device(kind: DT, condition, first, second, strides=(None, None, None), dims=None, leads=(0, 0, 0, 0)):
    """Operands as numpy arrays (logical shape = array shape unless `dims[i]` says otherwise)."""
    arrays = (condition, first, second)
    kinds = (DT.kBool, kind, kind)
    descs, tensors = [], []
    for i, array in enumerate(arrays):
        shape = list(dims[i]) if dims and dims[i] is not None else list(array.shape)
        descs.append(hc.TensorDesc.dense(kinds[i], shape) if strides[i] is None
                     else hc.TensorDesc.strided_bytes(kinds[i], shape, strides[i]))
        tensors.append(device_bytes(array, leads[i]))
    prepared = hc.prepare(context(), hc.Select(), *descs)
    shape = prepared.output_description().dimensions
    dtype = KINDS[kind][1]
    count = int(np.prod(shape)) if len(shape) else 1
    out = device_bytes(np.full(count, 0x5A5A5A5A5A5A5A5A, np.uint64).astype(dtype), leads[3])
    prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                        [t.data_ptr() for t in tensors], [out.data_ptr()])
    torch.cuda.synchronize()
    return out.cpu().numpy().view(dtype).reshape(shape), prepared


def oracle_select(kind, condition, first, second, strides=(None, None, None), dims=None):
    def triple(i, array):
        shape = list(dims[i]) if dims and dims[i] is not None else list(array.shape)
        return (array, shape, strides[i])
    out = orc.select(KINDS[kind][0], triple(0, condition), triple(1, first), triple(2, second))
    return out.reshape(-1).view(KINDS[kind][1]).reshape(out.shape)


@pytest.mark.parametrize("kind", list(KINDS))
def test_reference_route_case(kind):
    dtype = KINDS[kind][1]
    width = np.dtype(dtype).itemsize
    for count in (1, 3, 5, 64, 257, 4099):
        note(f"fill + select {kind.name} count {count} (tensor_test.cc:255-283)")
        rng = np.random.default_rng(count + int(kind))
        raw = random_words(rng, dtype, count)
        flags = (np.arange(count) % 2).astype(np.uint8)
        bits = 1 if kind == DT.kBool else SCALAR_BITS[width]
        filled = fill_on_device(kind, [count], bits)
        assert filled.tolist() == [bits] * count
        got, _ = select_on_device(kind, flags, raw, filled)
        expected = raw.copy()
        expected[flags == 0] = bits
        assert np.array_equal(got, expected)


def test_fill_shapes_alignments_and_rejections():
    ctx = context()
    for kind, bits in ((DT.kFloat32, 0x7FC00001), (DT.kBFloat16, 0x8000), (DT.kFloat16, 0x3C01), (DT.kUInt8, 0x7F),
                       (DT.kInt32, 0x80000001), (DT.kBool, 1)):
        width = np.dtype(KINDS[kind][1]).itemsize
        for dims in ([], [1], [15], [3, 11], [2, 3, 257], [40000]):
            for lead in (0, width, 16 - width, 16 + width):
                note(f"fill {kind.name} {dims} at +{lead} bytes")
                got = fill_on_device(kind, dims, bits, lead)
                assert got.shape == tuple(dims) and (got == bits).all()
    note("fill: zero elements is a no-op plan; type and shape errors follow operation.cc:1263-1275")
    empty = hc.prepare(ctx, hc.Fill((4, 0), DT.kFloat32, hc.ScalarValue.of(DT.kFloat32, 1.0)))
    assert empty.dispatch_count() == 0 and empty.output_description() == hc.TensorDesc.dense(DT.kFloat32, [4, 0])
    with pytest.raises(hc.StatusError) as err:   # scalar of another type
        hc.prepare(ctx, hc.Fill((4,), DT.kFloat32, hc.ScalarValue.of(DT.kBFloat16, 1.0)))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Fill((4,), DT.kUnknown, hc.ScalarValue()))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:   # bits wider than the element
        hc.prepare(ctx, hc.Fill((4,), DT.kBFloat16, hc.ScalarValue.from_bits(DT.kBFloat16, 0x13F80)))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    note("ScalarValue.of narrows to nearest even")
    assert hc.ScalarValue.of(DT.kBFloat16, 1.00390625).bits == 0x3F80      # tie to even
    assert hc.ScalarValue.of(DT.kBFloat16, 1.01171875).bits == 0x3F82      # tie to even, upwards
    assert hc.ScalarValue.of(DT.kFloat16, -2.0).bits == 0xC000
    assert hc.ScalarValue.of(DT.kInt32, -1).bits == 0xFFFFFFFF
    got = fill_on_device(DT.kFloat32, [9], hc.ScalarValue.of(DT.kFloat32, -0.0).bits)
    assert (got == 0x80000000).all()


SHAPES = [
    ([4, 1, 6], [5, 6], [4, 5, 1]),
    ([3, 7], [], [7]),
    ([1], [2, 3, 4], [2, 3, 4]),
    ([2, 3, 4], [2, 3, 4], []),      # masked residual with a rank-0 zero (graph_route_cuda/tensor_test.cc:73-82)
    ([33, 129], [33, 129], [33, 129]),
    ([], [], []),
    ([5, 0, 3], [1, 3], [5, 1, 1]),
]


@pytest.mark.parametrize("kind", [DT.kBool, DT.kBFloat16, DT.kFloat16, DT.kFloat32, DT.kInt32, DT.kInt8])
def test_select_broadcasts_like_the_oracle(kind):
    dtype = KINDS[kind][1]
    for n, shapes in enumerate(SHAPES):
        note(f"select {kind.name} {shapes}")
        rng = np.random.default_rng(n * 17 + int(kind))
        condition = rng.integers(0, 3, shapes[0]).astype(np.uint8)
        if condition.size:
            condition.reshape(-1)[::5] = 0x80
        first, second = random_words(rng, dtype, shapes[1]), random_words(rng, dtype, shapes[2])
        got, prepared = select_on_device(kind, condition, first, second)
        want = oracle_select(kind, condition, first, second)
        assert got.shape == want.shape and np.array_equal(got, want)
        assert np.array_equal(want, np.where(condition != 0, first, second))
        if 0 in got.shape:
            assert prepared.dispatch_count() == 0


def test_select_strided_and_unaligned_operands():
    rng = np.random.default_rng(5)
    note("select f32: transposed first branch, condition with holes, column second branch")
    base = random_words(rng, np.uint32, (6, 4))
    holes = rng.integers(0, 2, (4, 6, 2)).astype(np.uint8)
    column = random_words(rng, np.uint32, (4, 1))
    kwargs = dict(strides=([12, 2], [4, 16], None), dims=([4, 6], [4, 6], None))
    got, prepared = select_on_device(DT.kFloat32, holes, base, column, **kwargs)
    assert prepared.route_name() == "select"
    assert np.array_equal(got, oracle_select(DT.kFloat32, holes, base, column, **kwargs))
    assert np.array_equal(got, np.where(holes[:, :, 0] != 0, base.T, column))
    note("select bf16: byte strides that leave elements unaligned (read bytewise)")
    physical = rng.integers(0, 256, 64).astype(np.uint8)
    flags = rng.integers(0, 2, (3, 4)).astype(np.uint8)
    other = random_words(rng, np.uint16, (3, 4))
    kwargs = dict(strides=(None, [17, 3], None), dims=(None, [3, 4], None))
    got, _ = select_on_device(DT.kBFloat16, flags, physical, other, **kwargs)
    assert np.array_equal(got, oracle_select(DT.kBFloat16, flags, physical, other, **kwargs))
    for kind in (DT.kBool, DT.kBFloat16, DT.kFloat32):
        dtype = KINDS[kind][1]
        width = np.dtype(dtype).itemsize
        for count in (1, 15, 16, 17, 1000, 4099):
            for leads in ((0, 0, 0, 0), (1, width, 0, 0), (0, 0, width, 16 - width), (3, 0, 0, width)):
                note(f"select {kind.name} count {count} operands at +{leads} bytes")
                condition = rng.integers(0, 2, count).astype(np.uint8)
                first, second = random_words(rng, dtype, count), random_words(rng, dtype, count)
                got, _ = select_on_device(kind, condition, first, second, leads=leads)
                assert np.array_equal(got, np.where(condition != 0, first, second))


def test_select_in_place_and_alias_rules():
    ctx = context()
    D = hc.TensorDesc.dense
    rng = np.random.default_rng(9)
    for kind, shape in ((DT.kFloat32, [37, 129]), (DT.kBFloat16, [4099]), (DT.kBool, [5, 7])):
        dtype = KINDS[kind][1]
        prepared = hc.prepare(ctx, hc.Select(), D(DT.kBool, shape), D(kind, shape), D(kind, []))
        assert not prepared.alias_support(0, 0) and prepared.alias_support(0, 1) and not prepared.alias_support(0, 2)
        condition = rng.integers(0, 2, shape).astype(np.uint8)
        first, zero = random_words(rng, dtype, shape), np.zeros([], dtype)
        tensors = [device_bytes(condition), device_bytes(first), device_bytes(zero)]
        note(f"select {kind.name} {shape}: output written over the first branch")
        prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                            [t.data_ptr() for t in tensors], [tensors[1].data_ptr()])
        torch.cuda.synchronize()
        got = tensors[1].cpu().numpy().view(dtype).reshape(shape)
        assert np.array_equal(got, np.where(condition != 0, first, zero))
    note("select: the condition is never an alias, nor a broadcast branch")
    prepared = hc.prepare(ctx, hc.Select(), D(DT.kBool, [8]), D(DT.kBool, [8]), D(DT.kBool, [8]))
    storage = torch.zeros(64, dtype=torch.uint8, device=DEVICE)
    with pytest.raises(hc.StatusError) as err:
        prepared.create_invocation().submit(torch.cuda.current_stream().cuda_stream,
                                            [storage.data_ptr(), storage.data_ptr() + 16, storage.data_ptr() + 32],
                                            [storage.data_ptr()])
    assert err.value.code == hc.StatusCode.kInvalidArgument
    note("select: schema errors (operation.cc:1309-1330)")
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Select(), D(DT.kUInt8, [8]), D(DT.kFloat32, [8]), D(DT.kFloat32, [8]))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Select(), D(DT.kBool, [8]), D(DT.kFloat32, [8]), D(DT.kBFloat16, [8]))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Select(), D(DT.kBool, [8]), D(DT.kFloat32, [7]), D(DT.kFloat32, [8]))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Select(), D(DT.kBool, [8]), D(DT.kFloat32, [8]))
    assert err.value.code == hc.StatusCode.kInvalidArgument


def test_fill_and_select_at_benchmark_sizes():
    """[9496, 4096]: the oracle walks the whole tensor (a few seconds), and torch.where over the
    same device bytes gives a second, independent reading."""
    rows, cols = 9496, 4096
    rng = np.random.default_rng(77)
    for kind, torch_words in ((DT.kBFloat16, torch.int16), (DT.kFloat32, torch.int32)):
        dtype = KINDS[kind][1]
        note(f"fill {kind.name} [{rows}, {cols}]")
        bits = SCALAR_BITS[np.dtype(dtype).itemsize]
        out = torch.empty(rows * cols * np.dtype(dtype).itemsize, dtype=torch.uint8, device=DEVICE)
        run(hc.Fill((rows, cols), kind, hc.ScalarValue.from_bits(kind, bits)), outputs=[out])
        signed = bits - (1 << (8 * np.dtype(dtype).itemsize))
        assert bool((out.view(torch_words) == signed).all())
        note(f"select {kind.name} [{rows}, {cols}] with a row branch and a scalar branch")
        condition = torch.from_numpy(rng.integers(0, 2, (rows, cols)).astype(np.uint8)).to(DEVICE)
        signed_words = np.int16 if torch_words == torch.int16 else np.int32
        first = torch.from_numpy(random_words(rng, dtype, (rows, cols)).view(signed_words)).to(DEVICE)
        row = torch.from_numpy(random_words(rng, dtype, (cols,)).view(signed_words)).to(DEVICE)
        D = hc.TensorDesc.dense
        (general,) = run(hc.Select(), condition, first.view(torch.uint8), row.view(torch.uint8),
                         descs=[D(DT.kBool, [rows, cols]), D(kind, [rows, cols]), D(kind, [cols])],
                         outputs=[torch.empty_like(first)])
        assert torch.equal(general, torch.where(condition != 0, first, row))
        scalar = row[:1].clone()
        (flat,) = run(hc.Select(), condition, first.view(torch.uint8), scalar.view(torch.uint8),
                      descs=[D(DT.kBool, [rows, cols]), D(kind, [rows, cols]), D(kind, [])],
                      outputs=[torch.empty_like(first)])
        assert torch.equal(flat, torch.where(condition != 0, first, scalar))
        want = oracle_select(kind, condition.cpu().numpy(), first.cpu().numpy(), scalar.cpu().numpy().reshape(()))
        assert np.array_equal(flat.cpu().numpy().view(dtype), want)
