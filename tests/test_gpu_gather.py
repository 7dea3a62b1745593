"""Parity of Gather (through the C ABI) with the CPU oracle: bit-exact, storage only.

The cases are the reference's (tests/compute_provider_cuda/gather_collectives_test.cc): the
[2, 7, 3] matrix over axes, strides, element widths and index widths (…:13-24,143-170), megabyte
rows with repeated indices, odd byte counts and offset buffers (…:27-68,119-129), checked failures
that keep every output byte and report OutOfRange, a fresh launch recovering (…:70-117,172-212),
empty operands and alias rejection (…:279-338), plus an embedding-sized lookup."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import capi
from hyle_amd import compute as hc
from oracle import lib as orc

from gather_support import WORDS, byte_strides, lay_out, reference_indices, reference_values
from gpu_support import DEVICE, context, note

pytestmark = pytest.mark.gpu

DT = hc.DataType
STORAGE = {1: [DT.kBool, DT.kFloat8E4M3FN, DT.kFloat8E5M2, DT.kInt8, DT.kUInt8],
           2: [DT.kFloat16, DT.kBFloat16, DT.kInt16, DT.kUInt16],
           4: [DT.kFloat32, DT.kInt32, DT.kUInt32],
           8: [DT.kFloat64, DT.kInt64, DT.kUInt64]}


def on_device(raw: np.ndarray) -> torch.Tensor:
    flat = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    return torch.from_numpy(flat.copy()).to(DEVICE) if flat.size else torch.empty(16, dtype=torch.uint8, device=DEVICE)


def describe(kind, shape, strides, dense):
    return hc.TensorDesc.dense(kind, shape) if dense else hc.TensorDesc.strided_bytes(kind, shape, strides)


def gather_on_device(kind, size, storage, lead, shape, strides, dense, axis, index_storage, index_lead, index_shape,
                     index_strides, index_dense, wide, checked=True, poison=0x5A, out_lead=0, static=False):
    """Returns (status code or 0, output bytes viewed as the element's word)."""
    bounds = hc.IndexBoundsPolicy.kChecked if checked else hc.IndexBoundsPolicy.kUnchecked
    index_kind = DT.kInt64 if wide else DT.kInt32
    prepared = hc.prepare(context(), hc.Gather(axis, bounds), describe(kind, shape, strides, dense),
                          describe(index_kind, index_shape, index_strides, index_dense))
    normal = axis + len(shape) if axis < 0 else axis
    out_shape = list(shape[:normal]) + list(index_shape) + list(shape[normal + 1:])
    assert prepared.output_description() == hc.TensorDesc.dense(kind, out_shape)
    count = int(np.prod(out_shape)) if out_shape else 1
    # checked bounds: a dispatch that looks at the indices first, unless they are few and whole rows
    # move, when every moving block looks at them itself
    assert prepared.dispatch_count() == (0 if count == 0 else 1) or (checked and prepared.dispatch_count() == 2)
    source, ids = on_device(storage), on_device(index_storage)
    out = torch.full((out_lead + max(count, 1) * size + 16,), poison, dtype=torch.uint8, device=DEVICE)
    need = prepared.workspace_requirement()
    workspace = torch.empty(max(need.size, 1), dtype=torch.uint8, device=DEVICE)
    stream = torch.cuda.current_stream().cuda_stream
    status = 0
    try:
        if static:
            invocation = prepared.create_invocation_without_workspace()
            invocation.submit_without_workspace(stream, [source.data_ptr() + lead, ids.data_ptr() + index_lead],
                                                [out.data_ptr() + out_lead])
        else:
            invocation = prepared.create_invocation(workspace.data_ptr(), need.size)
            invocation.submit(stream, [source.data_ptr() + lead, ids.data_ptr() + index_lead], [out.data_ptr() + out_lead])
        invocation.wait(stream, static_scratch=static)
    except hc.StatusError as error:
        status = error.code
    torch.cuda.synchronize()
    host = out.cpu().numpy()
    assert (host[:out_lead] == poison).all() and (host[out_lead + count * size:] == poison).all(), "wrote outside the output"
    return status, host[out_lead:out_lead + count * size].copy().view(WORDS[size]).reshape(out_shape)


def reference_case(kind, size, shape, axis, index_shape, source_mode, index_mode, wide, checked=True):
    normal = axis + len(shape) if axis < 0 else axis
    strides = byte_strides(shape, size, normal, source_mode)
    storage, values = lay_out(reference_values(shape, size, kind == DT.kBool), strides, lead=size)
    width = 8 if wide else 4
    index_axis = len(index_shape) - 1 if index_shape else 0
    index_strides = byte_strides(index_shape, width, index_axis, index_mode)
    index_storage, ids = lay_out(reference_indices(index_shape, shape[normal], wide), index_strides, lead=width)
    status, got = gather_on_device(kind, size, storage, size, shape, strides, source_mode == 0, axis, index_storage, width,
                                   index_shape, index_strides, index_mode == 0, wide, checked)
    oracle_status, want = orc.gather(storage[size:].copy(), shape, strides, axis, index_storage[width:].copy(), index_shape,
                                     index_strides, checked=checked, width=size, wide=wide,
                                     into=np.zeros(got.shape, WORDS[size]))
    assert status == 0 and oracle_status == 0
    assert np.array_equal(got, want)
    assert np.array_equal(want, np.take(values, ids.astype(np.int64), axis=normal))


@pytest.mark.parametrize("size", [1, 2, 4, 8])
def test_reference_matrix_every_storage_type_and_index_width(size):
    for kind in STORAGE[size]:
        for wide in (False, True):
            for axis in (0, 1, -1):
                for source_mode in (0, 1):
                    for index_mode in (0, 1):
                        note(f"gather {kind.name} wide={wide} axis={axis} source_mode={source_mode} index_mode={index_mode}")
                        reference_case(kind, size, [2, 7, 3], axis, [2, 3], source_mode, index_mode, wide,
                                       checked=(source_mode + index_mode) % 2 == 0)


def test_reference_special_shapes():
    note("gather rank-8 f64 source")
    reference_case(DT.kFloat64, 8, [1, 2, 1, 3, 1, 5, 2, 1], 5, [4], 1, 1, True)
    note("gather rank-0 index, source broadcast on the axis")
    reference_case(DT.kBFloat16, 2, [2, 1, 7, 3, 1, 2], 2, [], 2, 0, False)
    note("gather 2-D indices broadcast along their last axis")
    reference_case(DT.kUInt8, 1, [4, 3], 0, [2, 3], 0, 2, True)


@pytest.mark.parametrize("kind,size,wide,columns,offset,index_mode,checked", [
    (DT.kFloat32, 4, False, 262144, False, 0, True),
    (DT.kFloat64, 8, True, 131072, False, 1, True),
    (DT.kUInt8, 1, True, 1048579, True, 0, True),
    (DT.kUInt32, 4, False, 262145, True, 1, False),
])
def test_wide_dense_rows_with_outer_groups_duplicates_and_tails(kind, size, wide, columns, offset, index_mode, checked):
    note(f"gather wide rows {kind.name} columns={columns} offset={offset} index_mode={index_mode} checked={checked}")
    shape = [2, 3, columns]
    strides = byte_strides(shape, size, 1, 0)
    lead = size if offset else 0
    storage, values = lay_out(reference_values(shape, size), strides, lead=lead)
    width = 8 if wide else 4
    index_strides = byte_strides([3], width, 0, index_mode)
    selected = np.array([2, 0, 2], np.int64 if wide else np.int32)   # repeated source rows are legal
    index_storage, ids = lay_out(selected, index_strides, lead=width)
    status, got = gather_on_device(kind, size, storage, lead, shape, strides, True, 1, index_storage, width, [3],
                                   index_strides, index_mode == 0, wide, checked, out_lead=lead)
    assert status == 0
    assert np.array_equal(got, values[:, [2, 0, 2], :])


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("static", [False, True])
def test_checked_failure_keeps_every_output_byte_and_a_fresh_launch_recovers(wide, static):
    kind = np.int64 if wide else np.int32
    shape = [3, 262144]
    values = (np.arange(3 * 262144, dtype=np.uint64) + 0x7FC00001).astype(np.uint32).reshape(shape)
    for invalid in (-1, 3, np.iinfo(kind).max, np.iinfo(kind).min):
        note(f"gather checked failure wide={wide} static={static} invalid={invalid}")
        ids = np.array([2, 0, invalid], kind)
        status, got = gather_on_device(DT.kFloat32, 4, values, 0, shape, None, True, 0, ids, 0, [3], None, True, wide,
                                       poison=0xEF, static=static)
        assert status == capi.OUT_OF_RANGE
        assert (got.view(np.uint8) == 0xEF).all()
        oracle_status, _ = orc.gather(values, shape, None, 0, ids, [3], None, checked=True)
        assert oracle_status == 1
    note(f"gather recovery wide={wide} static={static}")
    status, got = gather_on_device(DT.kFloat32, 4, values, 0, shape, None, True, 0, np.array([2, 0, 2], kind), 0, [3], None,
                                   True, wide, static=static)
    assert status == 0 and np.array_equal(got, values[[2, 0, 2]])


def test_checked_failure_in_a_strided_gather():
    # the failing index sits in a strided index tensor and the source is strided: the general kernels
    shape, size = [4, 3], 8
    strides = byte_strides(shape, size, 0, 1)
    storage, values = lay_out(np.arange(1, 13, dtype=np.uint64).reshape(shape), strides)
    index_strides = byte_strides([2], 8, 0, 1)
    for invalid in (-1, 4, np.iinfo(np.int64).max, np.iinfo(np.int64).min):
        note(f"gather strided checked failure invalid={invalid}")
        index_storage, _ = lay_out(np.array([0, invalid], np.int64), index_strides)
        status, got = gather_on_device(DT.kFloat64, size, storage, 0, shape, strides, False, 0, index_storage, 0, [2],
                                       index_strides, False, True, poison=0x77)
        assert status == capi.OUT_OF_RANGE and (got.view(np.uint8) == 0x77).all()
    index_storage, _ = lay_out(np.array([3, 1], np.int64), index_strides)
    status, got = gather_on_device(DT.kFloat64, size, storage, 0, shape, strides, False, 0, index_storage, 0, [2],
                                   index_strides, False, True)
    assert status == 0 and np.array_equal(got, [[10, 11, 12], [4, 5, 6]])


def test_one_bad_index_among_many_is_found():
    rows, width, count = 1000, 64, 200_000
    values = np.random.default_rng(1).integers(0, 1 << 16, (rows, width), dtype=np.uint64).astype(np.uint16)
    ids = np.random.default_rng(2).integers(0, rows, count).astype(np.int32)
    for place in (0, 65_537, count - 1):
        note(f"gather one bad index at {place}")
        bad = ids.copy()
        bad[place] = rows
        status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, bad, 0, [count], None, True,
                                       False, poison=0x11)
        assert status == capi.OUT_OF_RANGE and (got.view(np.uint8) == 0x11).all()
    status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, ids, 0, [count], None, True, False)
    assert status == 0 and np.array_equal(got, values[ids])


def test_empty_operands_and_rejected_bindings():
    desc = hc.TensorDesc.dense(DT.kInt32, [4])
    stream = torch.cuda.current_stream().cuda_stream
    source = torch.tensor([5, 6, 7, 8], dtype=torch.int32, device=DEVICE)
    ids = torch.tensor([3, 2, 1, 0], dtype=torch.int32, device=DEVICE)
    out = torch.zeros(4, dtype=torch.int32, device=DEVICE)
    prepared = hc.prepare(context(), hc.Gather(0, hc.IndexBoundsPolicy.kUnchecked), desc, desc)
    assert prepared.workspace_requirement().size == 0 and prepared.dispatch_count() == 1
    invocation = prepared.create_invocation(0, 0)
    for alias in (source, ids):   # the output may be neither input
        with pytest.raises(hc.StatusError) as refused:
            invocation.submit(stream, [source.data_ptr(), ids.data_ptr()], [alias.data_ptr()])
        assert refused.value.code == capi.INVALID_ARGUMENT
    with pytest.raises(hc.StatusError):  # nor overlap one partly
        invocation.submit(stream, [source.data_ptr(), ids.data_ptr()], [source.data_ptr() + 4])
    invocation.submit(stream, [source.data_ptr(), ids.data_ptr()], [out.data_ptr()])
    invocation.wait(stream)
    torch.cuda.synchronize()
    assert out.tolist() == [8, 7, 6, 5]
    # empty outputs launch nothing and look at no index
    for source_shape, index_shape in (([4, 0], [4]), ([4], [0])):
        empty = hc.prepare(context(), hc.Gather(), hc.TensorDesc.dense(DT.kInt32, source_shape),
                           hc.TensorDesc.dense(DT.kInt32, index_shape))
        assert empty.dispatch_count() == 0 and empty.workspace_requirement().size == 0
        empty.create_invocation(0, 0).submit(stream, [0, 0], [0])
    # an empty axis cannot be indexed (src/compute_provider_native/indexing.cc:189-195)
    hollow = hc.prepare(context(), hc.Gather(0, hc.IndexBoundsPolicy.kUnchecked), hc.TensorDesc.dense(DT.kInt32, [0, 3]),
                        hc.TensorDesc.dense(DT.kInt32, [2]))
    with pytest.raises(hc.StatusError) as refused:
        hollow.create_invocation(0, 0).submit(stream, [source.data_ptr(), ids.data_ptr()], [out.data_ptr()])
    assert refused.value.code == capi.OUT_OF_RANGE


def test_few_checked_indices_take_one_dispatch():
    wide = hc.prepare(context(), hc.Gather(0), hc.TensorDesc.dense(DT.kBFloat16, [4096, 2048]), hc.TensorDesc.dense(DT.kInt32, [8]))
    many = hc.prepare(context(), hc.Gather(0), hc.TensorDesc.dense(DT.kBFloat16, [4096, 2048]), hc.TensorDesc.dense(DT.kInt32, [2000]))
    assert wide.dispatch_count() == 1 and many.dispatch_count() == 2
    assert wide.workspace_requirement().size == many.workspace_requirement().size > 0   # the status word lives there either way
    rows, width = 4096, 2048
    values = np.random.default_rng(8).integers(0, 1 << 16, (rows, width), dtype=np.uint64).astype(np.uint16)
    for count in (1, 8, 1000):
        ids = np.random.default_rng(count).integers(0, rows, count).astype(np.int64)
        note(f"gather {count} checked indices in one dispatch")
        status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, ids, 0, [count], None, True, True)
        assert status == 0 and np.array_equal(got, values[ids])
        ids[count // 2] = rows
        status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, ids, 0, [count], None, True, True,
                                       poison=0x33)
        assert status == capi.OUT_OF_RANGE and (got.view(np.uint8) == 0x33).all()


def test_many_long_checked_rows_check_themselves_while_they_load():
    """A launch large enough for the blocks of sixteen chunks takes one dispatch up to 16384 indices: valid
    indices move every row, one bad index (negative, past the axis, first or last) moves none; both index
    widths, rows of 4 KiB and of 4 KiB + 16 bytes (a short last chunk), and an outer group."""
    D = hc.TensorDesc.dense
    one = hc.prepare(context(), hc.Gather(0), D(DT.kBFloat16, [5000, 2048]), D(DT.kInt32, [8192]))
    two = hc.prepare(context(), hc.Gather(0), D(DT.kBFloat16, [5000, 2048]), D(DT.kInt32, [20000]))
    short = hc.prepare(context(), hc.Gather(0), D(DT.kBFloat16, [5000, 1024]), D(DT.kInt32, [8192]))
    assert one.dispatch_count() == 1 and two.dispatch_count() == 2 and short.dispatch_count() == 2
    for rows, width, shape, wide in ((5000, 2048, [4096], False), (3000, 2056, [64, 80], True), (2, 2048, [4100], False)):
        count = int(np.prod(shape))
        values = np.random.default_rng(rows).integers(0, 1 << 16, (rows, width), dtype=np.uint64).astype(np.uint16)
        ids = np.random.default_rng(width).integers(0, rows, shape).astype(np.int64 if wide else np.int32)
        note(f"gather {shape} checked rows of {2 * width} bytes out of {rows}, one dispatch")
        status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, ids, 0, shape, None, True, wide)
        assert status == 0 and np.array_equal(got, values[ids])
        for place, value in ((0, -1), (count - 1, rows), (count // 3, 1 << 30)):
            bad = ids.copy().reshape(-1)
            bad[place] = value
            status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [rows, width], None, True, 0, bad.reshape(shape), 0, shape,
                                           None, True, wide, poison=0x77)
            assert status == capi.OUT_OF_RANGE and (got.view(np.uint8) == 0x77).all()
    note("gather [3, 1500, 2048] along axis 1 by 1400 checked indices, one dispatch")
    values = np.random.default_rng(5).integers(0, 1 << 16, (3, 1500, 2048), dtype=np.uint64).astype(np.uint16)
    ids = np.random.default_rng(6).integers(0, 1500, 1400).astype(np.int32)
    status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [3, 1500, 2048], None, True, 1, ids, 0, [1400], None, True, False)
    assert status == 0 and np.array_equal(got, values[:, ids])
    ids[700] = 1500
    status, got = gather_on_device(DT.kBFloat16, 2, values, 0, [3, 1500, 2048], None, True, 1, ids, 0, [1400], None, True, False,
                                   poison=0x42)
    assert status == capi.OUT_OF_RANGE and (got.view(np.uint8) == 0x42).all()


def test_embedding_sized_lookup():
    note("gather embedding [151936, 2048] bf16 by 8192 int32 indices")
    rows, width, count = 151936, 2048, 8192
    table = torch.randint(-32768, 32767, (rows, width), dtype=torch.int16, device=DEVICE)
    ids = torch.randint(0, rows, (count,), dtype=torch.int32, device=DEVICE)
    out = torch.zeros((count, width), dtype=torch.int16, device=DEVICE)
    prepared = hc.prepare(context(), hc.Gather(0), hc.TensorDesc.dense(DT.kBFloat16, [rows, width]),
                          hc.TensorDesc.dense(DT.kInt32, [count]))
    need = prepared.workspace_requirement()
    workspace = torch.empty(need.size, dtype=torch.uint8, device=DEVICE)
    stream = torch.cuda.current_stream().cuda_stream
    invocation = prepared.create_invocation(workspace.data_ptr(), need.size)
    invocation.submit(stream, [table.data_ptr(), ids.data_ptr()], [out.data_ptr()])
    invocation.wait(stream)
    host_ids = ids.cpu().numpy()
    picked = table[ids.long()[:64]].cpu().numpy()   # a sample through the oracle, the whole through row identity
    status, want = orc.gather(picked.view(np.uint16), [64, width], None, 0, np.arange(64, dtype=np.int32), [64], None)
    assert status == 0 and np.array_equal(out[:64].cpu().numpy().view(np.uint16), want)
    assert torch.equal(out, table[ids.long()])
    assert host_ids.min() >= 0


@pytest.mark.parametrize("unit", [1, 2, 4, 8, 16])
def test_whole_rows_in_every_unit_form_and_index_layout(unit):
    """Rows moved whole take the widest unit (1 to 16 bytes) that divides the row and both addresses,
    in one of three forms: short rows unit by unit, long rows chunk by chunk, and many chunks in fat
    blocks that resolve their lookups first; each with 32- and 64-bit indices, dense and strided."""
    size = min(unit, 8)
    kind = {1: DT.kUInt8, 2: DT.kUInt16, 4: DT.kUInt32, 8: DT.kUInt64}[size]
    per_unit = unit // size
    for form, units_per_row, picks in (("units", 9, 50), ("rows", 257, 100), ("rows_fat", 257, 2100)):
        shape = [37, units_per_row * per_unit]       # an odd number of units: no wider unit divides the row
        strides = byte_strides(shape, size, 0, 0)
        storage, values = lay_out(reference_values(shape, size), strides, lead=unit)   # the source starts `unit` bytes in
        for wide in (False, True):
            for index_mode in (0, 1):
                width = 8 if wide else 4
                index_strides = byte_strides([picks], width, 0, index_mode)
                index_storage, ids = lay_out(reference_indices([picks], shape[0], wide), index_strides, lead=width)
                note(f"gather whole rows: unit {unit} form {form} wide={wide} index_mode={index_mode}")
                status, got = gather_on_device(kind, size, storage, unit, shape, strides, True, 0, index_storage, width, [picks],
                                               index_strides, index_mode == 0, wide, checked=index_mode == 0)
                assert status == 0
                assert np.array_equal(got, np.take(values, ids.astype(np.int64), axis=0))
                label = f"gather_{form}/{unit}-bytes/{'i64' if wide else 'i32'}/{'dense' if index_mode == 0 else 'strided'}"
                assert label in hc.last_launch_variant().split(" + "), (hc.last_launch_variant(), label)
