"""Parity of Cast and Copy (through the C ABI) with the CPU oracle: bit-exact for every pair.

Layout follows tests/compute_provider_native/cast_test.cc of the reference: its known-answer
cases first (f32 -> f16 bit patterns, a strided f16 input, int32 rounding on both sides of the
2^24 ties with odd byte strides, Boolean truth of signed zeros / subnormals / NaNs), then every
admitted pair over edge sizes and special values, then the benchmark shapes.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, context, note, run

pytestmark = pytest.mark.gpu

DT = hc.DataType
# hyle DataType -> (oracle type id, numpy storage dtype, torch dtype that owns the bytes)
KINDS = {
    DT.kFloat32: (orc.F32, np.uint32, torch.int32),
    DT.kFloat16: (orc.F16, np.uint16, torch.int16),
    DT.kBFloat16: (orc.BF16, np.uint16, torch.int16),
    DT.kBool: (orc.BOOL, np.uint8, torch.uint8),
    DT.kInt32: (orc.I32, np.uint32, torch.int32),
}
FLOATS = (DT.kFloat32, DT.kFloat16, DT.kBFloat16)
PAIRS = ([(s, d) for s in FLOATS for d in FLOATS] + [(DT.kInt32, DT.kFloat32)] +
         [(DT.kBool, d) for d in FLOATS] + [(s, DT.kBool) for s in FLOATS])


def device_bytes(raw: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(raw).view(np.uint8).reshape(-1).copy()).to(DEVICE)


def cast_on_device(src: DT, dst: DT, storage: np.ndarray, dims, byte_strides=None):
    """storage: the input's bytes (any numpy dtype).  Returns the dense output as dst's storage dtype."""
    desc = (hc.TensorDesc.dense(src, dims) if byte_strides is None
            else hc.TensorDesc.strided_bytes(src, dims, byte_strides))
    data = device_bytes(storage)
    operation = hc.Copy() if src == dst else hc.Cast(dst)
    (out,) = run(operation, data, descs=[desc])
    raw = out.contiguous().view(torch.uint8).cpu().numpy()
    return raw.view(KINDS[dst][1]).reshape(dims)


def specials(kind: DT, rng, count: int) -> np.ndarray:
    """Stored bit patterns: random words plus zeros, subnormals, infinities, NaNs, extremes."""
    if kind == DT.kBool:
        values = rng.integers(0, 3, count).astype(np.uint8)
        values[::7] = 255
        return values
    if kind in (DT.kFloat32, DT.kInt32):
        words = rng.integers(0, 1 << 32, count, dtype=np.uint64).astype(np.uint32)
        planted = [0, 0x80000000, 1, 0x80000001, 0x007FFFFF, 0x00800000, 0x3F800000, 0x7F7FFFFF, 0x7F800000,
                   0xFF800000, 0x7FC00001, 0xFFC12345, 0x7F800001, 0x477FE000, 0x477FF000, 0x38800000, 0x387FC000,
                   0x33000000, 0x33000001, 0x7FFFFFFF, 0x4B7FFFFF, 0x4B800001]
    else:
        words = rng.integers(0, 1 << 16, count, dtype=np.uint32).astype(np.uint16)
        planted = [0, 0x8000, 1, 0x8001, 0x03FF, 0x0400, 0x3C00, 0x3F80, 0x7BFF, 0x7C00, 0xFC00, 0x7E01, 0xFFC1,
                   0x7F7F, 0x7F80, 0xFF80, 0x7FC1, 0x7C01]
    words[:min(len(planted), count)] = np.array(planted[:count], words.dtype)
    return words


def test_cast_reference_known_answers():
    note("cast f32 -> f16 bit patterns (cast_test.cc:139-143)")
    got = cast_on_device(DT.kFloat32, DT.kFloat16, np.array([0.0, 1.0, -2.0, 0.5, 65504.0], np.float32), [5])
    assert got.tolist() == [0x0000, 0x3C00, 0xC000, 0x3800, 0x7BFF]

    note("cast strided f16 [2,2] strides {5,2} -> f32 (cast_test.cc:177-183)")
    physical = np.zeros(16, np.uint8)
    for bits, offset in zip((0x3C00, 0x4000, 0x4200, 0x4400), (0, 2, 5, 7)):
        physical[offset:offset + 2] = np.frombuffer(np.uint16(bits).tobytes(), np.uint8)
    got = cast_on_device(DT.kFloat16, DT.kFloat32, physical, [2, 2], [5, 2])
    assert got.view(np.float32).tolist() == [[1.0, 2.0], [3.0, 4.0]]

    values = np.array([0, 1, -1, 129279, 16777215, 16777216, 16777217, 16777219, -16777217, -16777219,
                       2147483520, 2147483583, 2147483584, 2**31 - 1, -2**31, -2**31 + 1], np.int64).astype(np.int32)
    expected = [0x00000000, 0x3F800000, 0xBF800000, 0x47FC7F80, 0x4B7FFFFF, 0x4B800000, 0x4B800000, 0x4B800002,
                0xCB800000, 0xCB800002, 0x4EFFFFFF, 0x4EFFFFFF, 0x4F000000, 0x4F000000, 0xCF000000, 0xCF000000]
    note("cast int32 -> f32 around the 2^24 ties and the 2^31 carry, dense (cast_test.cc:232-247)")
    assert cast_on_device(DT.kInt32, DT.kFloat32, values, [2, 8]).reshape(-1).tolist() == expected
    note("cast int32 -> f32 with byte strides {51, 5}: unaligned elements")
    physical = np.full(96, 0x5A, np.uint8)
    for i, v in enumerate(values):
        offset = (i // 8) * 51 + (i % 8) * 5
        physical[offset:offset + 4] = np.frombuffer(np.int32(v).tobytes(), np.uint8)
    assert cast_on_device(DT.kInt32, DT.kFloat32, physical, [2, 8], [51, 5]).reshape(-1).tolist() == expected

    for kind, words, one, dtype in (
            (DT.kFloat32, [0, 0x80000000, 1, 0x80000001, 0x3F800000, 0xBF800000, 0x7F800000, 0x7FC00001], 0x3F800000, np.uint32),
            (DT.kFloat16, [0, 0x8000, 1, 0x8001, 0x3C00, 0xBC00, 0x7C00, 0x7E01], 0x3C00, np.uint16),
            (DT.kBFloat16, [0, 0x8000, 1, 0x8001, 0x3F80, 0xBF80, 0x7F80, 0x7FC1], 0x3F80, np.uint16)):
        note(f"cast {kind.name} -> Bool and back (cast_test.cc:389-396)")
        assert cast_on_device(kind, DT.kBool, np.array(words, dtype), [2, 4]).reshape(-1).tolist() == [0, 0, 1, 1, 1, 1, 1, 1]
        boolean = np.array([0, 1, 2, 255, 1, 0, 0, 1], np.uint8)
        assert cast_on_device(DT.kBool, kind, boolean, [2, 4]).reshape(-1).tolist() == [one if b else 0 for b in boolean]
        note(f"cast Bool with byte strides {{11, 2}} -> {kind.name}")
        raw = np.full(32, 0x5A, np.uint8)
        for i, b in enumerate(boolean):
            raw[(i // 4) * 11 + (i % 4) * 2] = b
        assert cast_on_device(DT.kBool, kind, raw, [2, 4], [11, 2]).reshape(-1).tolist() == [one if b else 0 for b in boolean]


def test_cast_declines_and_rejections():
    ctx = context()
    D = hc.TensorDesc.dense
    note("cast f32 -> int32 is declined (cast_test.cc:296-301)")
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Cast(DT.kInt32), D(DT.kFloat32, [2, 8]))
    assert err.value.code == hc.StatusCode.kUnimplemented
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Cast(DT.kFloat16), D(DT.kInt32, [4]))
    assert err.value.code == hc.StatusCode.kUnimplemented
    with pytest.raises(hc.StatusError) as err:
        hc.prepare(ctx, hc.Cast(DT.kUnknown), D(DT.kFloat32, [4]))
    assert err.value.code == hc.StatusCode.kInvalidArgument
    note("cast output over its own input is rejected (cast_test.cc:303-327)")
    storage = torch.zeros(64, dtype=torch.uint8, device=DEVICE)
    prepared = hc.prepare(ctx, hc.Cast(DT.kBFloat16), D(DT.kFloat16, [4]))
    assert not prepared.alias_support(0, 0)
    invocation = prepared.create_invocation()
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(hc.StatusError) as err:
        invocation.submit(stream, [storage.data_ptr()], [storage.data_ptr()])
    assert err.value.code == hc.StatusCode.kInvalidArgument
    with pytest.raises(hc.StatusError) as err:  # partial overlap: output starts inside the input
        invocation.submit(stream, [storage.data_ptr()], [storage.data_ptr() + 6])
    assert err.value.code == hc.StatusCode.kInvalidArgument
    invocation.submit(stream, [storage.data_ptr()], [storage.data_ptr() + 8])  # adjacent: fine
    torch.cuda.synchronize()
    note("zero elements: prepared, nothing to dispatch")
    empty = hc.prepare(ctx, hc.Cast(DT.kFloat32), D(DT.kBFloat16, [0, 7]))
    assert empty.dispatch_count() == 0
    assert empty.output_description() == D(DT.kFloat32, [0, 7])


@pytest.mark.parametrize("src,dst", PAIRS, ids=lambda k: k.name[1:])
def test_cast_every_pair_edge_counts_and_specials(src, dst):
    rng = np.random.default_rng(200 + int(src) * 16 + int(dst))
    for count in (1, 7, 8, 9, 63, 64, 65, 1000, 4099, 65536 + 13, 1 << 20):
        bits = specials(src, rng, count)
        note(f"cast {src.name} -> {dst.name}, {count} elements, dense")
        got = cast_on_device(src, dst, bits, [count])
        want = orc.cast(KINDS[src][0], KINDS[dst][0], bits, [count]).view(KINDS[dst][1])
        assert np.array_equal(got, want), f"{src.name}->{dst.name} n={count}"
    note(f"cast {src.name} -> {dst.name}: 2-D strided view (row pitch, every other element)")
    size = np.dtype(KINDS[src][1]).itemsize
    grid = specials(src, rng, 33 * 80).reshape(33, 80)
    got = cast_on_device(src, dst, grid, [33, 40], [80 * size, 2 * size])
    want = orc.cast(KINDS[src][0], KINDS[dst][0], grid, [33, 40], [80 * size, 2 * size]).view(KINDS[dst][1])
    assert np.array_equal(got, want)
    note(f"cast {src.name} -> {dst.name}: misaligned base pointer takes the element route")
    bits = specials(src, rng, 1000)
    padded = np.concatenate([np.zeros(1, bits.dtype), bits])
    data = device_bytes(padded)
    desc = hc.TensorDesc.dense(src, [1000])
    (out,) = run(hc.Copy() if src == dst else hc.Cast(dst), data[size:], descs=[desc])
    got = out.contiguous().view(torch.uint8).cpu().numpy().view(KINDS[dst][1])
    assert np.array_equal(got, orc.cast(KINDS[src][0], KINDS[dst][0], bits, [1000]).view(KINDS[dst][1]))


def test_cast_all_16_bit_patterns():
    halves = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    for src, dst in ((DT.kFloat16, DT.kBFloat16), (DT.kBFloat16, DT.kFloat16), (DT.kFloat16, DT.kFloat32),
                     (DT.kBFloat16, DT.kFloat32), (DT.kFloat16, DT.kBool), (DT.kBFloat16, DT.kBool)):
        note(f"cast all 65,536 {src.name} patterns -> {dst.name}")
        got = cast_on_device(src, dst, halves, [1 << 16])
        want = orc.cast(KINDS[src][0], KINDS[dst][0], halves, [1 << 16]).view(KINDS[dst][1])
        assert np.array_equal(got, want)


@pytest.mark.parametrize("kind", [DT.kFloat32, DT.kBFloat16, DT.kBool, DT.kInt8, DT.kUInt8, DT.kInt32], ids=lambda k: k.name[1:])
def test_copy_keeps_bytes_dense_strided_and_transposed(kind):
    size = {DT.kFloat32: 4, DT.kBFloat16: 2, DT.kBool: 1, DT.kInt8: 1, DT.kUInt8: 1, DT.kInt32: 4}[kind]
    rng = np.random.default_rng(300 + int(kind))
    for count in (1, 3, 15, 16, 17, 4099, 1 << 20):
        note(f"copy {kind.name} dense, {count} elements")
        raw = rng.integers(0, 256, count * size, dtype=np.uint16).astype(np.uint8)
        desc = hc.TensorDesc.dense(kind, [count])
        (out,) = run(hc.Copy(), device_bytes(raw), descs=[desc])
        assert np.array_equal(out.contiguous().view(torch.uint8).cpu().numpy().reshape(-1), raw)
    note(f"copy {kind.name}: transposed [64, 48] view of a [48, 64] array")
    raw = rng.integers(0, 256, 48 * 64 * size, dtype=np.uint16).astype(np.uint8)
    desc = hc.TensorDesc.strided_bytes(kind, [64, 48], [size, 64 * size])
    (out,) = run(hc.Copy(), device_bytes(raw), descs=[desc])
    want = np.ascontiguousarray(raw.reshape(48, 64, size).transpose(1, 0, 2)).reshape(-1)
    assert np.array_equal(out.contiguous().view(torch.uint8).cpu().numpy().reshape(-1), want)
    note(f"copy {kind.name}: broadcast row (zero stride) materialised")
    row = rng.integers(0, 256, 40 * size, dtype=np.uint16).astype(np.uint8)
    desc = hc.TensorDesc.strided_bytes(kind, [5, 40], [0, size])
    (out,) = run(hc.Copy(), device_bytes(row), descs=[desc])
    assert np.array_equal(out.contiguous().view(torch.uint8).cpu().numpy().reshape(5, -1), np.tile(row, (5, 1)))


def test_cast_benchmark_shapes_bit_exact():
    # the casts the Qwen graph wraps around every RMSNorm (src/compute_models: f32 <-> bf16 rows)
    rng = np.random.default_rng(400)
    x = rng.normal(0, 2, (8192, 2048)).astype(np.float32)
    note("cast f32 [8192, 2048] -> bf16")
    narrow = cast_on_device(DT.kFloat32, DT.kBFloat16, x, [8192, 2048])
    assert np.array_equal(narrow, orc.from_f32(orc.BF16, x))
    note("cast bf16 [8192, 2048] -> f32")
    wide = cast_on_device(DT.kBFloat16, DT.kFloat32, narrow, [8192, 2048])
    assert np.array_equal(wide, narrow.astype(np.uint32) << 16)
    note("copy bf16 [8192, 6144]: byte-identical")
    big = rng.integers(0, 1 << 16, (8192, 6144), dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(cast_on_device(DT.kBFloat16, DT.kBFloat16, big, [8192, 6144]), big)


@pytest.mark.parametrize("narrow", [DT.kBFloat16, DT.kFloat16])
def test_cast_norm_cast_is_one_narrow_rms_norm(narrow):
    """The decoder graph wraps every RMSNorm in two casts (src/compute_models/graph_builder.cc:492-499):
    narrow -> f32, RMSNorm with an f32 scale, f32 -> narrow.  RMSNorm over the narrow tensor with the
    same f32 scale is that chain in one launch: the widening is exact, the arithmetic is the same
    f32 arithmetic, and the one rounding at the end is the closing cast.  The two differ only in the
    order the row's squares are added (the kernels split a row over lanes differently), so: equal
    within one unit in the last place, and equal bit for bit nearly everywhere."""
    from gpu_support import assert_narrow_ulp
    torch_type = torch.bfloat16 if narrow == DT.kBFloat16 else torch.float16
    generator = torch.Generator(device="cpu").manual_seed(1900)
    for rows, width in ((8192, 2048), (33, 4096), (7, 1000)):
        x = (torch.randn(rows, width, generator=generator) * 3.0).to(torch_type).to(DEVICE)
        w = (1.0 + 0.1 * torch.randn(width, generator=generator)).to(DEVICE)
        note(f"cast + rms_norm + cast against one rms_norm, {narrow.name} [{rows}, {width}]")
        (wide,) = run(hc.Cast(DT.kFloat32), x)
        (normed,) = run(hc.RmsNorm(epsilon=1e-6), wide, w)
        (chain,) = run(hc.Cast(narrow), normed)
        (single,) = run(hc.RmsNorm(epsilon=1e-6), x, w)
        got = single.view(torch.int16).cpu().numpy().view(np.uint16)
        want = chain.view(torch.int16).cpu().numpy().view(np.uint16)
        differing = assert_narrow_ulp(got, want, "bf16" if narrow == DT.kBFloat16 else "f16")
        assert differing <= got.size // 1000
