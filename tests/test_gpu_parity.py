"""Parity of the gfx950 kernels (through the C ABI) with the CPU oracle.

Bars: bit-exact for f32 add/mul, bf16 residual add, argmax indices and Q8_0 dequant;
<= 1 unit in the last place for bf16/f16 outputs; 1e-5 relative for f32 RMSNorm, softmax,
sum of squares.  Layout follows the reference's provider tests
(tests/compute_provider_native/{elementwise,normalization,transformer}_test.cc,
tests/compute_provider_cuda/tensor_test.cc): known-answer cases first, then edge sizes
{0, 1, 127, 128, 129, ...}, then the benchmark shapes.
"""
from __future__ import annotations

import os

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from hyle_amd import workloads as wl
from oracle import lib as orc

from gpu_support import (DEVICE, TYPES, assert_bits_equal, assert_close_f32, assert_narrow_ulp, context,
                         host_values, note, run, to_device, to_host)

pytestmark = pytest.mark.gpu

BK = hc.BinaryKind
ORC_KIND = {BK.kAdd: orc.ADD, BK.kSubtract: orc.SUBTRACT, BK.kMultiply: orc.MULTIPLY,
            BK.kDivide: orc.DIVIDE, BK.kMinimum: orc.MINIMUM, BK.kMaximum: orc.MAXIMUM}


# ============================================================ Binary / chain ====
def test_binary_broadcast_known_answer():
    # tests/compute_provider_native/elementwise_test.cc:532-565
    note("binary KAT [2,3]+[3]")
    left = to_device(np.array([[1, 2, 3], [4, 5, 6]], np.float32), "f32")
    right = to_device(np.array([10, 20, 30], np.float32), "f32")
    (out,) = run(hc.Binary(BK.kAdd), left, right)
    assert to_host(out).tolist() == [[11, 22, 33], [14, 25, 36]]


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_binary_every_kind_dense_edge_counts(tag):
    # tests/compute_provider_native/elementwise_test.cc:480-530 (NaN, -0) and the half-storage
    # bit-exact expectation :365-373; counts from tests/compute_provider_cuda/tensor_test.cc:128-167
    oid = TYPES[tag][1]
    rng = np.random.default_rng(100)
    for count in (0, 1, 127, 128, 129, 257, 2048, 6144):
        x = rng.normal(0, 2, count).astype(np.float32)
        y = rng.normal(0, 2, count).astype(np.float32)
        if count >= 6:
            x[:6] = [-2.0, -0.0, 1.0, 4.0, 8.0, np.nan]
            y[:6] = [1.0, -3.0, 2.0, 0.5, -2.0, 7.0]
        xs, ys = host_values(x, tag), host_values(y, tag)
        for kind in BK:
            note(f"binary {tag} kind={kind.name} count={count}")
            (out,) = run(hc.Binary(kind), to_device(xs, tag), to_device(ys, tag))
            want = orc.binary(ORC_KIND[kind], oid, xs, ys)
            assert_bits_equal(to_host(out), want)


def test_config1_broadcast_add_then_scale_f32_bit_exact():
    note("cfg1 full shape (A[4096,2048] + b[2048]) * 0.5")
    a, b, s = wl.config1()
    da, db, ds = (to_device(v, "f32") for v in (a, b, s))
    (fused,) = run(hc.BinaryChain(BK.kAdd, BK.kMultiply), da, db, ds)
    want = (a + b) * np.float32(0.5)  # IEEE closed form: two roundings, no contraction
    assert_bits_equal(to_host(fused), want)
    # the same through two provider operations, as the reference schema expresses it
    (summed,) = run(hc.Binary(BK.kAdd), da, db)
    (scaled,) = run(hc.Binary(BK.kMultiply), summed, ds)
    assert_bits_equal(to_host(scaled), want)
    # and against the oracle on a slice (the oracle's generic walk is slow)
    rows = 64
    assert_bits_equal(to_host(fused)[:rows], orc.binary_chain(orc.ADD, orc.MULTIPLY, orc.F32, a[:rows], b, s))


def test_binary_broadcast_row_over_a_large_launch_bit_exact():
    """A[6000, 2048] + b[2048] f32: 98 MB of traffic with a periodic operand, above the size where
    the launcher changes from fat blocks to one vector per lane."""
    note("binary f32 [6000,2048] + [2048]")
    rng = np.random.default_rng(101)
    a = rng.normal(0, 1, (6000, 2048)).astype(np.float32)
    b = rng.uniform(-1, 1, 2048).astype(np.float32)
    (out,) = run(hc.Binary(BK.kAdd), to_device(a, "f32"), to_device(b, "f32"))
    assert hc.last_launch_variant() == "ew_flat/1x256"
    assert_bits_equal(to_host(out), a + b[None, :])


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_binary_chain_rounds_intermediate_to_storage(tag):
    oid = TYPES[tag][1]
    rng = np.random.default_rng(101)
    for shape_a, shape_b, shape_c in (((33, 136), (136,), (1,)), ((5, 24), (5, 24), (24,)), ((7, 129), (129,), ())):
        a = host_values(rng.normal(0, 1, shape_a).astype(np.float32), tag)
        b = host_values(rng.uniform(-1, 1, shape_b).astype(np.float32), tag)
        c = host_values(rng.uniform(0.25, 4, shape_c).astype(np.float32), tag)
        for first, second in ((BK.kAdd, BK.kMultiply), (BK.kMultiply, BK.kAdd), (BK.kSubtract, BK.kSubtract),
                              (BK.kDivide, BK.kMaximum)):
            note(f"chain {tag} {first.name}->{second.name} {shape_a} {shape_b} {shape_c}")
            (out,) = run(hc.BinaryChain(first, second), to_device(a, tag), to_device(b, tag), to_device(c, tag))
            want = orc.binary_chain(ORC_KIND[first], ORC_KIND[second], oid, a, b, c)
            assert_bits_equal(to_host(out), want)


def test_binary_general_broadcast_and_strides():
    rng = np.random.default_rng(102)
    note("binary [3,1] x [1,5], column broadcast")
    col = rng.normal(0, 1, (3, 1)).astype(np.float32)
    row = rng.normal(0, 1, (1, 5)).astype(np.float32)
    (out,) = run(hc.Binary(BK.kMultiply), to_device(col, "f32"), to_device(row, "f32"))
    assert_bits_equal(to_host(out), col * row)
    note("binary rank-4 mixed broadcast")
    x = rng.normal(0, 1, (2, 1, 7, 33)).astype(np.float32)
    y = rng.normal(0, 1, (3, 1, 33)).astype(np.float32)
    (out,) = run(hc.Binary(BK.kSubtract), to_device(x, "f32"), to_device(y, "f32"))
    assert_bits_equal(to_host(out), x - y)
    note("binary strided view + expanded (zero-stride) view")
    base = to_device(rng.normal(0, 1, (6, 40)).astype(np.float32), "f32")
    view = base[:, 3:35:2]                      # byte strides (160, 8)
    bias = to_device(rng.normal(0, 1, (1, 16)).astype(np.float32), "f32").expand(6, 16)  # strides (0, 4)
    (out,) = run(hc.Binary(BK.kAdd), view, bias)
    assert_bits_equal(to_host(out), to_host(view.contiguous()) + to_host(bias.contiguous()))
    note("binary scalar rank-0 operand")
    s = to_device(np.array(0.5, np.float32), "f32")
    (out,) = run(hc.Binary(BK.kMultiply), base, s)
    assert_bits_equal(to_host(out), to_host(base) * np.float32(0.5))


def test_config3_residual_add_in_place_bit_exact():
    note("cfg3 residual R[8192,2048] += Y bf16, output aliases input 0")
    r, y = wl.config3_residual()
    dr, dy = to_device(r, "bf16"), to_device(y, "bf16")
    want = orc.binary(orc.ADD, orc.BF16, r, y)
    run(hc.Binary(BK.kAdd), dr, dy, outputs=[dr])
    assert_bits_equal(to_host(dr), want)


def test_binary_alias_rules_and_alignment_errors():
    ctx = context()
    a = hc.TensorDesc.dense(hc.DataType.kFloat32, [8, 16])
    b = hc.TensorDesc.dense(hc.DataType.kFloat32, [16])
    prepared = hc.prepare(ctx, hc.Binary(BK.kAdd), a, b)
    # src/compute_provider_native/elementwise.cc:645-655: only a same-shape dense input may alias
    assert prepared.alias_support(0, 0) and not prepared.alias_support(0, 1)
    assert prepared.workspace_requirement().size == 0 and prepared.dispatch_count() == 1
    full = torch.zeros(8 * 16 + 4, dtype=torch.float32, device=DEVICE)
    row = torch.zeros(16, dtype=torch.float32, device=DEVICE)
    inv = prepared.create_invocation()
    stream = torch.cuda.current_stream().cuda_stream
    note("binary: a broadcast input aliasing the output is rejected before launch")
    with pytest.raises(hc.StatusError) as err:  # elementwise.cc:230-237
        inv.submit(stream, [row.data_ptr(), full.data_ptr()], [full.data_ptr()])
    assert err.value.is_invalid_argument()
    note("binary: misaligned operand is a failed precondition")
    with pytest.raises(hc.StatusError) as err:  # elementwise.cc:321-325
        inv.submit(stream, [full.data_ptr() + 2, row.data_ptr()], [full.data_ptr()])
    assert err.value.is_failed_precondition()
    note("binary: element-aligned (not 16-byte aligned) operands take the scalar route")
    rng = np.random.default_rng(103)
    x = rng.normal(0, 1, 8 * 16 + 4).astype(np.float32)
    dx = to_device(x, "f32")
    out = torch.zeros(8 * 16 + 4, dtype=torch.float32, device=DEVICE)
    inv.submit(stream, [dx.data_ptr() + 4, row.data_ptr()], [out.data_ptr() + 4])
    torch.cuda.synchronize()
    assert_bits_equal(to_host(out)[1:129], x[1:129])
    note("binary: zero elements never touch storage")
    empty = hc.prepare(ctx, hc.Binary(BK.kAdd), hc.TensorDesc.dense(hc.DataType.kFloat32, [0, 16]), b)
    assert empty.dispatch_count() == 0
    empty.create_invocation().submit(stream, [0, 0], [0])


# ============================================================ SiLU / SwiGLU ====
SPECIALS = np.array([-np.inf, -0.0, 0.0, np.inf, np.nan, -2.0, 88.0, -88.0, -103.0, -104.5, 20.0, -20.0, 1e-30],
                    np.float32)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_silu_and_swiglu_edge_counts_and_specials(tag):
    # tests/simd/math_test.cc:689-709 (ramp), 758-780 (specials), 1052-1097 (split gates)
    oid = TYPES[tag][1]
    rng = np.random.default_rng(104)
    for count in (0, 1, 7, 8, 9, 127, 129, 257, 2048, 6144):
        x = np.concatenate([SPECIALS, rng.normal(0, 3, count)]).astype(np.float32)[:count]
        if count >= 257:
            x[-257:] = -12.0 + 24.0 * np.arange(1, 258, dtype=np.float32) / np.float32(258)
        u = rng.normal(0, 2, count).astype(np.float32)
        xs, us = host_values(x, tag), host_values(u, tag)
        note(f"silu {tag} count={count}")
        (out,) = run(hc.Unary(hc.UnaryKind.kSilu), to_device(xs, tag))
        want = orc.silu(oid, xs)
        if tag == "f32":
            assert_close_f32(to_host(out), want, rel=1e-5, abs_floor=1e-37)
        else:
            assert_narrow_ulp(to_host(out), want, tag)
        note(f"swiglu separate {tag} count={count}")
        (out,) = run(hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                     to_device(xs, tag), to_device(us, tag))
        want = orc.swiglu(oid, xs, us)
        if tag == "f32":
            assert_close_f32(to_host(out), want, rel=1e-5, abs_floor=1e-37)
        else:
            assert_narrow_ulp(to_host(out), want, tag)


def test_silu_bf16_every_gate_pattern():
    note("silu bf16 over all 65536 bit patterns")
    gates = np.arange(65536, dtype=np.uint16)
    (out,) = run(hc.Unary(hc.UnaryKind.kSilu), to_device(gates, "bf16"))
    differing = assert_narrow_ulp(to_host(out), orc.silu(orc.BF16, gates), "bf16")
    assert differing < 65536 * 0.02  # the fast sigmoid flips a rounding only rarely
    note("swiglu bf16: every gate pattern times a spread of up values")
    ups = host_values(np.array([1.0, -3.5, 0.007, 1e20, -1e-20], np.float32), "bf16")
    for up in ups:
        u = np.full(65536, up, np.uint16)
        (out,) = run(hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                     to_device(gates, "bf16"), to_device(u, "bf16"))
        assert_narrow_ulp(to_host(out), orc.swiglu(orc.BF16, gates, u), "bf16")


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_swiglu_packed_halves(tag):
    # GatedInputKind::kPackedHalves: row = [gate | value] (include/hyle/compute/operation.h:362-365)
    oid = TYPES[tag][1]
    rng = np.random.default_rng(105)
    for rows, hidden in ((3, 8), (5, 129), (4, 2048)):
        note(f"swiglu packed {tag} rows={rows} hidden={hidden}")
        packed = host_values(rng.normal(0, 2, (rows, 2 * hidden)).astype(np.float32), tag)
        (out,) = run(hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kPackedHalves),
                     to_device(packed, tag))
        want = orc.swiglu_packed(oid, packed)
        if tag == "f32":
            assert_close_f32(to_host(out), want, rel=1e-5, abs_floor=1e-37)
        else:
            assert_narrow_ulp(to_host(out), want, tag)


def test_config3_swiglu_bf16_full_shape():
    note("cfg3 swiglu gate/up [8192,6144] bf16")
    gate, up = wl.config3_swiglu()
    (out,) = run(hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                 to_device(gate, "bf16"), to_device(up, "bf16"))
    differing = assert_narrow_ulp(to_host(out), orc.swiglu(orc.BF16, gate, up), "bf16")
    assert differing < gate.size * 0.01


# ================================================================ RMSNorm ====
@pytest.mark.parametrize("tag,weight_tag", [("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16"), ("f32", "f32")])
def test_rms_norm_domain_values_every_route(tag, weight_tag):
    # tests/compute_provider_native/normalization_test.cc:186-199 values; hidden set :315-323,
    # extended past the register-resident widths and to sizes that break 16-byte alignment
    oid, wid = TYPES[tag][1], TYPES[weight_tag][1]
    for hidden in (1, 8, 24, 127, 128, 129, 264, 1000, 2048, 4096, 8192, 16384, 20000):
        rows = 5
        idx = np.arange(rows * hidden)
        vals = np.where(idx // hidden == 1, 2.0, ((idx % 97) - 48) / 16.0).astype(np.float32).reshape(rows, hidden)
        scale = (1.001 + (np.arange(hidden) % 7) / 16.0).astype(np.float32)
        xs, ws = host_values(vals, tag), host_values(scale, weight_tag)
        for eps in (1e-5, 1e-6):
            note(f"rmsnorm {tag}/{weight_tag} hidden={hidden} eps={eps}")
            (out,) = run(hc.RmsNorm(epsilon=eps), to_device(xs, tag), to_device(ws, weight_tag))
            want = orc.rms_norm(oid, xs, ws, eps, weight_type=wid)
            if tag == "f32":
                assert_close_f32(to_host(out), want, rel=1e-5)
            else:
                assert_narrow_ulp(to_host(out), want, tag)
        note(f"rmsnorm {tag} hidden={hidden} without weight")
        (out,) = run(hc.RmsNorm(epsilon=1e-6), to_device(xs, tag))
        want = orc.rms_norm(oid, xs, None, 1e-6)
        if tag == "f32":
            assert_close_f32(to_host(out), want, rel=1e-5)
        else:
            assert_narrow_ulp(to_host(out), want, tag)


@pytest.mark.parametrize("tag,weight_tag", [("bf16", "bf16"), ("bf16", "f32"), ("f16", "f16"), ("f32", "f32")])
def test_rms_norm_launches_that_cover_the_tensor_exactly(tag, weight_tag):
    """Rows of 16 to 128 whole vectors in multiples of a block's rows, and an even number of rows of 64 n,
    128 n or 256 n vectors: the launch shapes that mask nothing, with and without the weight; one width past
    them and an odd row count take the masked shapes."""
    oid, wid = TYPES[tag][1], TYPES[weight_tag][1]
    rng = np.random.default_rng(77)
    per_vector = 4 if tag == "f32" else 8
    for rows, vectors in ((64, 16), (64, 32), (64, 64), (64, 128), (96, 64), (6, 192), (6, 320), (6, 384), (6, 448), (6, 512), (6, 576), (6, 640), (6, 768), (6, 896), (6, 1024), (6, 1280),
                          (6, 1536), (6, 1792), (6, 2048), (64, 512), (6, 2304), (7, 512)):
        hidden = vectors * per_vector
        vals = (rng.normal(0, 1, (rows, hidden)) * rng.uniform(0.1, 10, (rows, 1))).astype(np.float32)
        scale = rng.normal(1, 0.1, hidden).astype(np.float32)
        xs, ws = host_values(vals, tag), host_values(scale, weight_tag)
        note(f"rmsnorm {tag}/{weight_tag} [{rows}, {hidden}]: with and without weight")
        (out,) = run(hc.RmsNorm(epsilon=1e-6), to_device(xs, tag), to_device(ws, weight_tag))
        want = orc.rms_norm(oid, xs, ws, 1e-6, weight_type=wid)
        if tag == "f32":
            assert_close_f32(to_host(out), want, rel=1e-5)
        else:
            assert_narrow_ulp(to_host(out), want, tag)
        if tag == weight_tag:
            (out,) = run(hc.RmsNorm(epsilon=1e-6), to_device(xs, tag))
            want = orc.rms_norm(oid, xs, None, 1e-6)
            if tag == "f32":
                assert_close_f32(to_host(out), want, rel=1e-5)
            else:
                assert_narrow_ulp(to_host(out), want, tag)


def test_rms_norm_zero_rows_and_zero_hidden():
    for shape in ((0, 128), (4, 0)):
        note(f"rmsnorm empty {shape}")
        x = torch.empty(shape, dtype=torch.bfloat16, device=DEVICE)
        w = torch.empty(shape[1], dtype=torch.bfloat16, device=DEVICE)
        (out,) = run(hc.RmsNorm(), x, w)
        assert tuple(out.shape) == shape


def test_config2_rms_norm_bf16_full_and_decode_and_in_place():
    note("cfg2 rmsnorm X[8192,2048] bf16")
    x, w = wl.config2()
    dx, dw = to_device(x, "bf16"), to_device(w, "bf16")
    (out,) = run(hc.RmsNorm(epsilon=1e-6), dx, dw)
    want = orc.rms_norm(orc.BF16, x, w, 1e-6)
    differing = assert_narrow_ulp(to_host(out), want, "bf16")
    assert differing < x.size * 0.01
    # the reference provider's own accumulation order lands within the same bar
    assert_narrow_ulp(to_host(out), orc.rms_norm(orc.BF16, x, w, 1e-6, native=True), "bf16")
    note("cfg2 decode row [1,2048]")
    (row,) = run(hc.RmsNorm(epsilon=1e-6), dx[:1].contiguous(), dw)
    assert_narrow_ulp(to_host(row), want[:1], "bf16")
    note("cfg2 in place (output aliases input 0)")
    run(hc.RmsNorm(epsilon=1e-6), dx, dw, outputs=[dx])
    assert_bits_equal(to_host(dx), to_host(out))


# ================================================================ Softmax ====
def softmax_bar(got, want):
    # 1e-5 relative; results below the smallest normal f32 are compared absolutely
    assert_close_f32(got, want, rel=1e-5, abs_floor=1.2e-38)


def test_softmax_reference_known_answers():
    # tests/simd/math_test.cc:1268-1337
    for n in (1, 7, 8, 9, 257, 4096):
        note(f"softmax generator row n={n}")
        i = np.arange(n, dtype=np.float32)
        x = (np.sin(i * np.float32(0.7)) * np.float32(9.0) + np.cos(i * np.float32(0.13))).astype(np.float32)
        (out,) = run(hc.Softmax(), to_device(x[None, :], "f32"))
        got = to_host(out)[0]
        softmax_bar(got, orc.softmax_f32_row(x))
        assert abs(float(got.astype(np.float64).sum()) - 1.0) <= 2e-5
    inf = np.inf
    note("softmax masked / invalid rows")
    rows = np.array([[0.0, -inf, -1.0, -inf], [0.0, np.nan, -1.0, 2.0], [0.0, inf, -1.0, 2.0], [-inf] * 4], np.float32)
    (out,) = run(hc.Softmax(), to_device(rows, "f32"))
    got = to_host(out)
    assert got[0, 1] == 0.0 and got[0, 3] == 0.0 and abs(float(got[0, 0]) + float(got[0, 2]) - 1.0) <= 2e-6
    assert np.isnan(got[1:]).all()


def test_softmax_provider_known_answers_masks_scale_alias():
    # tests/compute_provider_native/transformer_test.cc:259-301
    note("softmax scale 0.5 + Bool mask [1,3], in place")
    vals = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    data = to_device(vals, "f32")
    mask = torch.tensor([[1, 0, 1]], dtype=torch.bool, device=DEVICE)
    op = hc.Softmax(axis=-1, scale=0.5, mask=hc.MaskKind.kBoolean)
    prepared = hc.prepare(context(), op, hc.TensorDesc.dense(hc.DataType.kFloat32, [2, 3]),
                          hc.TensorDesc.dense(hc.DataType.kBool, [1, 3]))
    assert prepared.alias_support(0, 0)
    run(op, data, mask, outputs=[data])
    want = orc.softmax(orc.F32, vals, scale=0.5, mask_kind=orc.MASK_BOOLEAN, mask=np.array([[1, 0, 1]], np.uint8))
    softmax_bar(to_host(data), want)
    assert to_host(data)[0, 1] == 0.0
    # tests/compute_provider_native/transformer_test.cc:337-387
    note("softmax additive mask with -inf, then all masked")
    add = np.array([[0, -np.inf, -1]], np.float32)
    (out,) = run(hc.Softmax(mask=hc.MaskKind.kAdditive), to_device(vals, "f32"), to_device(add, "f32"))
    softmax_bar(to_host(out), orc.softmax(orc.F32, vals, mask_kind=orc.MASK_ADDITIVE, mask=add))
    allm = np.full((1, 3), -np.inf, np.float32)
    (out,) = run(hc.Softmax(mask=hc.MaskKind.kAdditive), to_device(vals, "f32"), to_device(allm, "f32"))
    assert np.isnan(to_host(out)).all()


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_softmax_widths_masks_every_route(tag):
    oid = TYPES[tag][1]
    rng = np.random.default_rng(106)
    for heads, q, width in ((2, 3, 8), (1, 5, 24), (3, 16, 64), (2, 8, 136), (2, 16, 512), (4, 8, 1024),
                            (2, 8, 4096), (1, 4, 9000), (1, 3, 20000), (1, 2, 70000), (2, 3, 129)):
        x = host_values(rng.normal(0, 3, (heads, q, width)).astype(np.float32), tag)
        keep = (rng.random((q, width)) < 0.7).astype(np.uint8)
        keep[:, 0] = 1
        if q > 2:
            keep[2, :] = 0  # a fully masked row -> NaN for every head
        note(f"softmax {tag} {heads}x{q}x{width} no mask")
        (out,) = run(hc.Softmax(), to_device(x, tag))
        want = orc.softmax(oid, x)
        softmax_bar(to_host(out), want) if tag == "f32" else assert_narrow_ulp(to_host(out), want, tag)
        note(f"softmax {tag} {heads}x{q}x{width} Bool mask broadcast over heads, scale 0.125")
        dmask = torch.from_numpy(keep).to(DEVICE).view(torch.bool)
        (out,) = run(hc.Softmax(scale=0.125, mask=hc.MaskKind.kBoolean), to_device(x, tag), dmask)
        want = orc.softmax(oid, x, scale=0.125, mask_kind=orc.MASK_BOOLEAN, mask=keep)
        softmax_bar(to_host(out), want) if tag == "f32" else assert_narrow_ulp(to_host(out), want, tag)
        note(f"softmax {tag} {heads}x{q}x{width} additive mask [heads,1,width]")
        add = host_values(np.where(rng.random((heads, 1, width)) < 0.2, -np.inf, rng.normal(0, 1, (heads, 1, width))
                                   ).astype(np.float32), tag)
        add[..., 0] = 0
        (out,) = run(hc.Softmax(mask=hc.MaskKind.kAdditive), to_device(x, tag), to_device(add, tag))
        want = orc.softmax(oid, x, mask_kind=orc.MASK_ADDITIVE, mask=add)
        softmax_bar(to_host(out), want) if tag == "f32" else assert_narrow_ulp(to_host(out), want, tag)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_softmax_unmasked_launches_that_cover_the_tensor_exactly(tag):
    """Unmasked rows of every width that has a launch shape of its own (sub-wave groups with two vectors
    per lane and four rows, then 64, 128 or 256 lanes with three to eight vectors and two rows), 32 rows
    each; with a scale; a row with a NaN, one with +inf, one of -inf only (all three undefined: NaN) and
    one with -inf elements (zeros).  33 rows of one width take the masked shapes."""
    oid = TYPES[tag][1]
    rng = np.random.default_rng(107)
    per_vector = 4 if tag == "f32" else 8
    for rows, vectors in [(32, v) for v in (16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1280,
                                            1536, 1792, 2048)] + [(33, 512)]:
        width = vectors * per_vector
        values = rng.normal(0, 3, (rows, width)).astype(np.float32)
        values[3, 5] = np.nan
        values[4, width - 1] = np.inf
        values[5, :] = -np.inf
        values[6, ::3] = -np.inf
        x = host_values(values, tag)
        for scale in (1.0, 0.125):
            note(f"softmax {tag} [{rows}, {width}] unmasked, scale {scale}")
            (out,) = run(hc.Softmax(scale=scale), to_device(x, tag))
            want = orc.softmax(oid, x, scale=scale)
            decoded = want if tag == "f32" else orc.to_f32(oid, want)
            assert np.isnan(decoded[3:6]).all() and (decoded[6, ::3] == 0).all()
            softmax_bar(to_host(out), want) if tag == "f32" else assert_narrow_ulp(to_host(out), want, tag)


@pytest.mark.parametrize("log_form", [False, True])
@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_softmax_masked_launches_that_cover_the_tensor_exactly(tag, log_form):
    """[heads, 16, width] under a [16, width] mask, widths with a launch shape of their own: a staircase
    Boolean mask (whole vectors left out, one row left out entirely -> NaN) from 512 vectors per row on,
    an additive mask with -inf columns for every width; specials under and beside the mask."""
    oid = TYPES[tag][1]
    rng = np.random.default_rng(108)
    per_vector = 4 if tag == "f32" else 8
    kind = hc.SoftmaxKind.kLogSoftmax if log_form else hc.SoftmaxKind.kSoftmax
    for vectors in (16, 64, 128, 192, 256, 320, 512, 640, 768, 1024, 1536, 2048):
        heads, q, width = 2, 16, vectors * per_vector
        values = rng.normal(0, 3, (heads, q, width)).astype(np.float32)
        keep = (np.arange(width)[None, :] <= (np.arange(q)[:, None] + 1) * (width // q) - 3).astype(np.uint8)
        keep[5, :] = 0                                  # nothing kept: NaN for every head
        values[0, 7, width - 1] = np.nan               # under the mask: hidden
        values[1, 9, 0] = np.inf                       # kept: the row is undefined
        x = host_values(values, tag)
        note(f"softmax {tag} log={log_form} [{heads}, {q}, {width}] staircase Bool mask, scale 0.25")
        dmask = torch.from_numpy(keep).to(DEVICE).view(torch.bool)
        (out,) = run(hc.Softmax(scale=0.25, kind=kind, mask=hc.MaskKind.kBoolean), to_device(x, tag), dmask)
        want = orc.softmax(oid, x, scale=0.25, mask_kind=orc.MASK_BOOLEAN, mask=keep, log=log_form)
        got = to_host(out)
        if tag != "f32":
            assert_narrow_ulp(got, want, tag)
        elif log_form:
            assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
            ok = np.isfinite(want)
            assert np.all(np.abs(got[ok].astype(np.float64) - want[ok]) <= np.abs(want[ok]) * 4e-6 + 2e-7)
        else:
            softmax_bar(got, want)
        note(f"softmax {tag} log={log_form} [{heads}, {q}, {width}] additive mask [{q}, {width}] with -inf columns")
        add = np.where(rng.random((q, width)) < 0.3, -np.inf, rng.normal(0, 1, (q, width))).astype(np.float32)
        add[:, 1] = 0
        values[0, 7, width - 1] = 1.0
        values[1, 9, 0] = -2.0
        x = host_values(values, tag)
        addend = host_values(add, tag)
        (out,) = run(hc.Softmax(kind=kind, mask=hc.MaskKind.kAdditive), to_device(x, tag), to_device(addend, tag))
        want = orc.softmax(oid, x, mask_kind=orc.MASK_ADDITIVE, mask=addend, log=log_form)
        got = to_host(out)
        if tag != "f32":
            assert_narrow_ulp(got, want, tag)
        elif log_form:
            assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
            ok = np.isfinite(want)
            assert np.all(np.abs(got[ok].astype(np.float64) - want[ok]) <= np.abs(want[ok]) * 4e-6 + 2e-7)
        else:
            softmax_bar(got, want)


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_softmax_boolean_mask_hides_specials_additive_mask_does_not(tag):
    # A masked element is replaced by -inf before anything looks at it
    # (src/compute_provider_native/transformer.cc:44-57): NaN and +inf under a false mask byte
    # leave the row defined.  Under an additive -inf they still poison it (NaN + -inf, inf - inf).
    oid = TYPES[tag][1]
    rng = np.random.default_rng(110)
    for width in (24, 512, 4096, 9000):
        x = rng.normal(0, 3, (2, 6, width)).astype(np.float32)
        keep = np.ones((6, width), np.uint8)
        keep[:, width // 2:] = 0          # whole vectors masked: never loaded
        keep[:, 3] = 0                    # a masked element inside a loaded vector
        x[0, 0, width - 1] = np.nan
        x[0, 1, width // 2] = np.inf
        x[1, 2, 3] = np.nan
        x[1, 3, 3] = np.inf
        x[1, 4, 1] = np.nan               # unmasked: this row is undefined
        x = host_values(x, tag)
        note(f"softmax {tag} width {width}: specials under a Boolean mask")
        dmask = torch.from_numpy(keep).to(DEVICE).view(torch.bool)
        (out,) = run(hc.Softmax(mask=hc.MaskKind.kBoolean), to_device(x, tag), dmask)
        got = to_host(out)
        want = orc.softmax(oid, x, mask_kind=orc.MASK_BOOLEAN, mask=keep)
        softmax_bar(got, want) if tag == "f32" else assert_narrow_ulp(got, want, tag)
        as_f32 = got if tag == "f32" else orc.to_f32(oid, got)
        assert np.isnan(as_f32[1, 4]).all()
        assert not np.isnan(np.delete(as_f32.reshape(12, width), 10, axis=0)).any()
        note(f"softmax {tag} width {width}: the same specials under an additive mask")
        add = host_values(np.where(keep == 0, -np.inf, 0.0).astype(np.float32), tag)
        (out,) = run(hc.Softmax(mask=hc.MaskKind.kAdditive), to_device(x, tag), to_device(add, tag))
        got = to_host(out)
        want = orc.softmax(oid, x, mask_kind=orc.MASK_ADDITIVE, mask=add)
        softmax_bar(got, want) if tag == "f32" else assert_narrow_ulp(got, want, tag)
        as_f32 = got if tag == "f32" else orc.to_f32(oid, got)
        for h, q in ((0, 0), (0, 1), (1, 2), (1, 3), (1, 4)):
            assert np.isnan(as_f32[h, q]).all()


def test_softmax_subnormal_tail_and_wide_range():
    note("softmax f32 row spanning 160 units of range")
    rng = np.random.default_rng(107)
    x = rng.uniform(-120, 40, (4, 512)).astype(np.float32)
    (out,) = run(hc.Softmax(), to_device(x, "f32"))
    softmax_bar(to_host(out), orc.softmax(orc.F32, x))


def test_softmax_non_trailing_axis_and_strided_input():
    rng = np.random.default_rng(108)
    note("softmax over axis 1 of [2,9,5]")
    x = rng.normal(0, 2, (2, 9, 5)).astype(np.float32)
    (out,) = run(hc.Softmax(axis=1), to_device(x, "f32"))
    want = np.moveaxis(orc.softmax(orc.F32, np.ascontiguousarray(np.moveaxis(x, 1, -1))), -1, 1)
    softmax_bar(to_host(out), want)
    note("softmax over the last axis of a strided view")
    base = to_device(rng.normal(0, 2, (6, 80)).astype(np.float32), "f32")
    view = base[:, 8:72:2]
    (out,) = run(hc.Softmax(), view)
    softmax_bar(to_host(out), orc.softmax(orc.F32, to_host(view.contiguous())))


def test_config4_softmax_causal_slice_and_full_shape():
    note("cfg4 softmax slice S[4,256,256] with causal Bool mask")
    s, mask = wl.config4_softmax(heads=4, seq=256)
    dmask = torch.from_numpy(mask).to(DEVICE).view(torch.bool)
    (out,) = run(hc.Softmax(mask=hc.MaskKind.kBoolean), to_device(s, "f32"), dmask)
    softmax_bar(to_host(out), orc.softmax(orc.F32, s, mask_kind=orc.MASK_BOOLEAN, mask=mask))

    note("cfg4 softmax full shape S[32,4096,4096]: every row against the oracle, head by head")
    heads, seq = 32, 4096
    s, mask = wl.config4_softmax()  # the bytes bench.py and its CPU leg use
    big = torch.from_numpy(s).to(DEVICE)
    causal = torch.from_numpy(mask).to(DEVICE).view(torch.bool)
    (res,) = run(hc.Softmax(mask=hc.MaskKind.kBoolean), big, causal)
    # size-independent properties: rows sum to one, masked lanes are exactly zero
    sums = res.sum(dim=-1, dtype=torch.float64)
    assert float((sums - 1.0).abs().max()) <= 2e-5
    assert int(torch.count_nonzero(res.masked_select(~causal.expand(heads, seq, seq)))) == 0
    del big, sums
    threads = min(16, len(os.sched_getaffinity(0)))
    for h in range(heads):
        note(f"cfg4 softmax head {h}: 4096 rows against the oracle")
        want = orc.softmax_bool_f32_rows(s[h], mask, threads=threads)
        softmax_bar(to_host(res[h]), want)


# ======================================================== Reduce / argmax ====
@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_reduce_last_axis_row_max_and_sum(tag):
    # src/compute_provider_native/reduction.cc:24-47 (NaN propagates; identities +-inf)
    oid = TYPES[tag][1]
    rng = np.random.default_rng(110)
    kinds = {hc.ReductionKind.kMaximum: orc.MAX, hc.ReductionKind.kMinimum: orc.MIN,
             hc.ReductionKind.kSum: orc.SUM, hc.ReductionKind.kMean: orc.MEAN}
    for rows, width in ((3, 1), (5, 7), (4, 129), (9, 2048), (2, 4096), (2, 70001), (3, 0)):
        x = rng.normal(0, 2, (rows, width)).astype(np.float32)
        if width > 5:
            x[0, 3] = np.nan
            x[1, 2], x[1, 4] = 0.0, -0.0
        xs = host_values(x, tag)
        for kind, okind in kinds.items():
            note(f"reduce {tag} {kind.name} [{rows},{width}]")
            (out,) = run(hc.Reduce(kind, hc.Axes.from_([-1]), accumulation_type=hc.DataType.kFloat32), to_device(xs, tag))
            want = orc.reduce_last_axis(okind, oid, xs)
            got = to_host(out)
            if kind in (hc.ReductionKind.kMaximum, hc.ReductionKind.kMinimum):
                assert_bits_equal(got, want) if tag == "f32" else assert_narrow_ulp(got, want, tag, ulps=0)
            elif tag == "f32":
                # summation order is free in the reference (reduction_kernel.cu:92-116): compare
                # against a float64 sum with a bound that scales with the row's magnitude
                exact = np.sum(x.astype(np.float64), axis=1)
                exact = exact / width if (kind == hc.ReductionKind.kMean and width) else exact
                scale = np.sum(np.abs(x.astype(np.float64)), axis=1) / (width if kind == hc.ReductionKind.kMean and width else 1)
                ok = ~np.isnan(want)
                assert np.array_equal(np.isnan(got), np.isnan(want))
                assert np.all(np.abs(got[ok] - exact[ok]) <= 1e-5 * scale[ok] + 1e-30)
            else:
                assert np.array_equal(np.isnan(orc.to_f32(oid, got)), np.isnan(orc.to_f32(oid, want)))


def test_argmax_known_answers():
    # tests/simd/search_test.cc:166-213 data under the TopK ordering
    # (src/compute_provider_cuda/collectives.cu:478-495)
    note("argmax KAT 513 values, ties and NaN")
    data = np.full((3, 513), 4.0, np.float32)
    data[:, [9, 301]] = -17.0
    data[:, [13, 477]] = 29.0
    data[1, [71, 402]] = np.nan
    data[2, :] = np.nan
    data[2, 500] = -1e30
    values, indices = run(hc.TopK(), to_device(data, "f32"))
    assert to_host(indices)[:, 0].tolist() == [13, 13, 500]
    assert to_host(values)[:, 0].tolist() == [29.0, 29.0, np.float32(-1e30)]
    note("argmax signed zeros and all-NaN rows")
    z = np.zeros((3, 37), np.float32)
    z[0, [1, 19]] = -0.0
    z[1, :] = -0.0
    z[1, 30] = 0.0
    z[2, :] = np.nan
    values, indices = run(hc.TopK(), to_device(z, "f32"))
    assert to_host(indices)[:, 0].tolist() == [0, 0, 0]


@pytest.mark.parametrize("tag", ["f32", "bf16"])
def test_argmax_widths_against_oracle(tag):
    rng = np.random.default_rng(111)
    for rows, width in ((1, 1), (5, 7), (3, 1024), (2, 4097), (4, 20000), (1, 151936), (7, 33333)):
        note(f"argmax {tag} [{rows},{width}]")
        x = rng.integers(-50, 50, (rows, width)).astype(np.float32)  # many exact ties
        xs = host_values(x, tag)
        values, indices = run(hc.TopK(), to_device(xs, tag))
        xf = x if tag == "f32" else orc.to_f32(TYPES[tag][1], xs)
        want_values, want_indices = orc.topk1(xf)
        assert np.array_equal(to_host(indices)[:, 0], want_indices)
        got_values = to_host(values)[:, 0]
        got_values = got_values if tag == "f32" else orc.to_f32(TYPES[tag][1], got_values)
        assert np.array_equal(got_values, want_values)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_argmax_tiles_walked_in_several_steps(tag):
    """64 rows of 40000: sixteen tiles per row, each walked in more than one step with a ragged
    last step.  Rows of nothing but NaN, nothing but -inf, one number late among NaNs, one finite
    value among -inf, and exact ties across tiles take the full ordering as well as the fast one."""
    rng = np.random.default_rng(112)
    rows, width = 64, 40000
    x = rng.integers(-30, 30, (rows, width)).astype(np.float32)
    x[1, :] = np.nan
    x[2, :] = -np.inf
    x[3, :] = np.nan
    x[3, 39990] = -5.0
    x[4, :] = -np.inf
    x[4, 12345] = -60000.0         # finite in every storage type
    x[5, :] = 7.0                    # the same value everywhere: index 0
    x[6, :] = -np.inf
    x[6, 20000:] = np.nan            # -inf before NaN: index 0
    x[7, :] = np.nan
    x[7, 39999] = -np.inf            # a number (even -inf) beats every NaN
    note(f"argmax {tag} [{rows},{width}] special rows over walked tiles")
    xs = host_values(x, tag)
    values, indices = run(hc.TopK(), to_device(xs, tag))
    xf = x if tag == "f32" else orc.to_f32(TYPES[tag][1], xs)
    want_values, want_indices = orc.topk1(xf)
    assert np.array_equal(to_host(indices)[:, 0], want_indices)
    assert want_indices[[1, 2, 3, 4, 5, 6, 7]].tolist() == [0, 0, 39990, 12345, 0, 0, 39999]
    got_values = to_host(values)[:, 0]
    got_values = got_values if tag == "f32" else orc.to_f32(TYPES[tag][1], got_values)
    assert np.array_equal(got_values, want_values, equal_nan=True)


def test_config4_argmax_full_shape_bit_exact():
    note("cfg4 argmax logits[64,151936] with planted ties")
    logits = wl.config4_argmax()
    values, indices = run(hc.TopK(), to_device(logits, "f32"))
    want_values, want_indices = orc.topk1(logits)
    assert np.array_equal(to_host(indices)[:, 0], want_indices)
    assert_bits_equal(to_host(values)[:, 0], want_values)
    assert np.array_equal(want_indices, np.argmax(logits, axis=1).astype(np.int32))  # lowest index on ties


# =================================================================== Q8_0 ====
def q8_desc(k, n, stride=None):
    return hc.TensorDesc.gguf_q8_0_weight(hc.DataType.kBFloat16, k, n, stride)


def run_q8(blocks: np.ndarray, rows: int, k: int, stride=None):
    dev = torch.from_numpy(blocks).to(DEVICE)
    out, sumsq = run(hc.Q8_0DequantSumSquares(), dev, descs=[q8_desc(k, rows, stride)])
    return to_host(out), to_host(sumsq)


def test_config5_q8_0_full_and_decode_slice_bit_exact():
    for rows in (6144, 248):
        note(f"cfg5 q8_0 dequant rows={rows} k=2048")
        blocks = wl.config5(rows=rows)
        got, sumsq = run_q8(blocks, rows, 2048)
        want, want_sumsq, _ = orc.q8_0_dequant_bf16(blocks, rows, 2048)
        assert_bits_equal(got, want)
        assert_close_f32(sumsq, want_sumsq, rel=1e-5)


def test_q8_0_other_widths_strides_and_every_scale():
    rng = np.random.default_rng(112)
    for rows, k in ((1, 32), (3, 96), (5, 256), (7, 4096), (2, 8192), (3, 8192 + 256)):
        note(f"q8_0 rows={rows} k={k}")
        blocks = wl.config5(rows=rows, k=k, seed=int(rng.integers(1 << 30)))
        got, sumsq = run_q8(blocks, rows, k)
        want, want_sumsq, _ = orc.q8_0_dequant_bf16(blocks, rows, k)
        assert_bits_equal(got, want)
        assert_close_f32(sumsq, want_sumsq, rel=1e-5)
    note("q8_0 padded row stride")
    blocks = wl.config5(rows=9, k=512)
    padded = np.zeros((9, blocks.shape[1] + 48), np.uint8)
    padded[:, :blocks.shape[1]] = blocks
    got, _ = run_q8(padded, 9, 512, stride=padded.shape[1])
    assert_bits_equal(got, orc.q8_0_dequant_bf16(blocks, 9, 512)[0])
    note("q8_0 every finite fp16 scale against every quant value")
    scales = np.arange(65536, dtype=np.uint16)
    finite = (scales & 0x7C00) != 0x7C00
    scales = scales[finite]
    rows = scales.size
    blocks = np.empty((rows, 8, 34), np.uint8)      # k = 256: 8 blocks cover all 256 int8 values
    blocks[:, :, :2] = scales.view(np.uint8).reshape(rows, 1, 2)
    blocks[:, :, 2:] = np.arange(-128, 128, dtype=np.int8).view(np.uint8).reshape(1, 8, 32)
    blocks = blocks.reshape(rows, 8 * 34)
    got, _ = run_q8(blocks, rows, 256)
    assert_bits_equal(got, orc.q8_0_dequant_bf16(blocks, rows, 256)[0])
