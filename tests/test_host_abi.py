"""CPU-side checks of the drop-in boundary: the C ABI loads and exports what include/hyle_hip.h
declares, the schema (output inference) and the admission logic behave like the reference's,
and nothing here needs or touches a GPU.

Reference behaviour cited per case: src/compute_ops/operation.cc (inference),
src/compute_provider_native/*.cc and src/compute_provider_cuda/*_provider.cc (admission),
tests/compute/custom_kernel_test.cc (decline vs error at the provider boundary).
"""
from __future__ import annotations

import ctypes as C
import os
import re
import subprocess
import tempfile

import pytest

from hyle_amd import capi
from hyle_amd import compute as hc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hyle_hip.h")
DT = hc.DataType
D = hc.TensorDesc.dense
CTX = hc.Context.planning_only()


def test_library_exports_every_declared_symbol():
    text = "".join(open(os.path.join(ROOT, "include", name)).read()
                   for name in ("hyle_hip.h", "hyle_hip_stream.h", "hyle_hip_backend.h"))
    declared = set(re.findall(r"HYLE_HIP_API\s+[\w\s\*]+?\b(hyle_hip_\w+)\s*\(", text))
    assert declared, "no declarations parsed"
    lib = capi.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared but not exported"
    assert declared == set(capi.EXPORTS), (declared ^ set(capi.EXPORTS))
    assert lib.hyle_hip_abi_version() == capi.ABI_VERSION


def test_launch_shape_labels_are_listed_and_the_softmax_and_norm_tables_name_each_of_them():
    """The labels register themselves when the library loads (no device needed).  Every Softmax
    and norm launch shape compiled in must be a row of the table the GPU cases walk
    (tests/test_gpu_softmax_variants.py, tests/test_gpu_norm_variants.py), and the tables must name
    nothing the library lacks."""
    labels = hc.launch_variants()
    assert labels and len(set(labels)) == len(labels)
    assert capi.load().hyle_hip_variant_label(len(labels)) == b""
    assert hc.last_launch_variant() == ""  # nothing was launched on this thread
    import test_gpu_softmax_variants as table
    compiled = {label for label in labels if label.startswith("softmax")}
    tabled = {case[5] for case in table.CASES}
    assert compiled == tabled, (sorted(compiled - tabled), sorted(tabled - compiled))
    import test_gpu_norm_variants as norm_table
    compiled = {label for label in labels if label.startswith("norm")}
    tabled = {case[4] for case in norm_table.CASES}
    assert compiled == tabled, (sorted(compiled - tabled), sorted(tabled - compiled))


def test_header_is_plain_c_and_struct_layout_matches_ctypes():
    probe = r'''
#include <stdio.h>
#include <stddef.h>
#include "hyle_hip.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(hyle_hip_tensor_desc), offsetof(hyle_hip_tensor_desc, dims),
         offsetof(hyle_hip_tensor_desc, byte_strides), sizeof(hyle_hip_op_desc),
         offsetof(hyle_hip_op_desc, count), offsetof(hyle_hip_op_desc, input_count),
         offsetof(hyle_hip_op_desc, inputs));
  return 0;
}
'''
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.c")
        open(src, "w").write(probe)
        exe = os.path.join(tmp, "probe")
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.dirname(HEADER), src, "-o", exe],
                       check=True)
        got = [int(v) for v in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    want = [C.sizeof(capi.TensorDescC), capi.TensorDescC.dims.offset, capi.TensorDescC.byte_strides.offset,
            C.sizeof(capi.OpDescC), capi.OpDescC.count.offset, capi.OpDescC.input_count.offset,
            capi.OpDescC.inputs.offset]
    assert got == want


def test_no_device_here_is_reported_as_unavailable_not_hidden():
    try:
        import torch
        if torch.cuda.is_available():
            pytest.skip("a HIP device is present")
    except ImportError:
        pass
    with pytest.raises(hc.StatusError) as err:
        hc.Context.create(0)
    assert err.value.code == hc.StatusCode.kUnavailable


# ---------------------------------------------------------------- inference ----
def test_infer_binary_broadcast_and_type_rules():
    # src/compute_ops/operation.cc:249-278,480-490
    out = hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, [4096, 2048]), D(DT.kFloat32, [2048])])
    assert out == [D(DT.kFloat32, [4096, 2048])]
    out = hc.infer_output_descriptions(hc.Binary(), [D(DT.kBFloat16, [2, 1, 5]), D(DT.kBFloat16, [7, 1])])
    assert out == [D(DT.kBFloat16, [2, 7, 5])]
    assert hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, []), D(DT.kFloat32, [])]) == [D(DT.kFloat32, [])]
    assert hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, [0, 3]), D(DT.kFloat32, [1])])[0].byte_strides == (0, 0)
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, [2, 3]), D(DT.kFloat32, [4])])
    assert err.value.is_invalid_argument() and "cannot be broadcast" in err.value.message
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, [3]), D(DT.kBFloat16, [3])])
    assert err.value.is_invalid_argument() and "data types differ" in err.value.message
    with pytest.raises(hc.StatusError) as err:  # arity (operation.cc:1222-1225)
        hc.infer_output_descriptions(hc.Binary(), [D(DT.kFloat32, [3])])
    assert err.value.is_invalid_argument()
    chain = hc.infer_output_descriptions(hc.BinaryChain(), [D(DT.kFloat32, [8, 4]), D(DT.kFloat32, [4]), D(DT.kFloat32, [1])])
    assert chain == [D(DT.kFloat32, [8, 4])]


def test_infer_unary_gated_norm_rules():
    # src/compute_ops/operation.cc:1291-1305 (Unary), 1439-1469 (gated), 492-536 + 1395-1409 (norm)
    assert hc.infer_output_descriptions(hc.Unary(hc.UnaryKind.kSilu), [D(DT.kBFloat16, [3, 5])]) == [D(DT.kBFloat16, [3, 5])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Unary(hc.UnaryKind.kSilu), [D(DT.kInt32, [3])])
    assert err.value.is_invalid_argument()
    sep = hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate)
    assert hc.infer_output_descriptions(sep, [D(DT.kBFloat16, [8, 64]), D(DT.kBFloat16, [8, 64])]) == [D(DT.kBFloat16, [8, 64])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(sep, [D(DT.kBFloat16, [8, 64]), D(DT.kBFloat16, [8, 32])])
    assert "equal type and shape" in err.value.message
    packed = hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kPackedHalves)
    assert hc.infer_output_descriptions(packed, [D(DT.kFloat16, [4, 10])]) == [D(DT.kFloat16, [4, 5])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(packed, [D(DT.kFloat16, [4, 9])])
    assert "must be even" in err.value.message
    x = D(DT.kBFloat16, [8192, 2048])
    assert hc.infer_output_descriptions(hc.RmsNorm(1e-6), [x, D(DT.kBFloat16, [2048])]) == [x]
    assert hc.infer_output_descriptions(hc.RmsNorm(1e-6), [x, D(DT.kFloat32, [2048])]) == [x]  # promoted scale
    assert hc.infer_output_descriptions(hc.RmsNorm(1e-6), [x]) == [x]
    for bad_scale in (D(DT.kBFloat16, [2047]), D(DT.kBFloat16, [1, 2048]), D(DT.kFloat16, [2048])):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(hc.RmsNorm(), [x, bad_scale])
        assert "scale must match" in err.value.message
    with pytest.raises(hc.StatusError):  # f32 input does not take a narrow scale
        hc.infer_output_descriptions(hc.RmsNorm(), [D(DT.kFloat32, [4, 8]), D(DT.kBFloat16, [8])])
    for eps in (-1.0, float("inf"), float("nan")):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(hc.RmsNorm(epsilon=eps), [x])
        assert "epsilon" in err.value.message


def test_infer_softmax_reduce_topk_rules():
    # src/compute_ops/operation.cc:696-711,1593-1621 (softmax), 1345-1394 (reduce), 1622-1660 (TopK)
    s = D(DT.kFloat32, [32, 64, 64])
    boolean = hc.Softmax(mask=hc.MaskKind.kBoolean)
    assert hc.infer_output_descriptions(boolean, [s, D(DT.kBool, [64, 64])]) == [s]
    assert hc.infer_output_descriptions(boolean, [s, D(DT.kBool, [1, 64, 64])]) == [s]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(boolean, [s, D(DT.kFloat32, [64, 64])])
    assert "Bool data type" in err.value.message
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(boolean, [s, D(DT.kBool, [63, 64])])
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:  # a mask larger than the input is not a broadcast onto it
        hc.infer_output_descriptions(boolean, [D(DT.kFloat32, [1, 64]), D(DT.kBool, [5, 64])])
    assert "broadcast-compatible" in err.value.message
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Softmax(mask=hc.MaskKind.kAdditive), [s, D(DT.kBool, [64, 64])])
    assert "floating" in err.value.message
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Softmax(axis=3), [s])
    assert err.value.is_out_of_range()
    with pytest.raises(hc.StatusError):
        hc.infer_output_descriptions(hc.Softmax(scale=float("inf")), [s])
    with pytest.raises(hc.StatusError):  # mask supplied for a no-mask operation is an arity error
        hc.infer_output_descriptions(hc.Softmax(), [s, D(DT.kBool, [64, 64])])
    r = hc.Reduce(hc.ReductionKind.kMaximum, hc.Axes.from_([-1]))
    assert hc.infer_output_descriptions(r, [s]) == [D(DT.kFloat32, [32, 64])]
    keep = hc.Reduce(hc.ReductionKind.kSum, hc.Axes.from_([-1]), keep_dimensions=True)
    assert hc.infer_output_descriptions(keep, [s]) == [D(DT.kFloat32, [32, 64, 1])]
    logits = D(DT.kFloat32, [64, 151936])
    values, indices = hc.infer_output_descriptions(hc.TopK(), [logits])
    assert values == D(DT.kFloat32, [64, 1]) and indices == D(DT.kInt32, [64, 1])
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.TopK(count=151937), [logits])
    assert err.value.is_out_of_range()


def test_infer_q8_0_descriptor():
    # src/compute_ops/low_precision.cc:28-29,269-297: logical [K, N], 34-byte blocks on axis 0
    w = hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 2048, 6144)
    assert w.byte_strides == (34, 2176) and w.required_bytes() == 13369344
    out, sumsq = hc.infer_output_descriptions(hc.Q8_0DequantSumSquares(), [w])
    assert out == D(DT.kBFloat16, [6144, 2048]) and sumsq == D(DT.kFloat32, [6144])
    with pytest.raises(hc.StatusError):
        hc.infer_output_descriptions(hc.Q8_0DequantSumSquares(), [D(DT.kBFloat16, [2048, 6144])])
    with pytest.raises(hc.StatusError):
        hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 2047, 8)


def test_gguf_weight_descriptor_needs_whole_positive_blocks():
    # src/compute_ops/low_precision.cc:277-279: K and N positive, K a whole number of blocks -- so an
    # empty contraction (K = 0) never reaches a GGUF route
    for kind, per_block, block_bytes in ((hc.GgufQuantizedType.kQ8_0, 32, 34), (hc.GgufQuantizedType.kQ4K, 256, 144),
                                         (hc.GgufQuantizedType.kQ6K, 256, 210)):
        w = hc.TensorDesc.gguf_weight(kind, DT.kBFloat16, 4 * per_block, 3)
        assert w.byte_strides == (block_bytes, 4 * block_bytes)
        for k, n in ((0, 3), (4 * per_block, 0), (-per_block, 3), (per_block + 1, 3)):
            with pytest.raises(hc.StatusError) as err:
                hc.TensorDesc.gguf_weight(kind, DT.kBFloat16, k, n)
            assert err.value.is_invalid_argument()


# ---------------------------------------------------------------- admission ----
def test_routes_alias_support_and_cost_facts():
    a, b, s = D(DT.kFloat32, [4096, 2048]), D(DT.kFloat32, [2048]), D(DT.kFloat32, [1])
    fused = hc.prepare(CTX, hc.BinaryChain(), a, b, s)
    assert fused.route_name() == "elementwise-flat" and fused.dispatch_count() == 1
    assert fused.workspace_requirement().size == 0
    # only an input whose descriptor equals the output may alias it
    # (src/compute_provider_native/elementwise.cc:645-655)
    assert fused.alias_support(0, 0) and not fused.alias_support(0, 1) and not fused.alias_support(0, 2)
    same = hc.prepare(CTX, hc.Binary(), a, a)
    assert same.alias_support(0, 0) and same.alias_support(0, 1)
    column = hc.prepare(CTX, hc.Binary(), D(DT.kFloat32, [3, 1]), D(DT.kFloat32, [1, 5]))
    assert column.route_name() == "elementwise-strided"
    strided = hc.prepare(CTX, hc.Binary(), hc.TensorDesc.strided_bytes(DT.kFloat32, [6, 16], [160, 8]),
                         hc.TensorDesc.strided_bytes(DT.kFloat32, [6, 16], [0, 4]))
    assert strided.route_name() == "elementwise-strided" and not strided.alias_support(0, 0)
    norm = hc.prepare(CTX, hc.RmsNorm(1e-6), D(DT.kBFloat16, [8192, 2048]), D(DT.kBFloat16, [2048]))
    assert norm.route_name() == "norm-rows" and norm.alias_support(0, 0) and not norm.alias_support(0, 1)
    gated = hc.prepare(CTX, hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                       D(DT.kBFloat16, [8, 64]), D(DT.kBFloat16, [8, 64]))
    assert not gated.alias_support(0, 0)  # src/compute_provider_cuda/cuda_provider.cc:219-221
    for kind in hc.UnaryKind:  # every Unary kind is served for floating storage, in place allowed
        unary = hc.prepare(CTX, hc.Unary(kind), D(DT.kFloat16, [8, 64]))
        assert unary.route_name() == "elementwise-flat" and unary.alias_support(0, 0)
    for activation in hc.GatedActivationKind:
        for inputs, descs in ((hc.GatedInputKind.kSeparate, [D(DT.kBFloat16, [8, 64])] * 2),
                              (hc.GatedInputKind.kPackedHalves, [D(DT.kBFloat16, [8, 128])])):
            served = hc.prepare(CTX, hc.GatedActivation(activation, inputs), *descs)
            assert served.dispatch_count() == 1 and not served.alias_support(0, 0)
            assert served.output_description() == D(DT.kBFloat16, [8, 64])
    soft = hc.prepare(CTX, hc.Softmax(mask=hc.MaskKind.kBoolean), D(DT.kFloat32, [32, 64, 64]), D(DT.kBool, [64, 64]))
    assert soft.route_name() == "softmax-rows" and soft.alias_support(0, 0)
    topk = hc.prepare(CTX, hc.TopK(), D(DT.kFloat32, [64, 151936]))
    assert topk.route_name() == "argmax-tiles" and topk.dispatch_count() == 2
    need = topk.workspace_requirement()
    assert need.size == 64 * 16 * 8 and need.alignment == 16  # 16 tiles per row
    with pytest.raises(hc.StatusError) as err:  # workspace is the caller's to supply
        topk.create_invocation()
    assert err.value.is_invalid_argument()


def test_declines_are_unimplemented_and_errors_are_not():
    x = D(DT.kBFloat16, [4, 64])
    declines = [
        lambda: hc.prepare(CTX, hc.Unary(hc.UnaryKind.kAbs), D(DT.kInt32, [4])),   # integer Unary
        lambda: hc.prepare(CTX, hc.RmsNorm(accumulation_type=DT.kBFloat16), x),
        lambda: hc.prepare(CTX, hc.Softmax(accumulation_type=DT.kUnknown), x),   # half needs explicit f32
        lambda: hc.prepare(CTX, hc.Reduce(hc.ReductionKind.kSum, hc.Axes.from_([0])), x),   # half needs explicit f32
        lambda: hc.prepare(CTX, hc.TopK(count=2), D(DT.kUInt8, [4, 64])),          # TopK over bytes
        lambda: hc.prepare(CTX, hc.Binary(), D(DT.kInt32, [4]), D(DT.kInt32, [4])),
        lambda: hc.prepare(CTX, hc.LayerNorm(accumulation_type=DT.kFloat16), D(DT.kFloat16, [4, 64])),
        lambda: hc.prepare(CTX, hc.RmsNorm(), hc.TensorDesc.strided_bytes(DT.kBFloat16, [4, 64], [256, 2])),
    ]
    for attempt in declines:
        with pytest.raises(hc.StatusError) as err:
            attempt()
        assert err.value.is_unimplemented(), err.value
    with pytest.raises(hc.StatusError) as err:  # a wrong output descriptor is the caller's error
        hc.prepare(CTX, hc.Binary(), x, x, outputs=[D(DT.kBFloat16, [64, 4])])
    assert err.value.is_invalid_argument()
    assert hc.prepare(CTX, hc.Binary(), x, x, outputs=[x]).output_description() == x


def test_zero_elements_are_a_no_op_and_launch_needs_a_device():
    # src/compute_provider_native/elementwise.cc:222-223: success without touching storage
    empty = hc.prepare(CTX, hc.Binary(), D(DT.kFloat32, [0, 16]), D(DT.kFloat32, [16]))
    assert empty.route_name() == "no-op" and empty.dispatch_count() == 0
    empty.create_invocation().submit(0, [0, 0], [0])
    real = hc.prepare(CTX, hc.Binary(), D(DT.kFloat32, [4, 16]), D(DT.kFloat32, [16]))
    with pytest.raises(hc.StatusError) as err:
        real.create_invocation().submit(0, [16, 16], [32])
    assert err.value.is_failed_precondition()
    with pytest.raises(hc.StatusError) as err:  # binding count is checked first
        real.create_invocation().submit(0, [16], [32])
    assert err.value.is_invalid_argument()


def test_cast_and_copy_inference_and_admission():
    # src/compute_ops/operation.cc:1254-1285: dense output of the input's shape, Cast in the new type
    strided = hc.TensorDesc.strided_bytes(DT.kFloat16, [2, 2], [5, 2])
    assert hc.infer_output_descriptions(hc.Cast(DT.kFloat32), [strided]) == [D(DT.kFloat32, [2, 2])]
    assert hc.infer_output_descriptions(hc.Copy(), [strided]) == [D(DT.kFloat16, [2, 2])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Cast(DT.kUnknown), [D(DT.kFloat32, [4])])
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:  # blocked storage is Repack's business
        hc.infer_output_descriptions(hc.Copy(), [hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 64, 2)])
    assert err.value.is_unimplemented()
    # admitted pairs (src/compute_provider_native/cast.cc:127-176 plus the float pairs of the
    # mature providers); one dispatch, no workspace, no alias
    for src, dst in ((DT.kFloat32, DT.kBFloat16), (DT.kBFloat16, DT.kFloat32), (DT.kFloat16, DT.kBFloat16),
                     (DT.kInt32, DT.kFloat32), (DT.kBool, DT.kFloat16), (DT.kFloat32, DT.kBool)):
        prepared = hc.prepare(CTX, hc.Cast(dst), D(src, [8, 16]))
        assert prepared.route_name() == "cast-copy" and prepared.dispatch_count() == 1
        assert prepared.workspace_requirement().size == 0 and not prepared.alias_support(0, 0)
    assert hc.prepare(CTX, hc.Cast(DT.kFloat32), D(DT.kFloat32, [8])).route_name() == "cast-copy"  # = Copy
    assert hc.prepare(CTX, hc.Copy(), D(DT.kInt8, [3, 5])).dispatch_count() == 1
    for src, dst in ((DT.kFloat32, DT.kInt32), (DT.kInt32, DT.kBFloat16), (DT.kInt8, DT.kFloat32), (DT.kBool, DT.kInt32)):
        with pytest.raises(hc.StatusError) as err:
            hc.prepare(CTX, hc.Cast(dst), D(src, [8]))
        assert err.value.is_unimplemented()
    assert hc.prepare(CTX, hc.Copy(), D(DT.kFloat32, [0, 9])).dispatch_count() == 0


def test_fill_and_select_inference_and_admission():
    # src/compute_ops/operation.cc:1263-1275: Fill has no inputs; shape, type and scalar type must agree
    one = hc.ScalarValue.of(DT.kFloat32, 1.0)
    assert one.bits == 0x3F800000
    assert hc.infer_output_descriptions(hc.Fill((3, 5), DT.kFloat32, one), []) == [D(DT.kFloat32, [3, 5])]
    assert hc.infer_output_descriptions(hc.Fill((), DT.kBFloat16, hc.ScalarValue.from_bits(DT.kBFloat16, 0)), []) == [D(DT.kBFloat16, [])]
    for bad in (hc.Fill((3,), DT.kBFloat16, one), hc.Fill((3,), DT.kUnknown, hc.ScalarValue()), hc.Fill((-1,), DT.kFloat32, one)):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(bad, [])
        assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Fill((3,), DT.kFloat32, one), [D(DT.kFloat32, [3])])
    assert err.value.is_invalid_argument()
    prepared = hc.prepare(CTX, hc.Fill((9496, 4096), DT.kBFloat16, hc.ScalarValue.of(DT.kBFloat16, -1.0)))
    assert prepared.route_name() == "fill-pattern" and prepared.dispatch_count() == 1
    assert prepared.workspace_requirement().size == 0
    assert hc.prepare(CTX, hc.Fill((4, 0), DT.kInt32, hc.ScalarValue.of(DT.kInt32, 7))).dispatch_count() == 0
    # src/compute_ops/operation.cc:1309-1330: Bool condition, equal branch types, three-way broadcast
    assert hc.infer_output_descriptions(hc.Select(), [D(DT.kBool, [4, 1, 6]), D(DT.kInt8, [5, 6]), D(DT.kInt8, [4, 5, 1])]) \
        == [D(DT.kInt8, [4, 5, 6])]
    for bad in ([D(DT.kUInt8, [8]), D(DT.kFloat32, [8]), D(DT.kFloat32, [8])],
                [D(DT.kBool, [8]), D(DT.kFloat32, [8]), D(DT.kFloat16, [8])],
                [D(DT.kBool, [8]), D(DT.kFloat32, [3]), D(DT.kFloat32, [8])],
                [D(DT.kBool, [8]), D(DT.kFloat32, [8])]):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(hc.Select(), bad)
        assert err.value.is_invalid_argument()
    # a branch whose descriptor is the output's may be overwritten (tensor_provider.cc:190-194)
    prepared = hc.prepare(CTX, hc.Select(), D(DT.kBool, [8, 16]), D(DT.kFloat32, [8, 16]), D(DT.kFloat32, []))
    assert prepared.route_name() == "select" and prepared.dispatch_count() == 1
    assert [prepared.alias_support(0, i) for i in range(3)] == [False, True, False]
    with pytest.raises(hc.StatusError) as err:  # blocked storage is not plain
        hc.prepare(CTX, hc.Select(), D(DT.kBool, [64, 2]), hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 64, 2),
                   hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 64, 2))
    assert err.value.is_unimplemented()


def test_concat_inference_and_admission():
    # src/compute_ops/operation.cc:1516-1564
    assert hc.infer_output_descriptions(hc.Concat(1), [D(DT.kInt8, [2, 3, 5]), D(DT.kInt8, [2, 0, 5]), D(DT.kInt8, [2, 4, 5])]) \
        == [D(DT.kInt8, [2, 7, 5])]
    assert hc.infer_output_descriptions(hc.Concat(-1, total=40, start=8), [D(DT.kFloat32, [3, 8])]) == [D(DT.kFloat32, [3, 40])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Concat(2), [D(DT.kFloat32, [3, 8])])
    assert err.value.is_out_of_range()
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Concat(0), [D(DT.kFloat32, [3, 8]), D(DT.kFloat32, [3, 9])])
    assert err.value.is_invalid_argument()
    prepared = hc.prepare(CTX, hc.Concat(0), D(DT.kBFloat16, [8192, 2048]), D(DT.kBFloat16, [64, 2048]))
    assert prepared.route_name() == "concat" and prepared.dispatch_count() == 1 and prepared.workspace_requirement().size == 0
    assert hc.prepare(CTX, hc.Concat(0), D(DT.kBFloat16, [0, 2048]), D(DT.kBFloat16, [0, 2048])).dispatch_count() == 0
    with pytest.raises(hc.StatusError) as err:  # blocked storage is not plain
        hc.prepare(CTX, hc.Concat(0), hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 64, 2))
    assert err.value.is_unimplemented()


def test_gather_inference_and_admission():
    # src/compute_ops/operation.cc:616-637,1470-1489
    assert hc.infer_output_descriptions(hc.Gather(1), [D(DT.kFloat64, [2, 7, 3]), D(DT.kInt64, [2, 3])]) \
        == [D(DT.kFloat64, [2, 2, 3, 3])]
    assert hc.infer_output_descriptions(hc.Gather(-1), [D(DT.kBFloat16, [5, 9]), D(DT.kInt32, [])]) == [D(DT.kBFloat16, [5])]
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Gather(0), [D(DT.kFloat32, [4, 3]), D(DT.kFloat32, [2])])
    assert err.value.is_invalid_argument()   # indices must be Int32 or Int64
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.Gather(2), [D(DT.kFloat32, [4, 3]), D(DT.kInt32, [2])])
    assert err.value.is_out_of_range()
    with pytest.raises(hc.StatusError) as err:  # rank 5 - 1 + 5 > 8
        hc.infer_output_descriptions(hc.Gather(0), [D(DT.kFloat32, [2] * 5), D(DT.kInt32, [1] * 5)])
    assert err.value.is_invalid_argument()
    checked = hc.prepare(CTX, hc.Gather(0), D(DT.kBFloat16, [151936, 2048]), D(DT.kInt32, [20000]))
    assert checked.route_name() == "gather" and checked.dispatch_count() == 2
    large = hc.prepare(CTX, hc.Gather(0), D(DT.kBFloat16, [151936, 2048]), D(DT.kInt32, [8192]))   # checks inside the moving blocks
    assert large.dispatch_count() == 1 and large.workspace_requirement().size == checked.workspace_requirement().size
    assert 0 < checked.workspace_requirement().size <= 4096
    assert not checked.alias_support(0, 0) and not checked.alias_support(0, 1)
    few = hc.prepare(CTX, hc.Gather(0), D(DT.kBFloat16, [4096, 2048]), D(DT.kInt32, [8]))
    assert few.dispatch_count() == 1 and few.workspace_requirement().size == checked.workspace_requirement().size
    trusted = hc.prepare(CTX, hc.Gather(0, hc.IndexBoundsPolicy.kUnchecked), D(DT.kBFloat16, [151936, 2048]), D(DT.kInt32, [8192]))
    assert trusted.dispatch_count() == 1 and trusted.workspace_requirement().size == 0
    assert hc.prepare(CTX, hc.Gather(0), D(DT.kInt32, [4, 0]), D(DT.kInt32, [4])).dispatch_count() == 0
    with pytest.raises(hc.StatusError) as err:  # blocked storage is not plain
        hc.prepare(CTX, hc.Gather(0), hc.TensorDesc.gguf_q8_0_weight(DT.kBFloat16, 64, 2), D(DT.kInt32, [4]))
    assert err.value.is_unimplemented()


def test_every_scalar_type_is_storage_and_only_floats_are_arithmetic():
    # include/hyle/compute/providers/cuda.h:19-24: Copy / Fill / Select keep 1/2/4/8-byte storage,
    # arithmetic is FP32 / FP16 / BF16
    sizes = {DT.kBool: 1, DT.kFloat8E4M3FN: 1, DT.kFloat8E5M2: 1, DT.kInt8: 1, DT.kUInt8: 1, DT.kFloat16: 2, DT.kBFloat16: 2,
             DT.kInt16: 2, DT.kUInt16: 2, DT.kFloat32: 4, DT.kInt32: 4, DT.kUInt32: 4, DT.kFloat64: 8, DT.kInt64: 8, DT.kUInt64: 8}
    for kind, size in sizes.items():
        assert hc.data_type_size(kind) == size
        d = D(kind, [6, 10])
        assert d.byte_strides == (10 * size, size)
        assert hc.prepare(CTX, hc.Copy(), d).dispatch_count() == 1
        assert hc.prepare(CTX, hc.Copy(), hc.TensorDesc.strided_bytes(kind, [6, 10], [size, 6 * size + 1])).dispatch_count() == 1
        assert hc.prepare(CTX, hc.Fill((6, 10), kind, hc.ScalarValue.from_bits(kind, 1))).dispatch_count() == 1
        assert hc.prepare(CTX, hc.Select(), D(DT.kBool, [6, 10]), d, D(kind, [])).dispatch_count() == 1
        assert hc.prepare(CTX, hc.Concat(0), d, d).dispatch_count() == 1
        if kind not in (DT.kFloat16, DT.kBFloat16, DT.kFloat32):
            for operation in (hc.Binary(hc.BinaryKind.kAdd),):
                with pytest.raises(hc.StatusError) as err:
                    hc.prepare(CTX, operation, d, d)
                assert err.value.is_unimplemented()
            with pytest.raises(hc.StatusError) as err:   # the schema takes every float, the kernels three of them
                hc.prepare(CTX, hc.Softmax(), d)
            floating = kind in (DT.kFloat8E4M3FN, DT.kFloat8E5M2, DT.kFloat64)
            assert err.value.is_unimplemented() if floating else err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:   # bits wider than the element
        hc.prepare(CTX, hc.Fill((4,), DT.kUInt32, hc.ScalarValue.from_bits(DT.kUInt32, 1 << 32)))
    assert err.value.is_invalid_argument()
    assert hc.prepare(CTX, hc.Fill((4,), DT.kUInt64, hc.ScalarValue.from_bits(DT.kUInt64, (1 << 64) - 1))).dispatch_count() == 1


def test_sampling_inference_and_admission():
    # src/compute_ops/sampling_ops.cc:8-63
    U32 = DT.kUInt32
    assert hc.infer_output_descriptions(hc.RandomBits(17), [D(U32, [5, 4])]) == [D(U32, [5, 17])]
    assert hc.infer_output_descriptions(hc.RandomBits(0), [D(U32, [0, 4])]) == [D(U32, [0, 0])]
    for bad in (D(U32, [5, 3]), D(DT.kInt32, [5, 4]), D(U32, [20]), hc.TensorDesc.strided_bytes(U32, [5, 4], [32, 4])):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(hc.RandomBits(4), [bad])
        assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.RandomBits(1 << 31), [D(U32, [5, 4])])
    assert err.value.is_out_of_range()
    assert hc.infer_output_descriptions(hc.Categorical(), [D(DT.kBFloat16, [13, 17]), D(U32, [13, 4])]) == [D(DT.kInt32, [13])]
    assert hc.infer_output_descriptions(hc.Categorical(True), [D(DT.kFloat32, [13, 17]), D(U32, [13, 4])]) \
        == [D(DT.kInt32, [13]), D(DT.kFloat32, [13])]
    for logits, counters in ((D(DT.kFloat64, [13, 17]), D(U32, [13, 4])), (D(DT.kFloat32, [13, 17]), D(U32, [12, 4])),
                             (D(DT.kFloat32, [13, 0]), D(U32, [13, 4])), (D(DT.kFloat32, [13 * 17]), D(U32, [13, 4])),
                             (hc.TensorDesc.strided_bytes(DT.kFloat32, [13, 17], [128, 4]), D(U32, [13, 4]))):
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(hc.Categorical(), [logits, counters])
        assert err.value.is_invalid_argument()
    bits = hc.prepare(CTX, hc.RandomBits(4096), D(U32, [4096, 4]))
    assert bits.route_name() == "philox-words" and bits.dispatch_count() == 1 and bits.workspace_requirement().size == 0
    assert hc.prepare(CTX, hc.RandomBits(0), D(U32, [7, 4])).dispatch_count() == 0
    draw = hc.prepare(CTX, hc.Categorical(True), D(DT.kFloat32, [64, 151936]), D(U32, [64, 4]))
    assert draw.route_name() == "categorical-tiles" and draw.dispatch_count() == 2
    assert draw.workspace_requirement().size == 64 * 38 * 16 + 256    # a 16-byte record per tile of 4096, then the status word
    assert not draw.alias_support(0, 0) and not draw.alias_support(1, 0)
    assert hc.prepare(CTX, hc.Categorical(), D(DT.kFloat32, [0, 7]), D(U32, [0, 4])).dispatch_count() == 0


def test_rope_inference_and_admission():
    # src/compute_ops/operation.cc:639-696,1566-1574
    data, positions, frequencies = D(DT.kBFloat16, [1, 8192, 16, 128]), D(DT.kInt32, [8192]), D(DT.kFloat32, [64])
    rope = hc.RoPE(128, 1, hc.RopeLayout.kHalfSplit)
    assert hc.infer_output_descriptions(rope, [data, positions, frequencies]) == [data]
    assert hc.infer_output_descriptions(hc.RoPE(64, 1), [data, D(DT.kInt64, [1, 8192]), D(DT.kFloat32, [8192, 32])]) == [data]
    bad = [
        (hc.RoPE(0, 1), [data, positions, frequencies]), (hc.RoPE(3, 1), [data, positions, frequencies]),
        (hc.RoPE(130, 1), [data, positions, frequencies]), (hc.RoPE(128, 3), [data, positions, frequencies]),
        (rope, [data, D(DT.kInt32, [8191]), frequencies]), (rope, [data, D(DT.kInt32, [2, 8192]), frequencies]),
        (rope, [data, D(DT.kFloat32, [8192]), frequencies]), (rope, [data, positions, D(DT.kFloat32, [63])]),
        (rope, [data, positions, D(DT.kFloat32, [16, 64])]), (rope, [data, positions, D(DT.kInt32, [64])]),
        (rope, [D(DT.kBFloat16, [128]), positions, frequencies]),
    ]
    for operation, inputs in bad:
        with pytest.raises(hc.StatusError) as err:
            hc.infer_output_descriptions(operation, inputs)
        assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        hc.infer_output_descriptions(hc.RoPE(128, 7), [data, positions, frequencies])
    assert err.value.is_out_of_range()
    prepared = hc.prepare(CTX, rope, data, positions, frequencies)
    assert prepared.route_name() == "rope-rows" and prepared.dispatch_count() == 1 and prepared.workspace_requirement().size == 0
    assert prepared.alias_support(0, 0) and not prepared.alias_support(0, 1)
    for inputs in ([D(DT.kFloat64, [2, 3, 8]), D(DT.kInt32, [3]), D(DT.kFloat32, [2])],       # the schema's floats the kernels do not serve
                   [D(DT.kFloat32, [2, 3, 8]), D(DT.kInt32, [3]), D(DT.kBFloat16, [2])],
                   [hc.TensorDesc.strided_bytes(DT.kFloat32, [2, 3, 8], [128, 40, 4]), D(DT.kInt32, [3]), D(DT.kFloat32, [2])]):
        with pytest.raises(hc.StatusError) as err:
            hc.prepare(CTX, hc.RoPE(4, 1), *inputs)
        assert err.value.is_unimplemented()


def test_stream_abi_is_exported_and_validates_without_a_device():
    from hyle_amd import capi
    from hyle_amd import file_stream as fs
    lib = capi.load()
    for name in ("hyle_hip_copy_batch_submit", "hyle_hip_file_pipeline_create", "hyle_hip_file_pipeline_destroy",
                 "hyle_hip_file_pipeline_read", "hyle_hip_file_pipeline_wait"):
        assert hasattr(lib, name)
    with pytest.raises(hc.StatusError) as err:     # a planning-only context binds no device
        fs.FileResourcePipeline.create(CTX)
    assert err.value.is_invalid_argument()
    with pytest.raises(hc.StatusError) as err:
        fs.submit_copy_batch(CTX, [fs.CopyPhase()], [], 0)
    assert err.value.is_invalid_argument()


def test_backend_and_stream_calls_reject_bad_arguments_without_a_device():
    """include/hyle_hip_backend.h, include/hyle_hip_stream.h: argument errors are reported before
    anything touches a device."""
    lib = capi.load()
    count = C.c_size_t(99)
    assert lib.hyle_hip_backend_device_count(C.byref(count)) in (capi.OK, capi.UNAVAILABLE)
    assert lib.hyle_hip_backend_device_count(None) == capi.INVALID_ARGUMENT
    handle = C.c_void_p()
    assert lib.hyle_hip_memory_resource_create(None, 0, C.byref(handle)) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_queue_create(None, None, C.byref(handle)) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_queue_begin_sequence(None, C.byref(handle)) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_queue_copy_async(None, None, None, None, None, 16) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_completion_wait(None) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_file_pipeline_write(None, 0, None, 0, None, None) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_file_pipeline_submit_read(None, 0, None, 0, None, C.byref(handle)) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_stream_ticket_wait(None, None) == capi.INVALID_ARGUMENT
    lib.hyle_hip_stream_ticket_release(None)
    lib.hyle_hip_completion_release(None)
    assert lib.hyle_hip_status_name(capi.CANCELLED) == b"CANCELLED"
    # endpoints and transfer routes: a null queue has the invalid endpoint, which nobody may wait for
    endpoint = capi.CompletionEndpointC(1, 1)
    assert lib.hyle_hip_queue_completion_endpoint(None, C.byref(endpoint)) == capi.OK
    assert endpoint.authority is None and endpoint.identity is None
    assert lib.hyle_hip_queue_completion_endpoint(None, None) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_queue_can_wait_endpoint(None, endpoint) == 0
    route = capi.TransferPropertiesC()
    assert lib.hyle_hip_queue_transfer_properties(None, None, None, C.byref(route)) == capi.INVALID_ARGUMENT
    assert lib.hyle_hip_backend_same_device(10 ** 6, 10 ** 6) == 0
