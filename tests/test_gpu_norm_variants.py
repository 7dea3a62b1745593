"""Every launch shape of the RMSNorm / LayerNorm kernels is reached by a case here and checked
against the CPU oracle.

Which kernel serves a norm depends on the row width and on the number of rows: widths that a lane
group holds in whole vectors have launch shapes that cover the tensor exactly when the row count is
a multiple of the rows a block takes (norm_exact.h, and for LayerNorm the exact forms of norm.hip);
other widths and row counts take the masked shapes of norm.hip, and widths that are no whole
number of 16-byte vectors the generic kernel.  CASES is the table (operator, type, rows, width) ->
label of the launch shape the library must choose; `hyle_hip_last_launch_variant` reports the
shape actually launched.  The last test fails when a norm shape compiled into the library
(`hyle_hip_variant_label`) is reached by no case.

Semantics: src/compute_provider_native/normalization.cc:41-80 (RMSNorm),
src/simd/math/activations.cc:124-175 (LayerNorm); bars as in test_gpu_parity.py and
test_gpu_layer_norm.py.
"""
from __future__ import annotations

import numpy as np
import pytest

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import TYPES, assert_close_f32, assert_narrow_ulp, host_values, note, run, to_device, to_host
from test_gpu_layer_norm import layer_bar

pytestmark = pytest.mark.gpu

# (operator, type, rows, width, label)
CASES = [
    ("layer", "f32", 32, 32, "norm_rows/layer/8x1/256/1/exact"),
    ("layer", "f32", 3, 20, "norm_rows/layer/8x1/256/1/ragged"),
    ("layer", "f32", 16, 64, "norm_rows/layer/16x1/256/1/exact"),
    ("layer", "f32", 3, 52, "norm_rows/layer/16x1/256/1/ragged"),
    ("layer", "f32", 8, 128, "norm_rows/layer/32x1/256/1/exact"),
    ("layer", "f32", 3, 116, "norm_rows/layer/32x1/256/1/ragged"),
    ("layer", "f32", 4, 256, "norm_rows/layer/64x1/256/1/exact"),
    ("layer", "f32", 3, 244, "norm_rows/layer/64x1/256/1/ragged"),
    ("layer", "f32", 3, 500, "norm_rows/layer/64x2/256/2/ragged"),
    ("layer", "f32", 3, 768, "norm_rows/layer/64x4/64/2/ragged"),
    ("layer", "f32", 3, 1280, "norm_rows/layer/256x2/256/2/ragged"),
    ("layer", "f32", 3, 4096, "norm_rows/layer/256x4/256/1/exact"),
    ("layer", "f32", 3, 2304, "norm_rows/layer/256x4/256/1/ragged"),
    ("layer", "f32", 3, 8192, "norm_rows/layer/256x8/256/1/exact"),
    ("layer", "f32", 3, 5120, "norm_rows/layer/256x8/256/1/ragged"),
    ("layer", "f32", 3, 16384, "norm_rows/layer/1024x4/1024/1/exact"),
    ("layer", "f32", 3, 16372, "norm_rows/layer/1024x4/1024/1/ragged"),
    ("layer", "f32", 3, 32768, "norm_rows/layer/1024x8/1024/1/exact"),
    ("layer", "f32", 3, 32756, "norm_rows/layer/1024x8/1024/1/ragged"),
    ("layer", "f32", 3, 1027, "norm_generic/layer"),
    ("rms", "f32", 3, 20, "norm_rows/rms/8x1/256/1/ragged"),
    ("rms", "f32", 3, 52, "norm_rows/rms/16x1/256/1/ragged"),
    ("rms", "f32", 3, 116, "norm_rows/rms/32x1/256/1/ragged"),
    ("rms", "f32", 3, 244, "norm_rows/rms/64x1/256/1/ragged"),
    ("rms", "f32", 3, 500, "norm_rows/rms/64x2/256/2/ragged"),
    ("rms", "f32", 3, 768, "norm_rows/rms/64x4/256/2/ragged"),
    ("rms", "f32", 3, 1280, "norm_rows/rms/256x2/256/2/ragged"),
    ("rms", "f32", 3, 2304, "norm_rows/rms/256x4/256/1/ragged"),
    ("rms", "f32", 3, 5120, "norm_rows/rms/256x8/256/1/ragged"),
    ("rms", "f32", 3, 16372, "norm_rows/rms/1024x4/1024/1/ragged"),
    ("rms", "f32", 3, 32756, "norm_rows/rms/1024x8/1024/1/ragged"),
    ("rms", "f32", 3, 1027, "norm_generic/rms"),
    ("rms", "f32", 32, 64, "norm_rows_exact/rms/8x2/64/4"),
    ("rms", "f32", 16, 128, "norm_rows_exact/rms/16x2/64/4"),
    ("rms", "f32", 8, 256, "norm_rows_exact/rms/32x2/64/4"),
    ("rms", "f32", 4, 512, "norm_rows_exact/rms/64x2/64/4"),
    ("rms", "f32", 4, 768, "norm_rows_exact/rms/64x3/64/2"),
    ("rms", "f32", 4, 1280, "norm_rows_exact/rms/64x5/64/2"),
    ("rms", "f32", 4, 1536, "norm_rows_exact/rms/64x6/64/2"),
    ("rms", "f32", 4, 1792, "norm_rows_exact/rms/64x7/64/2"),
    ("rms", "f32", 4, 2048, "norm_rows_exact/rms/64x8/64/2"),
    ("rms", "f32", 4, 2304, "norm_rows_exact/rms/64x9/64/2"),
    ("rms", "f32", 4, 2560, "norm_rows_exact/rms/64x10/64/2"),
    ("rms", "f32", 4, 3072, "norm_rows_exact/rms/64x12/64/2"),
    ("rms", "f32", 4, 3584, "norm_rows_exact/rms/128x7/128/2"),
    ("rms", "f32", 4, 4096, "norm_rows_exact/rms/128x8/128/2"),
    ("rms", "f32", 4, 5120, "norm_rows_exact/rms/256x5/256/2"),
    ("rms", "f32", 4, 6144, "norm_rows_exact/rms/256x6/256/2"),
    ("rms", "f32", 4, 7168, "norm_rows_exact/rms/256x7/256/2"),
    ("rms", "f32", 4, 8192, "norm_rows_exact/rms/256x8/256/2"),
    ("layer", "f32", 32, 64, "norm_rows_exact/layer/8x2/64/4"),
    ("layer", "f32", 16, 128, "norm_rows_exact/layer/16x2/64/4"),
    ("layer", "f32", 8, 256, "norm_rows_exact/layer/32x2/64/4"),
    ("layer", "f32", 4, 512, "norm_rows_exact/layer/64x2/64/4"),
    ("layer", "f32", 4, 768, "norm_rows_exact/layer/64x3/64/2"),
    ("layer", "f32", 4, 1024, "norm_rows_exact/layer/64x4/64/2"),
    ("layer", "f32", 4, 1280, "norm_rows_exact/layer/64x5/64/2"),
    ("layer", "f32", 4, 1536, "norm_rows_exact/layer/64x6/64/2"),
    ("layer", "f32", 4, 1792, "norm_rows_exact/layer/64x7/64/2"),
    ("layer", "f32", 4, 2048, "norm_rows_exact/layer/64x8/64/2"),
    ("layer", "f32", 4, 2304, "norm_rows_exact/layer/64x9/64/2"),
    ("layer", "f32", 4, 2560, "norm_rows_exact/layer/64x10/64/2"),
    ("layer", "f32", 4, 3072, "norm_rows_exact/layer/64x12/64/2"),
    ("layer", "f32", 4, 3584, "norm_rows_exact/layer/128x7/128/2"),
    ("layer", "f32", 4, 4096, "norm_rows_exact/layer/128x8/128/2"),
    ("layer", "f32", 4, 5120, "norm_rows_exact/layer/256x5/256/2"),
    ("layer", "f32", 4, 6144, "norm_rows_exact/layer/256x6/256/2"),
    ("layer", "f32", 4, 7168, "norm_rows_exact/layer/256x7/256/2"),
    ("layer", "f32", 4, 8192, "norm_rows_exact/layer/256x8/256/2"),
    ("layer", "bf16", 32, 64, "norm_rows/layer/8x1/256/1/exact"),
    ("layer", "bf16", 3, 40, "norm_rows/layer/8x1/256/1/ragged"),
    ("layer", "bf16", 16, 128, "norm_rows/layer/16x1/256/1/exact"),
    ("layer", "bf16", 3, 104, "norm_rows/layer/16x1/256/1/ragged"),
    ("layer", "bf16", 8, 256, "norm_rows/layer/32x1/256/1/exact"),
    ("layer", "bf16", 3, 232, "norm_rows/layer/32x1/256/1/ragged"),
    ("layer", "bf16", 4, 512, "norm_rows/layer/64x1/256/1/exact"),
    ("layer", "bf16", 3, 488, "norm_rows/layer/64x1/256/1/ragged"),
    ("layer", "bf16", 3, 1000, "norm_rows/layer/64x2/256/2/ragged"),
    ("layer", "bf16", 3, 1536, "norm_rows/layer/64x4/64/2/ragged"),
    ("layer", "bf16", 3, 2560, "norm_rows/layer/256x2/256/2/ragged"),
    ("layer", "bf16", 3, 8192, "norm_rows/layer/256x4/256/1/exact"),
    ("layer", "bf16", 3, 4608, "norm_rows/layer/256x4/256/1/ragged"),
    ("layer", "bf16", 3, 16384, "norm_rows/layer/256x8/256/1/exact"),
    ("layer", "bf16", 3, 10240, "norm_rows/layer/256x8/256/1/ragged"),
    ("layer", "bf16", 3, 32768, "norm_rows/layer/1024x4/1024/1/exact"),
    ("layer", "bf16", 3, 32744, "norm_rows/layer/1024x4/1024/1/ragged"),
    ("layer", "bf16", 3, 65536, "norm_rows/layer/1024x8/1024/1/exact"),
    ("layer", "bf16", 3, 65512, "norm_rows/layer/1024x8/1024/1/ragged"),
    ("layer", "bf16", 3, 1027, "norm_generic/layer"),
    ("rms", "bf16", 3, 40, "norm_rows/rms/8x1/256/1/ragged"),
    ("rms", "bf16", 3, 104, "norm_rows/rms/16x1/256/1/ragged"),
    ("rms", "bf16", 3, 232, "norm_rows/rms/32x1/256/1/ragged"),
    ("rms", "bf16", 3, 488, "norm_rows/rms/64x1/256/1/ragged"),
    ("rms", "bf16", 3, 1000, "norm_rows/rms/64x2/256/2/ragged"),
    ("rms", "bf16", 3, 1536, "norm_rows/rms/64x4/256/2/ragged"),
    ("rms", "bf16", 3, 2560, "norm_rows/rms/256x2/256/2/ragged"),
    ("rms", "bf16", 3, 4608, "norm_rows/rms/256x4/256/1/ragged"),
    ("rms", "bf16", 3, 10240, "norm_rows/rms/256x8/256/1/ragged"),
    ("rms", "bf16", 3, 32744, "norm_rows/rms/1024x4/1024/1/ragged"),
    ("rms", "bf16", 3, 65512, "norm_rows/rms/1024x8/1024/1/ragged"),
    ("rms", "bf16", 3, 1027, "norm_generic/rms"),
    ("rms", "bf16", 32, 128, "norm_rows_exact/rms/8x2/64/4"),
    ("rms", "bf16", 16, 256, "norm_rows_exact/rms/16x2/64/4"),
    ("rms", "bf16", 8, 512, "norm_rows_exact/rms/32x2/64/4"),
    ("rms", "bf16", 4, 1024, "norm_rows_exact/rms/64x2/64/4"),
    ("rms", "bf16", 4, 1536, "norm_rows_exact/rms/64x3/64/2"),
    ("rms", "bf16", 4, 2560, "norm_rows_exact/rms/64x5/64/2"),
    ("rms", "bf16", 4, 3072, "norm_rows_exact/rms/64x6/64/2"),
    ("rms", "bf16", 4, 3584, "norm_rows_exact/rms/64x7/64/2"),
    ("rms", "bf16", 4, 4096, "norm_rows_exact/rms/64x8/64/2"),
    ("rms", "bf16", 4, 4608, "norm_rows_exact/rms/64x9/64/2"),
    ("rms", "bf16", 4, 5120, "norm_rows_exact/rms/64x10/64/2"),
    ("rms", "bf16", 4, 6144, "norm_rows_exact/rms/64x12/64/2"),
    ("rms", "bf16", 4, 7168, "norm_rows_exact/rms/128x7/128/2"),
    ("rms", "bf16", 4, 8192, "norm_rows_exact/rms/128x8/128/2"),
    ("rms", "bf16", 4, 10240, "norm_rows_exact/rms/256x5/256/2"),
    ("rms", "bf16", 4, 12288, "norm_rows_exact/rms/256x6/256/2"),
    ("rms", "bf16", 4, 14336, "norm_rows_exact/rms/256x7/256/2"),
    ("rms", "bf16", 4, 16384, "norm_rows_exact/rms/256x8/256/2"),
    ("layer", "bf16", 32, 128, "norm_rows_exact/layer/8x2/64/4"),
    ("layer", "bf16", 16, 256, "norm_rows_exact/layer/16x2/64/4"),
    ("layer", "bf16", 8, 512, "norm_rows_exact/layer/32x2/64/4"),
    ("layer", "bf16", 4, 1024, "norm_rows_exact/layer/64x2/64/4"),
    ("layer", "bf16", 4, 1536, "norm_rows_exact/layer/64x3/64/2"),
    ("layer", "bf16", 4, 2048, "norm_rows_exact/layer/64x4/64/2"),
    ("layer", "bf16", 4, 2560, "norm_rows_exact/layer/64x5/64/2"),
    ("layer", "bf16", 4, 3072, "norm_rows_exact/layer/64x6/64/2"),
    ("layer", "bf16", 4, 3584, "norm_rows_exact/layer/64x7/64/2"),
    ("layer", "bf16", 4, 4096, "norm_rows_exact/layer/64x8/64/2"),
    ("layer", "bf16", 4, 4608, "norm_rows_exact/layer/64x9/64/2"),
    ("layer", "bf16", 4, 5120, "norm_rows_exact/layer/64x10/64/2"),
    ("layer", "bf16", 4, 6144, "norm_rows_exact/layer/64x12/64/2"),
    ("layer", "bf16", 4, 7168, "norm_rows_exact/layer/128x7/128/2"),
    ("layer", "bf16", 4, 8192, "norm_rows_exact/layer/128x8/128/2"),
    ("layer", "bf16", 4, 10240, "norm_rows_exact/layer/256x5/256/2"),
    ("layer", "bf16", 4, 12288, "norm_rows_exact/layer/256x6/256/2"),
    ("layer", "bf16", 4, 14336, "norm_rows_exact/layer/256x7/256/2"),
    ("layer", "bf16", 4, 16384, "norm_rows_exact/layer/256x8/256/2"),
]

reached = set()


def run_case(operator, tag, weight_tag, rows, width, label, parameters, seed):
    """parameters: 0 none, 1 scale, 2 scale and bias (LayerNorm only)."""
    oid, wid = TYPES[tag][1], TYPES[weight_tag][1]
    rng = np.random.default_rng(seed)
    values = (rng.normal(0, 1, (rows, width)) * rng.uniform(0.1, 10, (rows, 1))).astype(np.float32)
    if rows > 1 and operator == "rms":
        values[1] = 2.0   # a constant row (tests/compute_provider_native/normalization_test.cc:186-199)
    xs = host_values(values, tag)
    scale = host_values(rng.normal(1, 0.1, width).astype(np.float32), weight_tag)
    bias = host_values(rng.normal(0, 0.5, width).astype(np.float32), weight_tag)
    note(f"{operator} norm {tag}/{weight_tag} [{rows}, {width}] parameters={parameters}: expecting {label}")
    operands = [to_device(xs, tag)]
    if parameters >= 1:
        operands.append(to_device(scale, weight_tag))
    if parameters == 2:
        operands.append(to_device(bias, weight_tag))
    if operator == "rms":
        (out,) = run(hc.RmsNorm(epsilon=1e-6), *operands)
        want = orc.rms_norm(oid, xs, scale if parameters else None, 1e-6, weight_type=wid if parameters else None)
    else:
        (out,) = run(hc.LayerNorm(epsilon=1e-5), *operands)
        want = orc.layer_norm(oid, xs, scale if parameters else None, bias if parameters == 2 else None, 1e-5,
                              param_type=wid if parameters else None)
    chosen = hc.last_launch_variant()
    assert chosen == label, f"{operator} [{rows}, {width}] {tag}: launched {chosen}, the table says {label}"
    reached.add(chosen)
    got = to_host(out)
    if operator == "layer":
        layer_bar(got, want, tag, bias if parameters == 2 else None)
    elif tag == "f32":
        assert_close_f32(got, want, rel=1e-5)
    else:
        assert_narrow_ulp(got, want, tag)


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}-{c[1]}-{c[2]}x{c[3]}")
def test_norm_case_reaches_its_launch_shape_and_matches_the_oracle(case):
    operator, tag, rows, width, label = case
    seed = 3000 + CASES.index(case)
    for parameters in ((0, 1) if operator == "rms" else (0, 1, 2)):
        run_case(operator, tag, tag, rows, width, label, parameters, seed + parameters)
    if tag == "bf16":   # f32 parameters under narrow storage (the cast + norm + cast of the decoder graph), and f16
        run_case(operator, "bf16", "f32", rows, width, label, 2 if operator == "layer" else 1, seed + 7)
        run_case(operator, "f16", "f16", rows, width, label, 1, seed + 8)


def test_every_norm_launch_shape_in_the_library_is_reached():
    """Runs after the cases above (file order): a norm launch shape compiled into the library that no
    case reached is either dead code or an untested kernel."""
    compiled = {label for label in hc.launch_variants() if label.startswith("norm")}
    tabled = {case[4] for case in CASES}
    assert compiled == tabled, f"not in the table: {sorted(compiled - tabled)}; not in the library: {sorted(tabled - compiled)}"
    if reached:
        assert tabled <= reached, f"tabled but not reached: {sorted(tabled - reached)}"
