"""Every launch shape of the Softmax / LogSoftmax kernels is reached by a case here and checked
against the CPU oracle.

Which kernel serves a Softmax depends on the row width, the number of rows, the mask form and the
size of the launch (launches of 64 MiB and more under a mask, or of more than 2^27 elements, leave
the shapes of softmax_exact.hip for the large-launch kernels of softmax.hip, and an additive mask
that repeats over leading axes is then steered by XCD: rows are permuted over the blocks).  CASES
is the table (type, heads, q, width, mask form) -> label of the launch shape the library must
choose; `hyle_hip_last_launch_variant` reports the shape actually launched.  The last test fails
when a Softmax shape compiled into the library (`hyle_hip_variant_label`) is reached by no case.

Semantics: src/compute_provider_native/transformer.cc:44-57,165-191 (scale, masks, the undefined
row); bars as in test_gpu_parity.py (f32 1e-5 relative, narrow types 1 unit in the last place,
LogSoftmax f32 at the reference's own 4e-6 relative + 2e-7,
tests/compute_provider_cuda/tensor_test.cc:1168-1199).
"""
from __future__ import annotations

import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from oracle import lib as orc

from gpu_support import DEVICE, TYPES, note, run

pytestmark = pytest.mark.gpu

# (type, heads, q, width, mask form, label): x is [heads, q, width], the mask [q, width] is shared
# by the heads.
CASES = [
    ("bf16", 2, 16, 64, "boolean", "softmax_rows/8x1/256/boolean/exact"),
    ("bf16", 2, 8, 40, "boolean", "softmax_rows/8x1/256/boolean/ragged"),
    ("bf16", 2, 16, 64, "additive", "softmax_rows/8x1/256/additive/exact"),
    ("bf16", 2, 8, 40, "additive", "softmax_rows/8x1/256/additive/ragged"),
    ("bf16", 2, 16, 64, "unmasked", "softmax_rows/8x1/256/unmasked/exact"),
    ("bf16", 2, 8, 40, "unmasked", "softmax_rows/8x1/256/unmasked/ragged"),
    ("bf16", 2, 8, 128, "boolean", "softmax_rows/16x1/256/boolean/exact"),
    ("bf16", 2, 8, 104, "boolean", "softmax_rows/16x1/256/boolean/ragged"),
    ("bf16", 2, 8, 128, "additive", "softmax_rows/16x1/256/additive/exact"),
    ("bf16", 2, 8, 104, "additive", "softmax_rows/16x1/256/additive/ragged"),
    ("bf16", 2, 8, 128, "unmasked", "softmax_rows/16x1/256/unmasked/exact"),
    ("bf16", 2, 8, 104, "unmasked", "softmax_rows/16x1/256/unmasked/ragged"),
    ("bf16", 2, 8, 256, "boolean", "softmax_rows/32x1/256/boolean/exact"),
    ("bf16", 2, 8, 232, "boolean", "softmax_rows/32x1/256/boolean/ragged"),
    ("bf16", 1, 131072, 256, "additive", "softmax_rows/32x1/256/additive/exact"),
    ("bf16", 2, 8, 232, "additive", "softmax_rows/32x1/256/additive/ragged"),
    ("bf16", 1, 524296, 256, "unmasked", "softmax_rows/32x1/256/unmasked/exact"),
    ("bf16", 2, 8, 232, "unmasked", "softmax_rows/32x1/256/unmasked/ragged"),
    ("bf16", 2, 8, 512, "boolean", "softmax_rows/64x1/256/boolean/exact"),
    ("bf16", 2, 8, 488, "boolean", "softmax_rows/64x1/256/boolean/ragged"),
    ("bf16", 1, 65536, 512, "additive", "softmax_rows/64x1/256/additive/exact"),
    ("bf16", 2, 8, 488, "additive", "softmax_rows/64x1/256/additive/ragged"),
    ("bf16", 1, 262152, 512, "unmasked", "softmax_rows/64x1/256/unmasked/exact"),
    ("bf16", 2, 8, 488, "unmasked", "softmax_rows/64x1/256/unmasked/ragged"),
    ("bf16", 2, 8, 1024, "boolean", "softmax_rows/64x2/256/boolean/exact"),
    ("bf16", 2, 8, 1000, "boolean", "softmax_rows/64x2/256/boolean/ragged"),
    ("bf16", 1, 32768, 1024, "additive", "softmax_rows/64x2/256/additive/exact"),
    ("bf16", 2, 8, 1000, "additive", "softmax_rows/64x2/256/additive/ragged"),
    ("bf16", 3972, 33, 1024, "unmasked", "softmax_rows/64x2/256/unmasked/exact"),
    ("bf16", 2, 8, 1000, "unmasked", "softmax_rows/64x2/256/unmasked/ragged"),
    ("bf16", 2, 8, 2048, "boolean", "softmax_rows/128x2/256/boolean/exact"),
    ("bf16", 2, 8, 1536, "boolean", "softmax_rows/128x2/256/boolean/ragged"),
    ("bf16", 1, 16384, 2048, "additive", "softmax_rows/128x2/256/additive/exact"),
    ("bf16", 2, 8, 2024, "additive", "softmax_rows/128x2/256/additive/ragged"),
    ("bf16", 1986, 33, 2048, "unmasked", "softmax_rows/128x2/256/unmasked/exact"),
    ("bf16", 2, 8, 2024, "unmasked", "softmax_rows/128x2/256/unmasked/ragged"),
    ("bf16", 1, 8192, 4096, "boolean", "softmax_rows/256x2/256/boolean/exact"),
    ("bf16", 2, 8, 2560, "boolean", "softmax_rows/256x2/256/boolean/ragged"),
    ("bf16", 512, 16, 4096, "additive", "softmax_rows/256x2/256/additive/exact/steered"),
    ("bf16", 1, 8192, 4096, "additive", "softmax_rows/256x2/256/additive/exact"),
    ("bf16", 2, 8, 4072, "additive", "softmax_rows/256x2/256/additive/ragged/steered"),
    ("bf16", 2, 9, 4072, "additive", "softmax_rows/256x2/256/additive/ragged"),
    ("bf16", 911, 9, 4096, "unmasked", "softmax_rows/256x2/256/unmasked/exact"),
    ("bf16", 2, 8, 4072, "unmasked", "softmax_rows/256x2/256/unmasked/ragged"),
    ("bf16", 1, 4096, 8192, "boolean", "softmax_rows/64x16/64/boolean/exact"),
    ("bf16", 2, 8, 6120, "boolean", "softmax_rows/256x4/256/boolean/ragged"),
    ("bf16", 256, 16, 8192, "additive", "softmax_rows/512x2/512/additive/exact/steered"),
    ("bf16", 1, 4096, 8192, "additive", "softmax_rows/512x2/512/additive/exact"),
    ("bf16", 2, 8, 6120, "additive", "softmax_rows/512x2/512/additive/ragged/steered"),
    ("bf16", 2, 9, 6120, "additive", "softmax_rows/512x2/512/additive/ragged"),
    ("bf16", 125, 33, 8192, "unmasked", "softmax_rows/512x2/512/unmasked/exact"),
    ("bf16", 2, 8, 6120, "unmasked", "softmax_rows/512x2/512/unmasked/ragged"),
    ("bf16", 1, 2048, 16384, "boolean", "softmax_rows/512x4/512/boolean/exact"),
    ("bf16", 2, 8, 16360, "boolean", "softmax_rows/512x4/512/boolean/ragged"),
    ("bf16", 128, 16, 16384, "additive", "softmax_rows/512x4/512/additive/exact/steered"),
    ("bf16", 1, 2048, 16384, "additive", "softmax_rows/512x4/512/additive/exact"),
    ("bf16", 2, 8, 16360, "additive", "softmax_rows/512x4/512/additive/ragged/steered"),
    ("bf16", 2, 9, 16360, "additive", "softmax_rows/512x4/512/additive/ragged"),
    ("bf16", 63, 33, 16384, "unmasked", "softmax_rows/512x4/512/unmasked/exact"),
    ("bf16", 2, 8, 16360, "unmasked", "softmax_rows/512x4/512/unmasked/ragged"),
    ("bf16", 2, 8, 32768, "boolean", "softmax_rows/1024x4/1024/boolean/exact"),
    ("bf16", 2, 8, 32744, "boolean", "softmax_rows/1024x4/1024/boolean/ragged"),
    ("bf16", 2, 8, 32768, "additive", "softmax_rows/1024x4/1024/additive/exact/steered"),
    ("bf16", 2, 9, 32768, "additive", "softmax_rows/1024x4/1024/additive/exact"),
    ("bf16", 2, 8, 32744, "additive", "softmax_rows/1024x4/1024/additive/ragged/steered"),
    ("bf16", 2, 9, 32744, "additive", "softmax_rows/1024x4/1024/additive/ragged"),
    ("bf16", 2, 8, 32768, "unmasked", "softmax_rows/1024x4/1024/unmasked/exact"),
    ("bf16", 2, 8, 32744, "unmasked", "softmax_rows/1024x4/1024/unmasked/ragged"),
    ("bf16", 2, 8, 65536, "boolean", "softmax_rows/1024x8/1024/boolean/exact"),
    ("bf16", 2, 8, 65512, "boolean", "softmax_rows/1024x8/1024/boolean/ragged"),
    ("bf16", 2, 8, 65536, "additive", "softmax_rows/1024x8/1024/additive/exact/steered"),
    ("bf16", 2, 9, 65536, "additive", "softmax_rows/1024x8/1024/additive/exact"),
    ("bf16", 2, 8, 65512, "additive", "softmax_rows/1024x8/1024/additive/ragged/steered"),
    ("bf16", 2, 9, 65512, "additive", "softmax_rows/1024x8/1024/additive/ragged"),
    ("bf16", 2, 8, 65536, "unmasked", "softmax_rows/1024x8/1024/unmasked/exact"),
    ("bf16", 2, 8, 65512, "unmasked", "softmax_rows/1024x8/1024/unmasked/ragged"),
    ("f32", 2, 3, 129, "unmasked", "softmax_general"),
    ("bf16", 2, 16, 128, "additive", "softmax_rows_exact/8x2/64/4/additive"),
    ("bf16", 2, 16, 128, "unmasked", "softmax_rows_exact/8x2/64/4/unmasked"),
    ("bf16", 2, 8, 256, "additive", "softmax_rows_exact/16x2/64/4/additive"),
    ("bf16", 2, 8, 256, "unmasked", "softmax_rows_exact/16x2/64/4/unmasked"),
    ("bf16", 2, 8, 512, "additive", "softmax_rows_exact/32x2/64/4/additive"),
    ("bf16", 2, 8, 512, "unmasked", "softmax_rows_exact/32x2/64/4/unmasked"),
    ("bf16", 2, 8, 1024, "additive", "softmax_rows_exact/64x2/64/4/additive"),
    ("bf16", 2, 8, 1024, "unmasked", "softmax_rows_exact/64x2/64/4/unmasked"),
    ("bf16", 2, 8, 1536, "additive", "softmax_rows_exact/64x3/64/2/additive"),
    ("bf16", 2, 8, 1536, "unmasked", "softmax_rows_exact/64x3/64/2/unmasked"),
    ("bf16", 2, 8, 2048, "additive", "softmax_rows_exact/128x2/128/2/additive"),
    ("bf16", 2, 8, 2048, "unmasked", "softmax_rows_exact/128x2/128/2/unmasked"),
    ("bf16", 2, 8, 2560, "additive", "softmax_rows_exact/64x5/64/2/additive"),
    ("bf16", 2, 8, 2560, "unmasked", "softmax_rows_exact/64x5/64/2/unmasked"),
    ("bf16", 2, 8, 3072, "additive", "softmax_rows_exact/128x3/128/2/additive"),
    ("bf16", 2, 8, 3072, "unmasked", "softmax_rows_exact/128x3/128/2/unmasked"),
    ("bf16", 2, 8, 3584, "additive", "softmax_rows_exact/64x7/64/2/additive"),
    ("bf16", 2, 8, 3584, "unmasked", "softmax_rows_exact/64x7/64/2/unmasked"),
    ("bf16", 2, 8, 4096, "boolean", "softmax_rows_exact/128x4/128/2/boolean"),
    ("bf16", 2, 8, 4096, "additive", "softmax_rows_exact/128x4/128/2/additive"),
    ("bf16", 2, 8, 4096, "unmasked", "softmax_rows_exact/128x4/128/2/unmasked"),
    ("bf16", 2, 8, 5120, "boolean", "softmax_rows_exact/128x5/128/2/boolean"),
    ("bf16", 2, 8, 5120, "additive", "softmax_rows_exact/128x5/128/2/additive"),
    ("bf16", 2, 8, 5120, "unmasked", "softmax_rows_exact/128x5/128/2/unmasked"),
    ("bf16", 2, 8, 6144, "boolean", "softmax_rows_exact/256x3/256/2/boolean"),
    ("bf16", 2, 8, 6144, "additive", "softmax_rows_exact/256x3/256/2/additive"),
    ("bf16", 2, 8, 6144, "unmasked", "softmax_rows_exact/256x3/256/2/unmasked"),
    ("bf16", 2, 8, 7168, "boolean", "softmax_rows_exact/128x7/128/2/boolean"),
    ("bf16", 2, 8, 7168, "additive", "softmax_rows_exact/128x7/128/2/additive"),
    ("bf16", 2, 8, 7168, "unmasked", "softmax_rows_exact/128x7/128/2/unmasked"),
    ("bf16", 2, 8, 8192, "boolean", "softmax_rows_exact/256x4/256/2/boolean"),
    ("bf16", 2, 8, 8192, "additive", "softmax_rows_exact/256x4/256/2/additive"),
    ("bf16", 2, 8, 8192, "unmasked", "softmax_rows_exact/256x4/256/2/unmasked"),
    ("bf16", 2, 8, 10240, "boolean", "softmax_rows_exact/256x5/256/2/boolean"),
    ("bf16", 2, 8, 10240, "additive", "softmax_rows_exact/256x5/256/2/additive"),
    ("bf16", 2, 8, 10240, "unmasked", "softmax_rows_exact/256x5/256/2/unmasked"),
    ("bf16", 2, 8, 12288, "boolean", "softmax_rows_exact/512x3/512/2/boolean"),
    ("bf16", 2, 8, 12288, "additive", "softmax_rows_exact/512x3/512/2/additive"),
    ("bf16", 2, 8, 12288, "unmasked", "softmax_rows_exact/512x3/512/2/unmasked"),
    ("bf16", 2, 8, 14336, "boolean", "softmax_rows_exact/256x7/256/2/boolean"),
    ("bf16", 2, 8, 14336, "additive", "softmax_rows_exact/256x7/256/2/additive"),
    ("bf16", 2, 8, 14336, "unmasked", "softmax_rows_exact/256x7/256/2/unmasked"),
    ("bf16", 2, 8, 16384, "boolean", "softmax_rows_exact/512x4/512/2/boolean"),
    ("bf16", 2, 8, 16384, "additive", "softmax_rows_exact/512x4/512/2/additive"),
    ("bf16", 2, 8, 16384, "unmasked", "softmax_rows_exact/512x4/512/2/unmasked"),
    ("f32", 2, 16, 32, "boolean", "softmax_rows/8x1/256/boolean/exact"),
    ("f32", 2, 8, 20, "boolean", "softmax_rows/8x1/256/boolean/ragged"),
    ("f32", 2, 16, 32, "additive", "softmax_rows/8x1/256/additive/exact"),
    ("f32", 2, 8, 20, "additive", "softmax_rows/8x1/256/additive/ragged"),
    ("f32", 2, 16, 32, "unmasked", "softmax_rows/8x1/256/unmasked/exact"),
    ("f32", 2, 8, 20, "unmasked", "softmax_rows/8x1/256/unmasked/ragged"),
    ("f32", 2, 8, 64, "boolean", "softmax_rows/16x1/256/boolean/exact"),
    ("f32", 2, 8, 52, "boolean", "softmax_rows/16x1/256/boolean/ragged"),
    ("f32", 2, 8, 64, "additive", "softmax_rows/16x1/256/additive/exact"),
    ("f32", 2, 8, 52, "additive", "softmax_rows/16x1/256/additive/ragged"),
    ("f32", 2, 8, 64, "unmasked", "softmax_rows/16x1/256/unmasked/exact"),
    ("f32", 2, 8, 52, "unmasked", "softmax_rows/16x1/256/unmasked/ragged"),
    ("f32", 2, 8, 128, "boolean", "softmax_rows/32x1/256/boolean/exact"),
    ("f32", 2, 8, 116, "boolean", "softmax_rows/32x1/256/boolean/ragged"),
    ("f32", 1, 131072, 128, "additive", "softmax_rows/32x1/256/additive/exact"),
    ("f32", 2, 8, 116, "additive", "softmax_rows/32x1/256/additive/ragged"),
    ("f32", 2, 8, 116, "unmasked", "softmax_rows/32x1/256/unmasked/ragged"),
    ("f32", 2, 8, 256, "boolean", "softmax_rows/64x1/256/boolean/exact"),
    ("f32", 2, 8, 244, "boolean", "softmax_rows/64x1/256/boolean/ragged"),
    ("f32", 1, 65536, 256, "additive", "softmax_rows/64x1/256/additive/exact"),
    ("f32", 2, 8, 244, "additive", "softmax_rows/64x1/256/additive/ragged"),
    ("f32", 2, 8, 244, "unmasked", "softmax_rows/64x1/256/unmasked/ragged"),
    ("f32", 2, 8, 512, "boolean", "softmax_rows/64x2/256/boolean/exact"),
    ("f32", 2, 8, 500, "boolean", "softmax_rows/64x2/256/boolean/ragged"),
    ("f32", 1, 32768, 512, "additive", "softmax_rows/64x2/256/additive/exact"),
    ("f32", 2, 8, 500, "additive", "softmax_rows/64x2/256/additive/ragged"),
    ("f32", 2, 8, 500, "unmasked", "softmax_rows/64x2/256/unmasked/ragged"),
    ("f32", 2, 8, 1024, "boolean", "softmax_rows/128x2/256/boolean/exact"),
    ("f32", 2, 8, 768, "boolean", "softmax_rows/128x2/256/boolean/ragged"),
    ("f32", 1, 16384, 1024, "additive", "softmax_rows/128x2/256/additive/exact"),
    ("f32", 2, 8, 1012, "additive", "softmax_rows/128x2/256/additive/ragged"),
    ("f32", 2, 8, 1012, "unmasked", "softmax_rows/128x2/256/unmasked/ragged"),
    ("f32", 1, 8192, 2048, "boolean", "softmax_rows/256x2/256/boolean/exact"),
    ("f32", 2, 8, 1280, "boolean", "softmax_rows/256x2/256/boolean/ragged"),
    ("f32", 512, 16, 2048, "additive", "softmax_rows/256x2/256/additive/exact/steered"),
    ("f32", 1, 8192, 2048, "additive", "softmax_rows/256x2/256/additive/exact"),
    ("f32", 2, 8, 2036, "additive", "softmax_rows/256x2/256/additive/ragged/steered"),
    ("f32", 2, 9, 2036, "additive", "softmax_rows/256x2/256/additive/ragged"),
    ("f32", 911, 9, 2048, "unmasked", "softmax_rows/256x2/256/unmasked/exact"),
    ("f32", 2, 8, 2036, "unmasked", "softmax_rows/256x2/256/unmasked/ragged"),
    ("f32", 1, 4096, 4096, "boolean", "softmax_rows/64x16/64/boolean/exact"),
    ("f32", 2, 8, 3060, "boolean", "softmax_rows/256x4/256/boolean/ragged"),
    ("f32", 256, 16, 4096, "additive", "softmax_rows/512x2/512/additive/exact/steered"),
    ("f32", 1, 4096, 4096, "additive", "softmax_rows/512x2/512/additive/exact"),
    ("f32", 2, 8, 3060, "additive", "softmax_rows/512x2/512/additive/ragged/steered"),
    ("f32", 2, 9, 3060, "additive", "softmax_rows/512x2/512/additive/ragged"),
    ("f32", 125, 33, 4096, "unmasked", "softmax_rows/512x2/512/unmasked/exact"),
    ("f32", 2, 8, 3060, "unmasked", "softmax_rows/512x2/512/unmasked/ragged"),
    ("f32", 1, 2048, 8192, "boolean", "softmax_rows/512x4/512/boolean/exact"),
    ("f32", 2, 8, 8180, "boolean", "softmax_rows/512x4/512/boolean/ragged"),
    ("f32", 128, 16, 8192, "additive", "softmax_rows/512x4/512/additive/exact/steered"),
    ("f32", 1, 2048, 8192, "additive", "softmax_rows/512x4/512/additive/exact"),
    ("f32", 2, 8, 8180, "additive", "softmax_rows/512x4/512/additive/ragged/steered"),
    ("f32", 2, 9, 8180, "additive", "softmax_rows/512x4/512/additive/ragged"),
    ("f32", 63, 33, 8192, "unmasked", "softmax_rows/512x4/512/unmasked/exact"),
    ("f32", 2, 8, 8180, "unmasked", "softmax_rows/512x4/512/unmasked/ragged"),
    ("f32", 2, 8, 16384, "boolean", "softmax_rows/1024x4/1024/boolean/exact"),
    ("f32", 2, 8, 16372, "boolean", "softmax_rows/1024x4/1024/boolean/ragged"),
    ("f32", 2, 8, 16384, "additive", "softmax_rows/1024x4/1024/additive/exact/steered"),
    ("f32", 2, 9, 16384, "additive", "softmax_rows/1024x4/1024/additive/exact"),
    ("f32", 2, 8, 16372, "additive", "softmax_rows/1024x4/1024/additive/ragged/steered"),
    ("f32", 2, 9, 16372, "additive", "softmax_rows/1024x4/1024/additive/ragged"),
    ("f32", 2, 8, 16384, "unmasked", "softmax_rows/1024x4/1024/unmasked/exact"),
    ("f32", 2, 8, 16372, "unmasked", "softmax_rows/1024x4/1024/unmasked/ragged"),
    ("f32", 2, 8, 32768, "boolean", "softmax_rows/1024x8/1024/boolean/exact"),
    ("f32", 2, 8, 32756, "boolean", "softmax_rows/1024x8/1024/boolean/ragged"),
    ("f32", 2, 8, 32768, "additive", "softmax_rows/1024x8/1024/additive/exact/steered"),
    ("f32", 2, 9, 32768, "additive", "softmax_rows/1024x8/1024/additive/exact"),
    ("f32", 2, 8, 32756, "additive", "softmax_rows/1024x8/1024/additive/ragged/steered"),
    ("f32", 2, 9, 32756, "additive", "softmax_rows/1024x8/1024/additive/ragged"),
    ("f32", 2, 8, 32768, "unmasked", "softmax_rows/1024x8/1024/unmasked/exact"),
    ("f32", 2, 8, 32756, "unmasked", "softmax_rows/1024x8/1024/unmasked/ragged"),
    ("f32", 2, 16, 64, "additive", "softmax_rows_exact/8x2/64/4/additive"),
    ("f32", 2, 16, 64, "unmasked", "softmax_rows_exact/8x2/64/4/unmasked"),
    ("f32", 2, 8, 128, "additive", "softmax_rows_exact/16x2/64/4/additive"),
    ("f32", 2, 8, 128, "unmasked", "softmax_rows_exact/16x2/64/4/unmasked"),
    ("f32", 2, 8, 256, "additive", "softmax_rows_exact/32x2/64/4/additive"),
    ("f32", 2, 8, 256, "unmasked", "softmax_rows_exact/32x2/64/4/unmasked"),
    ("f32", 2, 8, 512, "additive", "softmax_rows_exact/64x2/64/4/additive"),
    ("f32", 2, 8, 512, "unmasked", "softmax_rows_exact/64x2/64/4/unmasked"),
    ("f32", 2, 8, 768, "additive", "softmax_rows_exact/64x3/64/2/additive"),
    ("f32", 2, 8, 768, "unmasked", "softmax_rows_exact/64x3/64/2/unmasked"),
    ("f32", 2, 8, 1024, "additive", "softmax_rows_exact/128x2/128/2/additive"),
    ("f32", 2, 8, 1024, "unmasked", "softmax_rows_exact/128x2/128/2/unmasked"),
    ("f32", 2, 8, 1280, "additive", "softmax_rows_exact/64x5/64/2/additive"),
    ("f32", 2, 8, 1280, "unmasked", "softmax_rows_exact/64x5/64/2/unmasked"),
    ("f32", 2, 8, 1536, "additive", "softmax_rows_exact/128x3/128/2/additive"),
    ("f32", 2, 8, 1536, "unmasked", "softmax_rows_exact/128x3/128/2/unmasked"),
    ("f32", 2, 8, 1792, "additive", "softmax_rows_exact/64x7/64/2/additive"),
    ("f32", 2, 8, 1792, "unmasked", "softmax_rows_exact/64x7/64/2/unmasked"),
    ("f32", 2, 8, 2048, "boolean", "softmax_rows_exact/128x4/128/2/boolean"),
    ("f32", 2, 8, 2048, "additive", "softmax_rows_exact/128x4/128/2/additive"),
    ("f32", 2, 8, 2048, "unmasked", "softmax_rows_exact/128x4/128/2/unmasked"),
    ("f32", 2, 8, 2560, "boolean", "softmax_rows_exact/128x5/128/2/boolean"),
    ("f32", 2, 8, 2560, "additive", "softmax_rows_exact/128x5/128/2/additive"),
    ("f32", 2, 8, 2560, "unmasked", "softmax_rows_exact/128x5/128/2/unmasked"),
    ("f32", 2, 8, 3072, "boolean", "softmax_rows_exact/256x3/256/2/boolean"),
    ("f32", 2, 8, 3072, "additive", "softmax_rows_exact/256x3/256/2/additive"),
    ("f32", 2, 8, 3072, "unmasked", "softmax_rows_exact/256x3/256/2/unmasked"),
    ("f32", 2, 8, 3584, "boolean", "softmax_rows_exact/128x7/128/2/boolean"),
    ("f32", 2, 8, 3584, "additive", "softmax_rows_exact/128x7/128/2/additive"),
    ("f32", 2, 8, 3584, "unmasked", "softmax_rows_exact/128x7/128/2/unmasked"),
    ("f32", 2, 8, 4096, "boolean", "softmax_rows_exact/256x4/256/2/boolean"),
    ("f32", 2, 8, 4096, "additive", "softmax_rows_exact/256x4/256/2/additive"),
    ("f32", 2, 8, 4096, "unmasked", "softmax_rows_exact/256x4/256/2/unmasked"),
    ("f32", 2, 8, 5120, "boolean", "softmax_rows_exact/256x5/256/2/boolean"),
    ("f32", 2, 8, 5120, "additive", "softmax_rows_exact/256x5/256/2/additive"),
    ("f32", 2, 8, 5120, "unmasked", "softmax_rows_exact/256x5/256/2/unmasked"),
    ("f32", 2, 8, 6144, "boolean", "softmax_rows_exact/512x3/512/2/boolean"),
    ("f32", 2, 8, 6144, "additive", "softmax_rows_exact/512x3/512/2/additive"),
    ("f32", 2, 8, 6144, "unmasked", "softmax_rows_exact/512x3/512/2/unmasked"),
    ("f32", 2, 8, 7168, "boolean", "softmax_rows_exact/256x7/256/2/boolean"),
    ("f32", 2, 8, 7168, "additive", "softmax_rows_exact/256x7/256/2/additive"),
    ("f32", 2, 8, 7168, "unmasked", "softmax_rows_exact/256x7/256/2/unmasked"),
    ("f32", 2, 8, 8192, "boolean", "softmax_rows_exact/512x4/512/2/boolean"),
    ("f32", 2, 8, 8192, "additive", "softmax_rows_exact/512x4/512/2/additive"),
    ("f32", 2, 8, 8192, "unmasked", "softmax_rows_exact/512x4/512/2/unmasked"),
    # the large launches named one by one: cfg4's additive form at a sixteenth of its heads
    # (64 MiB, mask period 256), the same in bf16, and a Boolean mask over rows of 768 vectors
    ("f32", 16, 256, 4096, "additive", "softmax_rows/512x2/512/additive/exact/steered"),
    ("bf16", 32, 256, 4096, "additive", "softmax_rows/256x2/256/additive/exact/steered"),
    ("bf16", 16, 256, 8192, "additive", "softmax_rows/512x2/512/additive/exact/steered"),
    ("f32", 22, 256, 3072, "boolean", "softmax_rows/256x4/256/boolean/ragged"),
    ("f32", 4, 4096, 4096, "boolean", "softmax_rows/64x16/64/boolean/exact"),
    ("bf16", 2, 3, 70000, "boolean", "softmax_general"),
]

MASKS = {"unmasked": hc.MaskKind.kNone, "additive": hc.MaskKind.kAdditive, "boolean": hc.MaskKind.kBoolean}
ORC_MASKS = {"unmasked": orc.MASK_NONE, "additive": orc.MASK_ADDITIVE, "boolean": orc.MASK_BOOLEAN}
THREADS = min(16, len(os.sched_getaffinity(0)))
reached = set()


def make_inputs(tag, heads, q, width, mask_word, seed):
    """x on the device (read back for the oracle) with -inf elements, one NaN row and one +inf row
    per head; the mask leaves out whole vectors (a staircase) and single columns, and leaves one row
    out entirely (undefined for every head)."""
    dtype = TYPES[tag][2]
    gen = torch.Generator(device=DEVICE).manual_seed(seed)
    x = (torch.randn((heads, q, width), generator=gen, device=DEVICE, dtype=torch.float32) * 3.0).to(dtype)
    holes = torch.rand((heads, q, width), generator=gen, device=DEVICE) < 0.02
    x.masked_fill_(holes, float("-inf"))
    x[:, 0, 0] = 1.5                       # row 0 keeps a finite first column
    if q > 1:
        x[:, 1, 0] = float("nan")          # column 0 is never masked: the row is undefined
    if q > 2:
        x[:, 2, 0] = float("inf")
    mask_device = mask_host = None
    if mask_word == "boolean":
        r = torch.arange(q, device=DEVICE)[:, None]
        c = torch.arange(width, device=DEVICE)[None, :]
        keep = c * 38 <= ((r % 37) + 1) * width
        keep &= torch.rand((q, width), generator=gen, device=DEVICE) < 0.9
        keep[:, 0] = True
        if q > 3:
            keep[3, :] = False
        mask_device = keep
        mask_host = keep.cpu().numpy().view(np.uint8)
    elif mask_word == "additive":
        add = torch.randn((q, width), generator=gen, device=DEVICE, dtype=torch.float32)
        add.masked_fill_(torch.rand((q, width), generator=gen, device=DEVICE) < 0.25, float("-inf"))
        add[:, 0] = 0.0
        if q > 3:
            add[3, :] = float("-inf")
        mask_device = add.to(dtype)
        mask_host = storage_of(mask_device)
    return x, storage_of(x), mask_device, mask_host


def storage_of(t):
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.contiguous().cpu().numpy()


def oracle_softmax(tag, x_host, mask_word, mask_host, scale, log_form):
    """The oracle over [heads, q, width], heads (or, for one head, runs of rows) spread over threads."""
    oid = TYPES[tag][1]
    heads, q, width = x_host.shape
    want = np.empty_like(x_host)

    def piece(part):
        h, first, last = part
        mask = None if mask_host is None else mask_host[first:last]
        want[h, first:last] = orc.softmax(oid, x_host[h, first:last], scale=scale, mask_kind=ORC_MASKS[mask_word],
                                          mask=mask, log=log_form)

    if heads >= THREADS or q < 64:
        parts = [(h, 0, q) for h in range(heads)]
    else:
        cuts = [q * t // THREADS for t in range(THREADS + 1)]
        parts = [(h, cuts[t], cuts[t + 1]) for h in range(heads) for t in range(THREADS) if cuts[t] < cuts[t + 1]]
    with ThreadPoolExecutor(max_workers=THREADS) as pool:
        list(pool.map(piece, parts))
    return want


def compare_on_device(tag, got, want_host, log_form):
    """got (device tensor) against the oracle's result, compared on the device so that launches of
    hundreds of MiB cost little; returns (count of elements outside the bar, text for the first)."""
    if tag == "f32":
        want = torch.from_numpy(want_host).to(DEVICE)
        nan_w, nan_g = torch.isnan(want), torch.isnan(got)
        if not torch.equal(nan_w, nan_g):
            return int((nan_w != nan_g).sum()), "NaN positions differ"
        inf_w = torch.isinf(want)
        if not torch.equal(torch.where(inf_w, got, 0), torch.where(inf_w, want, 0)):
            return int(inf_w.sum()), "infinities differ"
        skip = nan_w | inf_w
        g, w = got.double(), want.double()
        limit = w.abs() * 4e-6 + 2e-7 if log_form else w.abs() * 1e-5 + 1.2e-38
        bad = ((g - w).abs() > limit) & ~skip
    else:
        want = torch.from_numpy(want_host.view(np.int16)).to(DEVICE).int() & 0xFFFF
        bits = got.contiguous().view(torch.int16).int() & 0xFFFF
        top = 0x7F80 if tag == "bf16" else 0x7C00
        nan_w, nan_g = (want & 0x7FFF) > top, (bits & 0x7FFF) > top
        if not torch.equal(nan_w, nan_g):
            return int((nan_w != nan_g).sum()), "NaN positions differ"
        wrong_zero = ((want & 0x7FFF) == 0) & ((bits & 0x7FFF) == 0) & (want != bits)
        ordered = lambda b: torch.where((b & 0x8000) != 0, -(b & 0x7FFF), b)
        bad = (((ordered(bits) - ordered(want)).abs() > 1) & ~nan_w) | wrong_zero
    count = int(bad.sum())
    if count == 0:
        return 0, ""
    at = tuple(int(i) for i in torch.nonzero(bad)[0])
    return count, f"first at {at}: got {got[at].item()!r} want {want_host[at]!r}"


def run_case(tag, heads, q, width, mask_word, label, log_form, seed):
    scale = 0.125 if mask_word != "unmasked" else 1.0
    kind = hc.SoftmaxKind.kLogSoftmax if log_form else hc.SoftmaxKind.kSoftmax
    note(f"softmax {tag} log={log_form} [{heads}, {q}, {width}] {mask_word}: expecting {label}")
    x, x_host, mask_device, mask_host = make_inputs(tag, heads, q, width, mask_word, seed)
    operands = [x] if mask_device is None else [x, mask_device]
    (out,) = run(hc.Softmax(scale=scale, kind=kind, mask=MASKS[mask_word]), *operands)
    chosen = hc.last_launch_variant()
    assert chosen == label, f"[{heads}, {q}, {width}] {tag} {mask_word}: launched {chosen}, the table says {label}"
    reached.add(chosen)
    want = oracle_softmax(tag, x_host, mask_word, mask_host, scale, log_form)
    if q > 3:  # the oracle itself must show the planted rows: NaN row, +inf row, the row left out
        decoded = want if tag == "f32" else orc.to_f32(TYPES[tag][1], want[:, :4])
        assert np.isnan(decoded[:, 1]).all() and np.isnan(decoded[:, 2]).all()
        if mask_word != "unmasked":
            assert np.isnan(decoded[:, 3]).all()
        assert not np.isnan(decoded[:, 0]).any()
    count, text = compare_on_device(tag, out, want, log_form)
    assert count == 0, f"{label}: {count} elements outside the bar, {text}"


def launch_bytes(case):
    tag, heads, q, width = case[:4]
    return heads * q * width * (4 if tag == "f32" else 2)


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}-{c[1]}x{c[2]}x{c[3]}-{c[4]}")
def test_softmax_case_reaches_its_launch_shape_and_matches_the_oracle(case):
    tag, heads, q, width, mask_word, label = case
    run_case(tag, heads, q, width, mask_word, label, False, seed=1000 + CASES.index(case))
    # LogSoftmax shares every launch shape (the kLog form of the same kernels): small launches and
    # the steered ones run it too
    if launch_bytes(case) <= (8 << 20) or "steered" in label:
        run_case(tag, heads, q, width, mask_word, label, True, seed=5000 + CASES.index(case))


def test_softmax_f16_shares_the_bf16_launch_shapes():
    for case in CASES:
        tag, heads, q, width, mask_word, label = case
        if tag == "bf16" and launch_bytes(case) <= (1 << 20):
            run_case("f16", heads, q, width, mask_word, label, False, seed=9000 + CASES.index(case))


def test_softmax_steered_rows_keep_their_places_when_heads_differ():
    """The steered kernel permutes (head, row) pairs over the blocks.  Every head gets its own constant
    shift here, so that a row written to another head's place would carry that head's values."""
    heads, q, width = 16, 256, 4096
    note(f"softmax f32 [{heads}, {q}, {width}] additive mask, rows that name their place")
    gen = torch.Generator(device=DEVICE).manual_seed(77)
    base = torch.randn((q, width), generator=gen, device=DEVICE)
    ramp = torch.arange(width, device=DEVICE, dtype=torch.float32) / width
    x = base[None] * (1.0 + torch.arange(heads, device=DEVICE, dtype=torch.float32)[:, None, None] / heads) + \
        ramp[None, None, :] * torch.arange(q, device=DEVICE, dtype=torch.float32)[None, :, None] / q
    add = torch.zeros((q, width), device=DEVICE)
    add.masked_fill_(torch.arange(width, device=DEVICE)[None, :] > 16 * (torch.arange(q, device=DEVICE)[:, None] + 1), float("-inf"))
    (out,) = run(hc.Softmax(mask=hc.MaskKind.kAdditive), x.contiguous(), add)
    assert hc.last_launch_variant() == "softmax_rows/512x2/512/additive/exact/steered"
    want = oracle_softmax("f32", storage_of(x), "additive", storage_of(add), 1.0, False)
    count, text = compare_on_device("f32", out, want, False)
    assert count == 0, f"{count} elements outside the bar, {text}"


def test_every_softmax_launch_shape_in_the_library_is_reached():
    """Runs after the cases above (file order): a Softmax launch shape compiled into the library
    that no case reached is either dead code or an untested kernel."""
    compiled = {label for label in hc.launch_variants() if label.startswith("softmax")}
    tabled = {case[5] for case in CASES}
    assert compiled == tabled, f"not in the table: {sorted(compiled - tabled)}; not in the library: {sorted(tabled - compiled)}"
    if reached:  # the cases ran in this session
        assert tabled <= reached, f"tabled but not reached: {sorted(tabled - reached)}"
