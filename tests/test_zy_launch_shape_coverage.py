"""Every kernel launch shape compiled into the library is launched by some test of the GPU suite.

The launchers pick a kernel shape from sizes, strides and alignments seen at launch; each shape has a
label that registers itself when the library loads (`hyle_hip_variant_label`), and `gpu_support`
notes the label(s) of every launch the tests make (`hyle_hip_last_launch_variant` after each submit),
whose results those tests hold against the CPU oracle.  A shape that is compiled in but launched by no test is
either dead code or an unchecked kernel: this file (collected after the operator tests, before the
last one) fails on it.  Softmax and the norms also have tables of their
own that name the expected shape case by case (test_gpu_softmax_variants.py, test_gpu_norm_variants.py).
"""
from __future__ import annotations

import sys

import pytest

from hyle_amd import compute as hc

import gpu_support

pytestmark = pytest.mark.gpu

# the modules whose cases reach the shapes; without them in the session there is nothing to hold
SUITE = ("test_gpu_parity", "test_gpu_softmax_variants", "test_gpu_norm_variants", "test_gpu_reduce", "test_gpu_cast_copy",
         "test_gpu_k_quants", "test_gpu_gguf_matvec_q8", "test_gpu_gguf_matvec", "test_gpu_topk", "test_gpu_unary_gated",
         "test_gpu_fill_select", "test_gpu_concat", "test_gpu_gather", "test_gpu_rope", "test_gpu_sampling", "test_gpu_storage_types")


def test_every_launch_shape_compiled_into_the_library_was_launched_by_a_test():
    absent = [name for name in SUITE if name not in sys.modules]
    if absent:
        pytest.skip(f"the whole GPU suite did not run in this session (not loaded: {absent})")
    compiled = set(hc.launch_variants())
    missing = sorted(compiled - gpu_support.LAUNCHED)
    assert not missing, f"{len(missing)} launch shapes compiled into the library were launched by no test: {missing}"
