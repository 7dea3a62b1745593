#!/usr/bin/env python3
"""Measures the tensor hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: the largest shape of
each of the five benchmark configurations, seven kernels launched back to back through the
C ABI of libhyle_hip.so on one HIP stream:

    cfg1  f32  (A[4096,2048] + b[2048]) * 0.5          BinaryChain (add, multiply)
    cfg2  bf16 RMSNorm X[8192,2048], w[2048], eps 1e-6
    cfg3  bf16 SwiGLU gate/up[8192,6144]                GatedActivation (SiLU, separate)
    cfg3' bf16 R[8192,2048] += Y                        Binary add, output aliases input 0
    cfg4  f32  softmax S[32,4096,4096] + causal Bool mask [4096,4096]
    cfg4' f32  argmax logits[64,151936]                 TopK(count = 1)
    cfg5  Q8_0 W[6144 rows x 2048] -> bf16 + f32 row sum of squares

Inputs are resident in HBM before the timed region.  Shapes whose traffic fits the 256 MB
memory-side cache rotate over several buffer sets (> 512 MB in total) so that HBM, not the
cache, is measured.  `value` is credited bytes per step / step time (algorithmic bytes, less
the masked loads the softmax skips); `roofline` describes
the dominant kernel (softmax) timed with HIP events inside the timed region; `per_op` holds
each kernel's own figure from an event-timed loop of back-to-back launches; `cpu_baseline`
times the CPU oracle ("port" of the reference's CPU path) on a bounded sample of the same
workload on the host cores.

Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--op-reps", type=int, default=200, help="launches per kernel in the per-op timing loops")
    p.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    p.add_argument("--cpu-seconds", type=float, default=2.0, help="target CPU seconds per kernel sample")
    p.add_argument("--file-stream-mib", type=int, default=0,
                   help="also stream a temporary file of this many MiB into HBM and report the rate (PCIe-inclusive; "
                        "never part of `value`)")
    p.add_argument("--only", default="", help="comma-separated op names: run and time just these kernels")
    p.add_argument("--copy-probe", action="store_true",
                   help="also run three plain device copies of 1 GiB (a kernel of known traffic that "
                        "calibrates the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return p.parse_args()


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from hyle_amd import compute as hc
    from hyle_amd import torch_io as tio
    from hyle_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)
    ctx = hc.Context.create(0)
    stream = torch.cuda.current_stream().cuda_stream
    BK = hc.BinaryKind

    def bf16(bits):
        return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.bfloat16)

    class Op:
        """One kernel of the step: a prepared operation plus `sets` rotating buffer sets."""

        def __init__(self, name, operation, descs, make_set, sets, algorithmic_bytes, elements, dtype,
                     credited_bytes=None, in_step=True, ceiling=None):
            self.name, self.bytes, self.elements, self.dtype = name, algorithmic_bytes, elements, dtype
            # name of the plain kernel (a copy or a read-only scan of about the same traffic, timed in
            # this run) whose GB/s is the practical ceiling for a launch of this size
            self.ceiling = ceiling
            # Bytes the kernel is credited with: the algorithmic bytes, minus loads it provably
            # does not need and does not issue (no bandwidth is claimed for bytes never moved).
            self.credited = algorithmic_bytes if credited_bytes is None else credited_bytes
            self.in_step = in_step
            began = time.perf_counter()
            self.bound = tio.Bound(ctx, operation, descs, device=dev)
            self.plan_us = (time.perf_counter() - began) * 1e6   # propose + prepare (plus the workspace allocation)
            self.first_launch_us = None
            self.variant = ""
            self.route = self.bound.prepared.route_name()
            self.sets = [make_set(i) for i in range(sets)]  # each: (inputs, outputs)
            self.addresses = [([t.data_ptr() for t in i], [t.data_ptr() for t in o]) for i, o in self.sets]
            self.turn = 0

        def launch(self, on_stream):
            """Enqueue on the HIP stream `on_stream`, rotating to the next buffer set."""
            inputs, outputs = self.addresses[self.turn]
            self.turn = (self.turn + 1) % len(self.sets)
            self.bound.invocation.submit(on_stream, inputs, outputs)

        def launch_first_set(self, on_stream):
            """Enqueue on the first buffer set only: the operands stay in the memory-side cache."""
            inputs, outputs = self.addresses[0]
            self.bound.invocation.submit(on_stream, inputs, outputs)

    D = hc.TensorDesc.dense
    F32, BF = hc.DataType.kFloat32, hc.DataType.kBFloat16
    ops = []
    wanted = {n for n in args.only.split(",") if n}

    def want(name):
        return not wanted or name in wanted

    # ---- cfg1 ---------------------------------------------------------------------------
    if want("cfg1_broadcast_add_mul_f32"):
        a, b, s = wl.config1()
        db, ds = torch.from_numpy(b).to(dev), torch.from_numpy(s).to(dev)

        def set1(i):
            da = torch.from_numpy(np.roll(a, i, axis=0)).to(dev)
            return [da, db, ds], [torch.empty_like(da)]
        ops.append(Op("cfg1_broadcast_add_mul_f32", hc.BinaryChain(BK.kAdd, BK.kMultiply),
                      [D(F32, [4096, 2048]), D(F32, [2048]), D(F32, [1])], set1, 10,
                      wl.ALGORITHMIC_BYTES["cfg1_broadcast_add_mul_f32"], 4096 * 2048, "f32",
                      ceiling="ceiling_copy_67mb"))
    # ---- cfg2 ---------------------------------------------------------------------------
    if want("cfg2_rmsnorm_bf16"):
        x, w = wl.config2()
        dw = bf16(w)

        def set2(i):
            dx = bf16(np.roll(x, i, axis=0))
            return [dx, dw], [torch.empty_like(dx)]
        ops.append(Op("cfg2_rmsnorm_bf16", hc.RmsNorm(epsilon=1e-6), [D(BF, [8192, 2048]), D(BF, [2048])], set2, 10,
                      wl.ALGORITHMIC_BYTES["cfg2_rmsnorm_bf16"], 8192 * 2048, "bf16", ceiling="ceiling_copy_67mb"))
    # ---- cfg3 ---------------------------------------------------------------------------
    if want("cfg3_swiglu_bf16"):
        gate, up = wl.config3_swiglu()

        def set3(i):
            dg, du = bf16(np.roll(gate, i, axis=0)), bf16(np.roll(up, i, axis=0))
            return [dg, du], [torch.empty_like(dg)]
        ops.append(Op("cfg3_swiglu_bf16", hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                      [D(BF, [8192, 6144]), D(BF, [8192, 6144])], set3, 3,
                      wl.ALGORITHMIC_BYTES["cfg3_swiglu_bf16"], 8192 * 6144, "bf16"))
    if want("cfg3_residual_add_bf16"):
        r, y = wl.config3_residual()

        def set3r(i):
            dr, dy = bf16(np.roll(r, i, axis=0)), bf16(np.roll(y, i, axis=0))
            return [dr, dy], [dr]  # R += Y
        ops.append(Op("cfg3_residual_add_bf16", hc.Binary(BK.kAdd), [D(BF, [8192, 2048]), D(BF, [8192, 2048])],
                      set3r, 10, wl.ALGORITHMIC_BYTES["cfg3_residual_add_bf16"], 8192 * 2048, "bf16"))
    # ---- cfg4 ---------------------------------------------------------------------------
    if want("cfg4_softmax_f32_causal"):
        s4_host, mask_host = wl.config4_softmax()  # seed 3: the bytes the parity test and the CPU leg use
        big = torch.from_numpy(s4_host).to(dev)
        causal = torch.from_numpy(mask_host).to(dev).view(torch.bool)
        del s4_host, mask_host
        big_out = torch.empty_like(big)
        # Under the Boolean mask the kernel does not load a 16-byte vector of S whose four
        # elements are all masked (they cannot influence the result), so row q reads q // 4 + 1
        # of its 1024 vectors.  Those skipped loads earn no credit.
        kept = 32 * sum((q // 4 + 1) * 16 for q in range(4096))
        ops.append(Op("cfg4_softmax_f32_causal", hc.Softmax(mask=hc.MaskKind.kBoolean),
                      [D(F32, [32, 4096, 4096]), D(hc.DataType.kBool, [4096, 4096])],
                      lambda i: ([big, causal], [big_out]), 1,
                      wl.ALGORITHMIC_BYTES["cfg4_softmax_f32_causal"], 32 * 4096 * 4096, "f32",
                      credited_bytes=kept + big.numel() * 4 + causal.numel()))
        # The same softmax under the additive form of the mask (f32 0 / -inf): every element of S
        # is needed (NaN + -inf is NaN), so every byte is loaded.  Timed on its own, not in the step.
        additive = torch.zeros((4096, 4096), dtype=torch.float32, device=dev).masked_fill_(~causal, float("-inf"))
        ops.append(Op("cfg4_softmax_f32_causal_additive", hc.Softmax(mask=hc.MaskKind.kAdditive),
                      [D(F32, [32, 4096, 4096]), D(F32, [4096, 4096])],
                      lambda i: ([big, additive], [big_out]), 1,
                      2 * big.numel() * 4 + additive.numel() * 4, 32 * 4096 * 4096, "f32", in_step=False))
    if want("cfg4_argmax_f32"):
        logits = wl.config4_argmax()

        def set4a(i):
            dl = torch.from_numpy(np.roll(logits, i, axis=0)).to(dev)
            return [dl], [torch.empty((64, 1), dtype=torch.float32, device=dev),
                          torch.empty((64, 1), dtype=torch.int32, device=dev)]
        ops.append(Op("cfg4_argmax_f32", hc.TopK(), [D(F32, [64, 151936])], set4a, 16,
                      wl.ALGORITHMIC_BYTES["cfg4_argmax_f32"], 64 * 151936, "f32", ceiling="ceiling_scan_38mb"))
    # ---- cfg5 ---------------------------------------------------------------------------
    if want("cfg5_q8_0_dequant_sumsq"):
        blocks = wl.config5()

        def set5(i):
            dbk = torch.from_numpy(np.roll(blocks, i, axis=0)).to(dev)
            return [dbk], [torch.empty((6144, 2048), dtype=torch.bfloat16, device=dev),
                           torch.empty(6144, dtype=torch.float32, device=dev)]
        ops.append(Op("cfg5_q8_0_dequant_sumsq", hc.Q8_0DequantSumSquares(),
                      [hc.TensorDesc.gguf_q8_0_weight(BF, 2048, 6144)], set5, 16,
                      wl.ALGORITHMIC_BYTES["cfg5_q8_0_dequant_sumsq"], 6144 * 2048, "u8/bf16", ceiling="ceiling_copy_38mb"))
    # ---- the K-quant siblings of cfg5 (GGUF Q4_K / Q6_K), timed beside the step ------------------
    for name, gguf, block_bytes in (("next_q4_k_dequant_sumsq", hc.GgufQuantizedType.kQ4K, 144),
                                    ("next_q6_k_dequant_sumsq", hc.GgufQuantizedType.kQ6K, 210)):
        if not want(name):
            continue

        def set_k(i, block_bytes=block_bytes):
            raw = torch.randint(0, 256, (6144, 8 * block_bytes), dtype=torch.uint8)
            fields = raw.view(6144, 8, block_bytes)      # keep the f16 scales finite
            for at in ((1, 3) if block_bytes == 144 else (209,)):
                fields[:, :, at] &= 0x3B
            return [raw.to(dev)], [torch.empty((6144, 2048), dtype=torch.bfloat16, device=dev),
                                   torch.empty(6144, dtype=torch.float32, device=dev)]
        ops.append(Op(name, hc.GgufDequantSumSquares(), [hc.TensorDesc.gguf_weight(gguf, BF, 2048, 6144)], set_k, 16,
                      6144 * (8 * block_bytes + 2048 * 2 + 4), 6144 * 2048, "u8/bf16", in_step=False,
                      ceiling="ceiling_copy_38mb"))
    # ---- decode-time MatMul over GGUF weights: one activation row against [K, N] ----------------
    EXACT, GGML_Q8 = hc.ActivationArithmetic.kExact, hc.ActivationArithmetic.kGgmlQ8
    for name, gguf, block_bytes, k, n_rows, sets, m, arithmetic in (
            ("next_matvec_q4_k_bf16_ffn", hc.GgufQuantizedType.kQ4K, 144, 2048, 6144, 80, 1, EXACT),
            ("next_matvec_q4_k_bf16_ffn_down", hc.GgufQuantizedType.kQ4K, 144, 6144, 2048, 80, 1, EXACT),
            ("next_matvec_q4_k_bf16_k4096", hc.GgufQuantizedType.kQ4K, 144, 4096, 14336, 16, 1, EXACT),
            ("next_matvec_q4_k_bf16_vocab", hc.GgufQuantizedType.kQ4K, 144, 2048, 151936, 4, 1, EXACT),
            ("next_matvec_q6_k_bf16_vocab", hc.GgufQuantizedType.kQ6K, 210, 2048, 151936, 3, 1, EXACT),
            ("next_matvec_q6_k_bf16_vocab_4_tokens", hc.GgufQuantizedType.kQ6K, 210, 2048, 151936, 3, 4, EXACT),
            ("next_matvec_q8_0_bf16_vocab", hc.GgufQuantizedType.kQ8_0, 34, 2048, 151936, 3, 1, EXACT),
            # the same products as the reference's ggml route computes them: 8-bit activation blocks, integer dots
            ("next_matvec_ggml_q8_q4_k_ffn", hc.GgufQuantizedType.kQ4K, 144, 2048, 6144, 80, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_ffn_down", hc.GgufQuantizedType.kQ4K, 144, 6144, 2048, 80, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_vocab", hc.GgufQuantizedType.kQ4K, 144, 2048, 151936, 4, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_vocab_4_tokens", hc.GgufQuantizedType.kQ4K, 144, 2048, 151936, 4, 4, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_vocab_8_tokens", hc.GgufQuantizedType.kQ4K, 144, 2048, 151936, 4, 8, GGML_Q8),
            ("next_matvec_ggml_q8_q6_k_vocab", hc.GgufQuantizedType.kQ6K, 210, 2048, 151936, 3, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q6_k_vocab_4_tokens", hc.GgufQuantizedType.kQ6K, 210, 2048, 151936, 3, 4, GGML_Q8),
            ("next_matvec_ggml_q8_q6_k_vocab_8_tokens", hc.GgufQuantizedType.kQ6K, 210, 2048, 151936, 3, 8, GGML_Q8),
            ("next_matvec_ggml_q8_q8_0_vocab", hc.GgufQuantizedType.kQ8_0, 34, 2048, 151936, 3, 1, GGML_Q8),
            # the reference's own projection shapes (tests/compute_models/cpu_c5_gguf_inputs.h:231-314): widths that
            # are no multiple of 2048 (Q8_0: the span kernel with a short last span; Q4_K: the matrix-unit kernel)
            ("next_matvec_ggml_q8_q8_0_1024_to_32768", hc.GgufQuantizedType.kQ8_0, 34, 1024, 32768, 16, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_5120_to_10240", hc.GgufQuantizedType.kQ4K, 144, 5120, 10240, 18, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q8_0_7168_to_3072", hc.GgufQuantizedType.kQ8_0, 34, 7168, 3072, 24, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q8_0_17408_to_5120", hc.GgufQuantizedType.kQ8_0, 34, 17408, 5120, 6, 1, GGML_Q8),
            ("next_matvec_ggml_q8_q4_k_5120_to_10240_4_tokens", hc.GgufQuantizedType.kQ4K, 144, 5120, 10240, 18, 4, GGML_Q8)):
        if not want(name):
            continue
        per_row = k // (32 if block_bytes == 34 else 256)   # blocks in a row of k values

        def set_mv(i, block_bytes=block_bytes, n_rows=n_rows, per_row=per_row, k=k, m=m):
            raw = torch.randint(0, 256, (n_rows, per_row * block_bytes), dtype=torch.uint8)
            fields = raw.view(n_rows, per_row, block_bytes)
            for at in {144: (1, 3), 210: (209,), 34: (1,)}[block_bytes]:   # finite f16 scales
                fields[:, :, at] &= 0x3B
            x = torch.empty([k] if m == 1 else [m, k], dtype=torch.bfloat16, device=dev).normal_()
            return [raw.to(dev), x], [torch.empty([n_rows] if m == 1 else [m, n_rows], dtype=torch.bfloat16, device=dev)]
        ops.append(Op(name, hc.GgufMatVec(arithmetic), [hc.TensorDesc.gguf_weight(gguf, BF, k, n_rows), D(BF, [k] if m == 1 else [m, k])],
                      set_mv, sets, n_rows * (per_row * block_bytes + 2 * m) + m * k * 2, m * n_rows * k, "u8/bf16", in_step=False))
    # ---- the next row of the path: Cast and Copy, timed beside the step -------------------------
    if want("next_cast_f32_to_bf16") or want("next_cast_bf16_to_f32"):
        x32 = np.random.default_rng(5).normal(0, 2, (8192, 2048)).astype(np.float32)

        def set_narrow(i):
            dx = torch.from_numpy(np.roll(x32, i, axis=0)).to(dev)
            return [dx], [torch.empty((8192, 2048), dtype=torch.bfloat16, device=dev)]

        def set_widen(i):
            dx = torch.from_numpy(np.roll(x32, i, axis=0)).to(dev).to(torch.bfloat16)
            return [dx], [torch.empty((8192, 2048), dtype=torch.float32, device=dev)]
        if want("next_cast_f32_to_bf16"):
            ops.append(Op("next_cast_f32_to_bf16", hc.Cast(BF), [D(F32, [8192, 2048])], set_narrow, 6,
                          8192 * 2048 * 6, 8192 * 2048, "f32->bf16", in_step=False))
        if want("next_cast_bf16_to_f32"):
            ops.append(Op("next_cast_bf16_to_f32", hc.Cast(F32), [D(BF, [8192, 2048])], set_widen, 6,
                          8192 * 2048 * 6, 8192 * 2048, "bf16->f32", in_step=False))
    if want("next_layer_norm_bf16"):
        xl, wl_ = wl.config2()
        bias_bits = wl.config2(rows=1)[0].reshape(-1)  # any bf16 vector of the right length

        def set_ln(i):
            dx = bf16(np.roll(xl, i, axis=0))
            return [dx, bf16(wl_), bf16(bias_bits)], [torch.empty_like(dx)]
        ops.append(Op("next_layer_norm_bf16", hc.LayerNorm(epsilon=1e-6),
                      [D(BF, [8192, 2048]), D(BF, [2048]), D(BF, [2048])], set_ln, 10,
                      2 * 8192 * 2048 * 2 + 2 * 4096, 8192 * 2048, "bf16", in_step=False))
    if want("next_softmax_bf16_unmasked"):
        # attention rows without a mask (a decode step over its cache, an encoder): [4096, 4096] bf16
        def set_rows(i):
            dx = torch.empty((4096, 4096), dtype=torch.bfloat16, device=dev).normal_(0.0, 3.0)
            return [dx], [torch.empty_like(dx)]
        ops.append(Op("next_softmax_bf16_unmasked", hc.Softmax(), [D(BF, [4096, 4096])], set_rows, 10,
                      2 * 4096 * 4096 * 2, 4096 * 4096, "bf16", in_step=False, ceiling="ceiling_copy_67mb"))
    # the norms at other hidden sizes (the same 67 MB): launch shapes that cover the tensor exactly
    for name, layer, rows_n, hidden_n in (("next_rms_norm_bf16_hidden_4096", False, 4096, 4096),
                                         ("next_layer_norm_bf16_hidden_8192", True, 2048, 8192)):
        if not want(name):
            continue

        def set_wide(i, layer=layer, rows_n=rows_n, hidden_n=hidden_n):
            dx = torch.empty((rows_n, hidden_n), dtype=torch.bfloat16, device=dev).normal_()
            scale = torch.empty(hidden_n, dtype=torch.bfloat16, device=dev).normal_(1.0, 0.1)
            return ([dx, scale, scale.clone()] if layer else [dx, scale]), [torch.empty_like(dx)]
        descs = [D(BF, [rows_n, hidden_n]), D(BF, [hidden_n])] + ([D(BF, [hidden_n])] if layer else [])
        ops.append(Op(name, hc.LayerNorm(epsilon=1e-6) if layer else hc.RmsNorm(epsilon=1e-6), descs, set_wide, 10,
                      2 * rows_n * hidden_n * 2 + (2 if layer else 1) * hidden_n * 2, rows_n * hidden_n, "bf16",
                      in_step=False, ceiling="ceiling_copy_67mb"))
    if want("next_geglu_tanh_bf16") or want("next_gelu_bf16"):
        gate_g, up_g = wl.config3_swiglu()

        def set_geglu(i):
            dg, du = bf16(np.roll(gate_g, i, axis=0)), bf16(np.roll(up_g, i, axis=0))
            return [dg, du], [torch.empty_like(dg)]

        def set_gelu(i):
            dg = bf16(np.roll(gate_g, i, axis=0))
            return [dg], [torch.empty_like(dg)]
        if want("next_geglu_tanh_bf16"):
            ops.append(Op("next_geglu_tanh_bf16",
                          hc.GatedActivation(hc.GatedActivationKind.kGeluTanh, hc.GatedInputKind.kSeparate),
                          [D(BF, [8192, 6144]), D(BF, [8192, 6144])], set_geglu, 3,
                          3 * 8192 * 6144 * 2, 8192 * 6144, "bf16", in_step=False))
        if want("next_gelu_bf16"):
            ops.append(Op("next_gelu_bf16", hc.Unary(hc.UnaryKind.kGelu), [D(BF, [8192, 6144])], set_gelu, 3,
                          2 * 8192 * 6144 * 2, 8192 * 6144, "bf16", in_step=False))
    # Reduce over the innermost axis, over the leading axis and over every axis (two dispatches
    # that meet in the workspace when there are too few results to fill the chip).
    reduce_lines = (
        ("next_reduce_sum_rows_bf16", hc.ReductionKind.kSum, [-1], BF, torch.bfloat16, [8192, 2048], 16, 2 * 8192, "ceiling_scan_38mb"),
        ("next_reduce_sum_columns_bf16", hc.ReductionKind.kSum, [0], BF, torch.bfloat16, [8192, 2048], 16, 2 * 2048, "ceiling_scan_38mb"),
        ("next_reduce_max_all_f32", hc.ReductionKind.kMaximum, None, F32, torch.float32, [4096, 4096], 8, 4, "ceiling_scan_67mb"),
    )
    for name, kind, axes, dtype, torch_dtype, dims, sets, out_bytes, ceiling in reduce_lines:
        if not want(name):
            continue

        def set_reduce(i, dims=dims, torch_dtype=torch_dtype, axes=axes):
            src = torch.empty(dims, dtype=torch_dtype, device=dev).normal_()
            shape = [] if axes is None else [d for a, d in enumerate(dims) if a != axes[0] % len(dims)]
            return [src], [torch.empty(shape, dtype=torch_dtype, device=dev)]
        size = 4 if dtype == F32 else 2
        ops.append(Op(name, hc.Reduce(kind, hc.Axes.all() if axes is None else hc.Axes.from_(axes),
                                      accumulation_type=F32),
                      [D(dtype, dims)], set_reduce, sets, dims[0] * dims[1] * size + out_bytes, dims[0] * dims[1],
                      "f32" if dtype == F32 else "bf16", in_step=False, ceiling=ceiling))
    if want("next_topk64_f32"):
        def set_topk(i):
            logits = torch.empty((64, 151936), dtype=torch.float32, device=dev).normal_()
            return [logits], [torch.empty((64, 64), dtype=torch.float32, device=dev),
                              torch.empty((64, 64), dtype=torch.int32, device=dev)]
        ops.append(Op("next_topk64_f32", hc.TopK(count=64), [D(F32, [64, 151936])], set_topk, 14,
                      64 * 151936 * 4 + 64 * 64 * 8, 64 * 151936, "f32", in_step=False, ceiling="ceiling_scan_38mb"))
    if want("next_copy_bf16"):
        def set_copy(i):
            src = torch.empty((8192, 6144), dtype=torch.bfloat16, device=dev).normal_()
            return [src], [torch.empty_like(src)]
        ops.append(Op("next_copy_bf16", hc.Copy(), [D(BF, [8192, 6144])], set_copy, 3,
                      8192 * 6144 * 4, 8192 * 6144, "bf16", in_step=False))
    if want("next_fill_bf16"):
        def set_fill(i):
            return [], [torch.empty((8192, 6144), dtype=torch.bfloat16, device=dev)]
        ops.append(Op("next_fill_bf16", hc.Fill((8192, 6144), BF, hc.ScalarValue.of(BF, 1.0)), [], set_fill, 3,
                      8192 * 6144 * 2, 8192 * 6144, "bf16", in_step=False))
    if want("next_select_bf16"):
        # the masked residual: Bool mask, a full branch, a rank-0 zero (1 + 2 bytes read, 2 written per element)
        def set_select(i):
            mask = torch.empty((8192, 6144), dtype=torch.uint8, device=dev).random_(0, 2)
            src = torch.empty((8192, 6144), dtype=torch.bfloat16, device=dev).normal_()
            return [mask, src, torch.zeros((), dtype=torch.bfloat16, device=dev)], [torch.empty_like(src)]
        ops.append(Op("next_select_bf16", hc.Select(), [D(hc.DataType.kBool, [8192, 6144]), D(BF, [8192, 6144]), D(BF, [])],
                      set_select, 3, 8192 * 6144 * 5, 8192 * 6144, "bf16", in_step=False))
    if want("next_concat_bf16"):
        # a join along the last axis: rows of 4 KiB and 8 KiB interleaved into rows of 12 KiB
        def set_concat(i):
            left = torch.empty((8192, 2048), dtype=torch.bfloat16, device=dev).normal_()
            right = torch.empty((8192, 4096), dtype=torch.bfloat16, device=dev).normal_()
            return [left, right], [torch.empty((8192, 6144), dtype=torch.bfloat16, device=dev)]
        ops.append(Op("next_concat_bf16", hc.Concat(-1), [D(BF, [8192, 2048]), D(BF, [8192, 4096])], set_concat, 3,
                      8192 * 6144 * 4, 8192 * 6144, "bf16", in_step=False))
    if want("next_gather_bf16") or want("next_gather_unchecked_bf16") or want("next_gather_last_rows_bf16"):
        # the embedding lookup: 8192 rows of 4 KiB picked from a [151936, 2048] table by Int32 ids; one
        # table for both lines (622 MB).  Checked bounds add the dispatch that looks at every id.
        table = torch.empty((151936, 2048), dtype=torch.bfloat16, device=dev).normal_()
        def set_gather(i):
            ids = torch.randint(0, 151936, (8192,), dtype=torch.int32, device=dev)
            return [table, ids], [torch.empty((8192, 2048), dtype=torch.bfloat16, device=dev)]
        gather_bytes = 8192 * 2048 * 4 + 8192 * 4
        if want("next_gather_bf16"):
            ops.append(Op("next_gather_bf16", hc.Gather(0), [D(BF, [151936, 2048]), D(hc.DataType.kInt32, [8192])], set_gather,
                          8, gather_bytes + 8192 * 4, 8192 * 2048, "bf16", in_step=False, ceiling="ceiling_copy_67mb"))
        if want("next_gather_last_rows_bf16"):
            # what a step does for its last tokens: 64 checked row picks out of [8192, 2048] hidden states
            hidden = torch.empty((8192, 2048), dtype=torch.bfloat16, device=dev).normal_()
            def set_last(i):
                ids = torch.randint(0, 8192, (64,), dtype=torch.int32, device=dev)
                return [hidden, ids], [torch.empty((64, 2048), dtype=torch.bfloat16, device=dev)]
            ops.append(Op("next_gather_last_rows_bf16", hc.Gather(0), [D(BF, [8192, 2048]), D(hc.DataType.kInt32, [64])], set_last,
                          8, 64 * 2048 * 4 + 64 * 4, 64 * 2048, "bf16", in_step=False))
        if want("next_gather_unchecked_bf16"):
            ops.append(Op("next_gather_unchecked_bf16", hc.Gather(0, hc.IndexBoundsPolicy.kUnchecked),
                          [D(BF, [151936, 2048]), D(hc.DataType.kInt32, [8192])], set_gather, 8, gather_bytes, 8192 * 2048,
                          "bf16", in_step=False, ceiling="ceiling_copy_67mb"))
    if want("next_rope_bf16"):
        # the queries of a prefill: [1, 8192, 16, 128] bf16 rotated in the half-split layout, one position per step
        def set_rope(i):
            x = torch.empty((1, 8192, 16, 128), dtype=torch.bfloat16, device=dev).normal_()
            positions = torch.arange(8192, dtype=torch.int32, device=dev)
            frequencies = (1000000.0 ** (-torch.arange(64, dtype=torch.float32, device=dev) / 64.0)).contiguous()
            return [x, positions, frequencies], [torch.empty_like(x)]
        ops.append(Op("next_rope_bf16", hc.RoPE(128, 1, hc.RopeLayout.kHalfSplit),
                      [D(BF, [1, 8192, 16, 128]), D(hc.DataType.kInt32, [8192]), D(F32, [64])], set_rope, 10,
                      8192 * 16 * 128 * 4 + 8192 * 4 + 256, 8192 * 16 * 128, "bf16", in_step=False, ceiling="ceiling_copy_67mb"))
    if want("next_categorical_f32"):
        # one draw per row of the argmax shape, with the selected log probability: the row is read once
        def set_categorical(i):
            logits = torch.empty((64, 151936), dtype=torch.float32, device=dev).normal_(0, 3)
            ids = torch.randint(0, 1 << 31, (64, 4), dtype=torch.int64, device=dev).to(torch.int32)
            return [logits, ids], [torch.empty(64, dtype=torch.int32, device=dev), torch.empty(64, dtype=torch.float32, device=dev)]
        ops.append(Op("next_categorical_f32", hc.Categorical(True), [D(F32, [64, 151936]), D(hc.DataType.kUInt32, [64, 4])],
                      set_categorical, 16, 64 * 151936 * 4 + 64 * 24, 64 * 151936, "f32", in_step=False,
                      ceiling="ceiling_scan_38mb"))
    if want("next_random_bits_u32"):
        # Philox4x32-10 words: ten rounds of two 32 x 32 -> 64 products per 16 bytes written
        def set_bits(i):
            ids = torch.randint(0, 1 << 31, (4096, 4), dtype=torch.int64, device=dev).to(torch.int32)
            return [ids], [torch.empty((4096, 4096), dtype=torch.int32, device=dev)]
        ops.append(Op("next_random_bits_u32", hc.RandomBits(4096), [D(hc.DataType.kUInt32, [4096, 4])], set_bits, 4,
                      4096 * 4096 * 4 + 4096 * 16, 4096 * 4096, "u32", in_step=False))
    # ---- practical ceilings for launches of 38 / 67 MB: a plain copy and a plain read-only scan (a
    # row maximum, one wave per row, one dispatch) of the traffic of the step's small shapes, through
    # the same C ABI and rotated the same way.  Kernels of this size run for 6 - 12 us, of which the
    # start and the drain of the launch are a fixed part no kernel avoids; `frac_of_ceiling` of a
    # small op is its GB/s over the GB/s of the plain kernel named in `ceiling`.
    ceiling_lines = (
        ("ceiling_copy_38mb", "copy", BF, torch.bfloat16, [4712, 2048], 16),
        ("ceiling_copy_67mb", "copy", F32, torch.float32, [4096, 2048], 10),
        ("ceiling_scan_38mb", "scan", F32, torch.float32, [9496, 1024], 16),
        ("ceiling_scan_67mb", "scan", F32, torch.float32, [16384, 1024], 10),
        # the same read-only kernel far above the 256 MB memory-side cache: does a launch that only reads
        # saturate where the small ones do, or higher?
        ("ceiling_scan_1gib", "scan", F32, torch.float32, [262144, 1024], 2),
    )
    needed = {o.ceiling for o in ops if o.ceiling}
    for name, form, dtype, torch_dtype, dims, sets in ceiling_lines:
        if not (want(name) if wanted else True) and name not in needed:
            continue
        size = 4 if dtype == F32 else 2
        if form == "copy":
            def set_plain(i, dims=dims, torch_dtype=torch_dtype):
                src = torch.empty(dims, dtype=torch_dtype, device=dev).normal_()
                return [src], [torch.empty_like(src)]
            ops.append(Op(name, hc.Copy(), [D(dtype, dims)], set_plain, sets, 2 * dims[0] * dims[1] * size,
                          dims[0] * dims[1], "bf16" if dtype == BF else "f32", in_step=False))
        else:
            def set_plain(i, dims=dims, torch_dtype=torch_dtype):
                src = torch.empty(dims, dtype=torch_dtype, device=dev).normal_()
                return [src], [torch.empty(dims[:1], dtype=torch_dtype, device=dev)]
            ops.append(Op(name, hc.Reduce(hc.ReductionKind.kMaximum, hc.Axes.from_([-1]), accumulation_type=F32),
                          [D(dtype, dims)], set_plain, sets, dims[0] * dims[1] * size + dims[0] * size,
                          dims[0] * dims[1], "f32", in_step=False))
    if not any(o.in_step for o in ops):
        print("no kernel of the step selected", file=sys.stderr)
        return 2

    step_ops = [o for o in ops if o.in_step]
    dominant = max(step_ops, key=lambda o: o.bytes)
    step_bytes = sum(o.bytes for o in step_ops)
    step_credited = sum(o.credited for o in step_ops)
    step_elements = sum(o.elements for o in step_ops)
    before = step_ops[:step_ops.index(dominant)]
    after = step_ops[step_ops.index(dominant) + 1:]

    # Every kernel runs once eagerly (code objects load on first use), then the short
    # kernels are captured into HIP graphs: their 5-50 us run times are of the order of
    # one launch call, so eager submission would measure the host, not the GPU.  The
    # reference replays captured graphs the same way (capture_compatible,
    # include/hyle/compute/provider.h:136-139).  One graph per rotation phase.
    # The first launch of a kernel out of each source file of the library also loads that file's code
    # object (the reference's contract: "kernel/configuration binding is cold",
    # include/hyle/compute/providers/cuda.h:55-56): each op's first launch is timed to its completion.
    torch.cuda.synchronize()
    for op in ops:
        began = time.perf_counter()
        op.launch(stream)
        op.variant = hc.last_launch_variant()
        torch.cuda.synchronize()
        op.first_launch_us = (time.perf_counter() - began) * 1e6
    PHASES = 16

    def capture(members, launches_each=1):
        graphs = []
        if not members:
            return graphs
        for _ in range(PHASES if launches_each == 1 else 1):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                s = torch.cuda.current_stream().cuda_stream
                for _ in range(launches_each):
                    for op in members:
                        op.launch(s)
            graphs.append(g)
        return graphs

    graphs_before, graphs_after = capture(before), capture(after)

    def step(i, events=None):
        if graphs_before:
            graphs_before[i % PHASES].replay()
        if events is not None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            dominant.launch(stream)
            e1.record()
            events.append((e0, e1))
        else:
            dominant.launch(stream)
        if graphs_after:
            graphs_after[i % PHASES].replay()

    # ---- whole-step timing ----------------------------------------------------------------
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i, events)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    dominant_us = sum(a.elapsed_time(b) for a, b in events) * 1e3 / len(events)

    # ---- per-kernel timing: a graph of back-to-back launches between two HIP events ---------
    per_op = []
    for op in ops:
        reps = args.op_reps if op.bytes < (1 << 30) else max(10, args.op_reps // 10)
        (graph,) = capture([op], launches_each=reps)
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        gbps = op.credited / us / 1e3
        entry = {"op": op.name, "in_step": op.in_step, "route": op.route, "variant": op.variant, "dtype": op.dtype,
                 "plan_us": round(op.plan_us, 1), "first_launch_us": round(op.first_launch_us, 1),
                 "bytes": op.bytes, "bytes_credited": op.credited,
                 "buffer_sets": len(op.sets), "launches": reps, "us": round(us, 3),
                 "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4),
                 "gelem_per_s": round(op.elements / us / 1e3, 2)}
        del graph
        if op.in_step and len(op.sets) > 1:
            # the same launches on one buffer set: operands served by the 256 MB memory-side cache
            cached = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cached):
                s = torch.cuda.current_stream().cuda_stream
                for _ in range(reps):
                    op.launch_first_set(s)
            cached.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            cached.replay()
            e1.record()
            torch.cuda.synchronize()
            us_cached = e0.elapsed_time(e1) * 1e3 / reps
            entry["us_cached"] = round(us_cached, 3)
            entry["gbps_cached"] = round(op.credited / us_cached / 1e3, 1)
            del cached
        per_op.append(entry)

    by_name = {entry["op"]: entry for entry in per_op}
    for op in ops:
        if op.ceiling and op.ceiling in by_name:
            entry, plain = by_name[op.name], by_name[op.ceiling]
            entry["ceiling"] = op.ceiling
            entry["ceiling_gbps"] = plain["gbps"]
            entry["frac_of_ceiling"] = round(entry["gbps"] / plain["gbps"], 4)

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)  # one elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    achieved = dominant.credited / dominant_us / 1e3
    # every kernel of the step in short keys (us per launch, GB/s of credited bytes, fraction of the
    # 8 TB/s peak, and against the plain kernel of the same traffic where one was timed)
    per_config = {}
    for op in step_ops:
        entry = by_name[op.name]
        line = {"us": entry["us"], "gbps": entry["gbps"], "frac": entry["frac"]}
        if "ceiling" in entry:
            line["ceiling"] = entry["ceiling"]
            line["ceiling_gbps"] = entry["ceiling_gbps"]
            line["frac_of_ceiling"] = entry["frac_of_ceiling"]
        per_config[op.name] = line
    ceilings = {entry["op"]: {"us": entry["us"], "gbps": entry["gbps"], "frac": entry["frac"]}
                for entry in per_op if entry["op"].startswith("ceiling_")}
    cold = {"first_launch_ms_max": round(max(o.first_launch_us for o in ops) / 1e3, 2),
            "first_launch_ms": {o.name: round(o.first_launch_us / 1e3, 2) for o in step_ops},
            "plan_create_us_max": round(max(o.plan_us for o in ops), 1)}
    result = {
        "metric": "achieved HBM GB/s and % of 8 TB/s peak per op (RMSNorm, SwiGLU, softmax)",
        "value": round(step_credited / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32+bf16+u8", "data": "synthetic",
        "config": {"workload": "one pass over the largest shape of configs 1-5: " + ", ".join(o.name for o in step_ops),
                   "algorithmic_bytes_per_step": step_bytes, "credited_bytes_per_step": step_credited,
                   "credit_rule": "GB/s figures use credited bytes = algorithmic bytes minus the loads of fully "
                                  "masked vectors the Boolean-mask softmax never issues",
                   "elements_per_step": step_elements,
                   "gelem_per_s": round(step_elements / (ms_per_step * 1e-3) / 1e9, 2),
                   "buffer_rotation": "shapes under 256 MB rotate over buffer sets totalling > 512 MB"},
        "roofline": {"bound": "hbm", "kernel": dominant.name, "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "us_per_launch": round(dominant_us, 2), "algorithmic_bytes": dominant.bytes,
                     "credited_bytes": dominant.credited, "traffic": TRAFFIC.get(dominant.name),
                     "traffic_source": "profiles/hot_path_step_hbm_traffic_pmc.md (rocprofv3 --pmc FETCH_SIZE / "
                                       "WRITE_SIZE of an earlier run of this script: a recorded figure, not a "
                                       "counter read in this run)",
                     "per_config": per_config, "ceilings": ceilings},
        "cold": cold,
        "per_op": per_op,
    }
    result["device"] = device_state(torch)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args, step_ops, np, torch, wl)
    if args.file_stream_mib > 0:
        result["file_stream"] = file_stream_rate(args.file_stream_mib, ctx, torch, dev)
    print(json.dumps(result))
    return 0


def device_state(torch):
    """Name, compute units and the clock and power state the driver shows in sysfs during the run
    (plain file reads: no child process is started from a process that holds the GPU)."""
    import glob
    props = torch.cuda.get_device_properties(0)
    state = {"name": props.name, "compute_units": props.multi_processor_count,
             "memory_gib": round(props.total_memory / 2 ** 30, 1)}

    def active_level(path):
        # pp_dpm_* list one level per line, the active one marked with "*"
        with open(path) as levels:
            marked = [line.split(":", 1)[1].replace("*", "").strip() for line in levels if "*" in line]
        return marked[0] if marked else None

    sysfs = {}
    for card in sorted(glob.glob("/sys/class/drm/card[0-9]*/device")):
        try:
            with open(card + "/vendor") as vendor:
                if vendor.read().strip() != "0x1002":
                    continue
            entry = {}
            for name in ("pp_dpm_sclk", "pp_dpm_mclk", "pp_dpm_fclk"):
                try:
                    entry[name[len("pp_dpm_"):]] = active_level(f"{card}/{name}")
                except OSError:
                    pass
            try:
                with open(card + "/power_dpm_force_performance_level") as level:
                    entry["performance_level"] = level.read().strip()
            except OSError:
                pass
            if entry:
                sysfs[card.split("/")[4]] = entry
        except OSError:
            continue
    state["sysfs"] = sysfs if sysfs else "unavailable"
    return state


def file_stream_rate(mib, ctx, torch, dev):
    """File (page cache) -> pinned staging -> HBM through the pipeline of include/hyle_hip_stream.h."""
    import tempfile
    from hyle_amd import file_stream as fs
    total = mib << 20
    chunk = torch.randint(0, 256, (min(total, 64 << 20),), dtype=torch.uint8)
    with tempfile.NamedTemporaryFile(delete=False) as handle:
        path = handle.name
        written = 0
        while written < total:
            piece = min(total - written, chunk.numel())
            handle.write(chunk.numpy()[:piece].tobytes())
            written += piece
    fd = os.open(path, os.O_RDONLY)
    try:
        target = torch.empty(total, dtype=torch.uint8, device=dev)
        best = {}
        for slots, slot_mib in ((2, 1), (4, 8), (4, 32)):
            pipeline = fs.FileResourcePipeline.create(ctx, fs.FileStreamOptions(slots, slot_mib << 20))
            stream = torch.cuda.current_stream().cuda_stream
            seconds = []
            for _ in range(3):
                torch.cuda.synchronize()
                begin = time.perf_counter()
                pipeline.read(fd, [fs.StreamReadRange(0, target.data_ptr(), total)], stream)
                pipeline.wait()
                seconds.append(time.perf_counter() - begin)
            pipeline.close()
            best[f"{slots}x{slot_mib}MiB"] = round(total / min(seconds) / 1e9, 2)
        ok = bool((target[:chunk.numel()].cpu() == chunk[:min(total, chunk.numel())]).all())
        return {"bytes": total, "unit": "GB/s", "rates": best, "bytes_identical": ok,
                "note": "file in the page cache; pread on one thread overlapped with the copies of the other slots"}
    finally:
        os.close(fd)
        os.unlink(path)


# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script
# (profiles/hot_path_step_hbm_traffic_pmc.md: FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0, the factors
# the same counters need to read a plain 1 GiB copy correctly).
TRAFFIC = {
    "cfg4_softmax_f32_causal": 3256527872,
    "cfg4_softmax_f32_causal_additive": 4362134118,
    "cfg3_swiglu_bf16": 302044160,
    "cfg3_residual_add_bf16": 100732518,
    "cfg1_broadcast_add_mul_f32": 67312742,
    "cfg2_rmsnorm_bf16": 67252838,
    "cfg4_argmax_f32": 39140659,
    "cfg5_q8_0_dequant_sumsq": 38641869,
}


def cpu_baseline(args, ops, np, torch, wl):
    """Times the CPU oracle's dense row loops (the "port" of the reference's CPU provider path)
    on a bounded sample of each kernel's workload, rows fanned out over threads with the
    reference's rule: tasks = min(cores, rows, ceil(rows * width / 16384)), contiguous ranges,
    remainder over the first tasks (src/compute_provider_native/native_provider.cc:47-69,
    native_plan.h:74-111)."""
    import ctypes as C

    from oracle import lib as orc

    lib = C.CDLL(os.path.join(ROOT, "oracle", "libhyle_oracle.so"))
    vp, sz = C.c_void_p, C.c_size_t
    THREAD_CAP = 16  # the CPU share of a one-GPU box, whatever the host shows
    cores = min(len(os.sched_getaffinity(0)), THREAD_CAP)
    pool = ThreadPoolExecutor(max_workers=cores)

    def ptr(a):
        return a.ctypes.data_as(vp)

    def fan_out(rows, width, call):
        tasks = max(1, min(cores, rows, -(-rows * width // 16384)))
        base, rem = divmod(rows, tasks)
        ranges, begin = [], 0
        for i in range(tasks):
            end = begin + base + (1 if i < rem else 0)
            ranges.append((begin, end))
            begin = end
        list(pool.map(lambda be: call(*be), ranges))

    def timed(rows_full, width, bytes_full, make_call):
        """Grow the sample until it costs about --cpu-seconds; return (rows, seconds)."""
        rows = max(cores, min(rows_full, 64))
        while True:
            call = make_call(rows)
            t0 = time.perf_counter()
            fan_out(rows, width, call)
            dt = time.perf_counter() - t0
            if dt >= args.cpu_seconds * 0.5:
                return rows, dt
            if rows == rows_full:
                # the whole shape costs less than the target: repeat it
                passes = max(2, int(args.cpu_seconds / max(dt, 1e-4)))
                t0 = time.perf_counter()
                for _ in range(passes):
                    fan_out(rows, width, call)
                return rows * passes, time.perf_counter() - t0
            grow = max(2.0, min(16.0, args.cpu_seconds / max(dt, 1e-4)))
            rows = int(min(rows_full, rows * grow))

    names = {o.name for o in ops}
    samples, total_seconds_full = [], 0.0

    def record(name, rows_full, rows, dt, bytes_full):
        nonlocal total_seconds_full
        full = dt * rows_full / rows
        total_seconds_full += full
        samples.append(f"{name}: {rows}/{rows_full} rows in {dt:.2f}s = {bytes_full * rows / rows_full / dt / 1e9:.2f} GB/s")

    if "cfg1_broadcast_add_mul_f32" in names:
        a, b, s = wl.config1()
        out = np.empty_like(a)
        fn = lib.hyle_oracle_rows_add_row_scale_f32
        fn.argtypes = [vp, vp, C.c_float, vp, sz, sz, sz]
        rows, dt = timed(4096, 2048, 0, lambda n: (lambda b0, e0: fn(ptr(a), ptr(b), 0.5, ptr(out), 2048, b0, e0)))
        record("cfg1", 4096, rows, dt, wl.ALGORITHMIC_BYTES["cfg1_broadcast_add_mul_f32"])
    if "cfg2_rmsnorm_bf16" in names:
        x, w = wl.config2()
        out = np.empty_like(x)
        fn = lib.hyle_oracle_rows_rms_norm_bf16
        fn.argtypes = [vp, vp, vp, sz, C.c_float, sz, sz]
        rows, dt = timed(8192, 2048, 0, lambda n: (lambda b0, e0: fn(ptr(x), ptr(w), ptr(out), 2048, 1e-6, b0, e0)))
        record("cfg2", 8192, rows, dt, wl.ALGORITHMIC_BYTES["cfg2_rmsnorm_bf16"])
    if "cfg3_swiglu_bf16" in names:
        gate, up = wl.config3_swiglu(rows=2048)
        out = np.empty_like(gate)
        fn = lib.hyle_oracle_rows_swiglu_bf16
        fn.argtypes = [vp, vp, vp, sz, sz, sz]
        rows, dt = timed(2048, 6144, 0, lambda n: (lambda b0, e0: fn(ptr(gate), ptr(up), ptr(out), 6144, b0, e0)))
        record("cfg3", 8192, rows, dt, wl.ALGORITHMIC_BYTES["cfg3_swiglu_bf16"])
    if "cfg3_residual_add_bf16" in names:
        r, y = wl.config3_residual()
        out = np.empty_like(r)
        fn = lib.hyle_oracle_rows_add_bf16
        fn.argtypes = [vp, vp, vp, sz, sz, sz]
        rows, dt = timed(8192, 2048, 0, lambda n: (lambda b0, e0: fn(ptr(r), ptr(y), ptr(out), 2048, b0, e0)))
        record("cfg3r", 8192, rows, dt, wl.ALGORITHMIC_BYTES["cfg3_residual_add_bf16"])
    if "cfg4_softmax_f32_causal" in names:
        srows = 4096  # the last query rows of head 0: full-length causal rows, the costliest kind
        s4, mask = wl.config4_softmax(heads=1, seq=4096)
        x4 = s4.reshape(4096, 4096)
        out = np.empty_like(x4)
        fn = lib.hyle_oracle_rows_softmax_bool_f32
        fn.argtypes = [vp, vp, vp, sz, sz, sz, sz]
        rows, dt = timed(srows, 4096, 0, lambda n: (lambda b0, e0: fn(ptr(x4), ptr(mask), ptr(out), 4096, 4096, b0, e0)))
        record("cfg4", 32 * 4096, rows, dt, wl.ALGORITHMIC_BYTES["cfg4_softmax_f32_causal"])
    if "cfg4_argmax_f32" in names:
        logits = wl.config4_argmax()
        values, indices = np.empty(64, np.float32), np.empty(64, np.int32)
        fn = lib.hyle_oracle_rows_topk1_f32
        fn.argtypes = [vp, vp, vp, sz, sz, sz]
        rows, dt = timed(64, 151936, 0, lambda n: (lambda b0, e0: fn(ptr(logits), ptr(values), ptr(indices), 151936, b0, e0)))
        record("cfg4a", 64, rows, dt, wl.ALGORITHMIC_BYTES["cfg4_argmax_f32"])
    if "cfg5_q8_0_dequant_sumsq" in names:
        blocks = wl.config5()
        out, sumsq = np.empty((6144, 2048), np.uint16), np.empty(6144, np.float32)
        fn = lib.hyle_oracle_rows_q8_0_bf16
        fn.argtypes = [vp, vp, vp, sz, sz, sz, sz]
        rows, dt = timed(6144, 2048, 0, lambda n: (lambda b0, e0: fn(ptr(blocks), ptr(out), ptr(sumsq), 2048, 2176, b0, e0)))
        record("cfg5", 6144, rows, dt, wl.ALGORITHMIC_BYTES["cfg5_q8_0_dequant_sumsq"])
    pool.shutdown()
    step_bytes = sum(o.bytes for o in ops)
    return {"value": round(step_bytes / total_seconds_full / 1e9, 3), "unit": "GB/s", "cores": cores,
            "thread_cap": THREAD_CAP, "host_cores_visible": len(os.sched_getaffinity(0)),
            "kind": "port",
            "build": "oracle/hyle_oracle.c, gcc -O3 -march=x86-64-v3 -ffp-contract=off (AVX2 + FMA, not "
                     "-march=native: the library is built before it travels to this host)",
            "sample": "row subsets of the same seeded inputs, per-kernel time scaled to the full shape; " + "; ".join(samples)}


if __name__ == "__main__":
    sys.exit(main())
