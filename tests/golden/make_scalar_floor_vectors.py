"""Writes tests/golden/scalar_floor_vectors.npz.

Inputs are generated here; expected outputs come from the reference's own scalar
semantic floor compiled from its sources (oracle/_ref, built by oracle/Makefile
where the reference tree is present).  The fixture holds data only: input and
output arrays.  It lets the oracle be checked bit for bit on machines where
oracle/_ref does not exist.

Run from the repo root:  python tests/golden/make_scalar_floor_vectors.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import ref  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scalar_floor_vectors.npz")

SPECIAL_F32 = np.array(
    [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38, 3.4028235e38,
     -3.4028235e38, 65504.0, 65520.0, 65519.996, 6.1035156e-05, 5.9604645e-08, 2.9802322e-08,
     2.9802326e-08, 8.940697e-08, 88.0, -88.0, -87.4, -103.0, -104.5, 20.0, -20.0, 0.5, -0.5],
    dtype=np.float32)


def main() -> None:
    if not ref.available():
        raise SystemExit("oracle/_ref is not built: run `make -C oracle` where the reference tree exists")
    rng = np.random.default_rng(20240607)
    out: dict[str, np.ndarray] = {}

    # codecs: boundary patterns in the discarded bits for every upper half would be
    # 393k values; keep a strided subset plus random words (bit patterns, so NaN
    # payloads survive)
    upper = np.arange(0, 65536, 7, dtype=np.uint32) << 16
    lower = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x0040, 0x1000, 0x2000, 0x3000],
                     dtype=np.uint32)
    words = (upper[:, None] | lower[None, :]).reshape(-1)
    words = np.concatenate([words, rng.integers(0, 2**32, 20000, dtype=np.uint64).astype(np.uint32),
                            SPECIAL_F32.view(np.uint32)])
    out["codec_f32_words"] = words
    out["codec_bf16_bits"] = ref.f32_to_bf16(words.view(np.float32))
    out["codec_f16_bits"] = ref.f32_to_f16(words.view(np.float32))
    all16 = np.arange(65536, dtype=np.uint16)
    out["codec_f16_all_to_f32_words"] = ref.f16_to_f32(all16).view(np.uint32)

    # activations
    x32 = np.concatenate([
        SPECIAL_F32,
        rng.normal(0, 2, 600).astype(np.float32),
        rng.uniform(-110, 110, 400).astype(np.float32),
        (-12.0 + 24.0 * np.arange(1, 258, dtype=np.float32) / np.float32(258)),
    ]).astype(np.float32)
    u32 = np.concatenate([rng.normal(0, 2, x32.size - 4).astype(np.float32),
                          np.array([np.inf, -np.inf, np.nan, 0.0], np.float32)])
    out["act_x_f32_words"] = x32.view(np.uint32)
    out["act_u_f32_words"] = u32.view(np.uint32)
    out["silu_f32_words"] = ref.silu(0, x32).view(np.uint32)
    out["swiglu_f32_words"] = ref.swiglu(0, x32, u32).view(np.uint32)
    xb = ref.f32_to_bf16(x32)
    ub = ref.f32_to_bf16(u32)
    xh = ref.f32_to_f16(x32)
    uh = ref.f32_to_f16(u32)
    out["act_x_bf16"], out["act_u_bf16"] = xb, ub
    out["act_x_f16"], out["act_u_f16"] = xh, uh
    out["silu_bf16"] = ref.silu(2, xb)
    out["silu_f16"] = ref.silu(1, xh)
    out["swiglu_bf16"] = ref.swiglu(2, xb, ub)
    out["swiglu_f16"] = ref.swiglu(1, xh, uh)
    # every bf16 gate pattern against a fixed up value of 1.0 (0x3F80)
    all_gate = np.arange(65536, dtype=np.uint16)
    out["silu_bf16_all"] = ref.silu(2, all_gate)

    # rms norm rows (one call per row in the reference's scalar floor)
    for n in (1, 7, 127, 128, 129, 257, 2048):
        row = (rng.normal(0, 1, n) * rng.uniform(0.1, 10)).astype(np.float32)
        w = rng.normal(1, 0.1, n).astype(np.float32)
        out[f"rms_x_f32_{n}"] = row
        out[f"rms_w_f32_{n}"] = w
        out[f"rms_y_f32_{n}"] = ref.rms_norm_row(0, row, w, 1e-6)
        out[f"rms_y_f32_nw_{n}"] = ref.rms_norm_row(0, row, None, 1e-5)
        rb, wb = ref.f32_to_bf16(row), ref.f32_to_bf16(w)
        out[f"rms_x_bf16_{n}"], out[f"rms_w_bf16_{n}"] = rb, wb
        out[f"rms_y_bf16_{n}"] = ref.rms_norm_row(2, rb, wb, 1e-6)
        rh, wh = ref.f32_to_f16(row), ref.f32_to_f16(w)
        out[f"rms_x_f16_{n}"], out[f"rms_w_f16_{n}"] = rh, wh
        out[f"rms_y_f16_{n}"] = ref.rms_norm_row(1, rh, wh, 1e-5)

    # softmax rows
    for n in (1, 7, 8, 9, 257, 4096):
        row = rng.normal(0, 3, n).astype(np.float32)
        out[f"softmax_x_{n}"] = row
        out[f"softmax_y_{n}"] = ref.softmax_f32(row)
    masked = rng.normal(0, 3, 512).astype(np.float32)
    masked[rng.random(512) < 0.5] = -np.inf
    out["softmax_x_masked"] = masked
    out["softmax_y_masked"] = ref.softmax_f32(masked)
    wide = rng.uniform(-120, 40, 300).astype(np.float32)
    out["softmax_x_wide"] = wide
    out["softmax_y_wide_words"] = ref.softmax_f32(wide).view(np.uint32)

    # layer norm rows (drawn last so that every array above keeps its values)
    for n in (1, 7, 127, 128, 129, 257, 2048):
        row = (rng.normal(0.5, 1, n) * rng.uniform(0.1, 10)).astype(np.float32)
        scale = rng.normal(1, 0.1, n).astype(np.float32)
        bias = rng.normal(0, 0.5, n).astype(np.float32)
        out[f"ln_x_f32_{n}"], out[f"ln_s_f32_{n}"], out[f"ln_b_f32_{n}"] = row, scale, bias
        out[f"ln_y_f32_{n}"] = ref.layer_norm_row(0, row, scale, bias, 1e-5)
        out[f"ln_y_f32_plain_{n}"] = ref.layer_norm_row(0, row, None, None, 1e-6)
        for tag, type_id, narrow in (("bf16", 2, ref.f32_to_bf16), ("f16", 1, ref.f32_to_f16)):
            rn, sn, bn = narrow(row), narrow(scale), narrow(bias)
            out[f"ln_x_{tag}_{n}"], out[f"ln_s_{tag}_{n}"], out[f"ln_b_{tag}_{n}"] = rn, sn, bn
            out[f"ln_y_{tag}_{n}"] = ref.layer_norm_row(type_id, rn, sn, bn, 1e-5)

    # the other activations of the floor and the gates built on them (drawn last, see above)
    xa = np.concatenate([SPECIAL_F32, rng.normal(0, 3, 800).astype(np.float32),
                         rng.uniform(-12, 12, 400).astype(np.float32)]).astype(np.float32)
    ua = rng.normal(0, 2, xa.size).astype(np.float32)
    out["more_x_f32_words"], out["more_u_f32_words"] = xa.view(np.uint32), ua.view(np.uint32)
    for name in ("gelu", "gelu_tanh", "sigmoid", "relu"):
        out[f"{name}_f32_words"] = ref.activation(name, 0, xa).view(np.uint32)
    out["geglu_f32_words"] = ref.gated("geglu", 0, xa, ua).view(np.uint32)
    out["geglu_tanh_f32_words"] = ref.gated("geglu_tanh", 0, xa, ua).view(np.uint32)
    for tag, type_id, narrow in (("bf16", 2, ref.f32_to_bf16), ("f16", 1, ref.f32_to_f16)):
        xn, un = narrow(xa), narrow(ua)
        out[f"more_x_{tag}"], out[f"more_u_{tag}"] = xn, un
        out[f"gelu_{tag}"] = ref.activation("gelu", type_id, xn)
        out[f"gelu_tanh_{tag}"] = ref.activation("gelu_tanh", type_id, xn)
    out["geglu_bf16"] = ref.gated("geglu", 2, out["more_x_bf16"], out["more_u_bf16"])
    out["geglu_tanh_bf16"] = ref.gated("geglu_tanh", 2, out["more_x_bf16"], out["more_u_bf16"])

    # log-softmax rows of the floor (drawn last, see above)
    for n in (1, 7, 8, 9, 257, 4096):
        row = rng.normal(0, 3, n).astype(np.float32)
        out[f"log_softmax_x_{n}"] = row
        out[f"log_softmax_y_{n}"] = ref.log_softmax_f32(row)
    masked = rng.normal(0, 3, 512).astype(np.float32)
    masked[rng.random(512) < 0.5] = -np.inf
    out["log_softmax_x_masked"] = masked
    out["log_softmax_y_masked_words"] = ref.log_softmax_f32(masked).view(np.uint32)
    wide = rng.uniform(-120, 40, 300).astype(np.float32)
    out["log_softmax_x_wide"] = wide
    out["log_softmax_y_wide_words"] = ref.log_softmax_f32(wide).view(np.uint32)
    for width in (129, 8193):   # tests/compute_provider_cuda/tensor_test.cc:1168-1199: near-one tails
        tails = np.full((3, width), -20.0, np.float32)
        tails[0, width - 1] = 0
        tails[1, 0] = tails[1, width - 1] = 0
        tails[2, :] = 0
        out[f"log_softmax_y_tails_{width}"] = np.stack([ref.log_softmax_f32(r) for r in tails])

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT}: {os.path.getsize(OUT)} bytes, {len(out)} arrays")


if __name__ == "__main__":
    main()
