// Decoders of GGUF weight blocks, eight neighbouring values at a time, from block bytes in LDS
// (or any byte-addressable memory).  Geometry from the reference
// (src/compute_ops/low_precision.cc:22-29: Q8_0 32 elements in 34 bytes, Q4_K 256 in 144, Q6_K 256
// in 210); the arithmetic is ggml's dequantize_row_q8_0 / _q4_K / _q6_K, restated from the
// published block layouts, checked against the two readings of these formats the reference
// tree holds (third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38;
// tests/compute_models/qwen27_original_nextn_reference.h:74-86,262-287):
//   Q8_0  {f16 d; i8 qs[32]}                              y = d * q           (exact in f32)
//   Q4_K  {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]}    y = (d * sc) * q - (dmin * m)
//   Q6_K  {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d}   y = (d * scale) * (q - 32)
#pragma once

#include "device_common.h"

namespace hyle_hip {
namespace {

constexpr int kSuper = 256;                      // values per super-block

__device__ __forceinline__ float lds_f16(const unsigned char *p) {
  return f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

// Eight values of a Q4_K block starting at position p (a multiple of 8).
__device__ __forceinline__ void decode_q4_k(const unsigned char *blk, uint32_t p, float (&y)[8]) {
  const float d = lds_f16(blk), dmin = lds_f16(blk + 2);
  const unsigned char *scales = blk + 4;
  const uint32_t sub = p / 32, within = p % 32, chunk = sub / 2;
  uint32_t sc, m;
  if (sub < 4) {
    sc = scales[sub] & 63u;
    m = scales[sub + 4] & 63u;
  } else {
    sc = (scales[sub + 4] & 0xFu) | ((uint32_t)(scales[sub - 4] >> 6) << 4);
    m = (uint32_t)(scales[sub + 4] >> 4) | ((uint32_t)(scales[sub] >> 6) << 4);
  }
  const float step = d * (float)sc, offset = dmin * (float)m;
  const unsigned char *q = blk + 16 + 32 * chunk + within;
  const uint32_t shift = (sub & 1u) * 4;
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = step * (float)((q[j] >> shift) & 0xFu) - offset;
}

// Eight values of a Q6_K block starting at position p (a multiple of 8).
__device__ __forceinline__ void decode_q6_k(const unsigned char *blk, uint32_t p, float (&y)[8]) {
  const uint32_t half = p / 128, group = (p % 128) / 32, l = p % 32;
  const unsigned char *ql = blk + 64 * half + l + 32 * (group & 1u);
  const unsigned char *qh = blk + 128 + 32 * half + l;
  const int scale = (int)(int8_t)blk[192 + 8 * half + 2 * group + l / 16];
  const float step = lds_f16(blk + 208) * (float)scale;
  const uint32_t low_shift = (group >> 1) * 4, high_shift = group * 2;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int q = (int)(((ql[j] >> low_shift) & 0xFu) | (((qh[j] >> high_shift) & 3u) << 4)) - 32;
    y[j] = step * (float)q;
  }
}


// Eight values of a Q8_0 block starting at position p (a multiple of 8) of its 32.
__device__ __forceinline__ void decode_q8_0(const unsigned char *blk, uint32_t p, float (&y)[8]) {
  const float d = lds_f16(blk);
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = (float)(int8_t)blk[2 + p + j] * d;
}

// ---------------------------------------------------------------------------------
// The same decoders over 32-bit words, for blocks in LDS.
// ---------------------------------------------------------------------------------

// Eight bytes at a 2-byte aligned LDS address, as three aligned words and two byte-wise funnel
// shifts (an LDS read that is not naturally aligned stalls).
__device__ __forceinline__ void lds_piece(const unsigned char *base, uint32_t offset, uint32_t (&out)[2]) {
  const uint32_t *words = reinterpret_cast<const uint32_t *>(base + (offset & ~3u));
  const uint32_t w0 = words[0], w1 = words[1], w2 = words[2];
  out[0] = __builtin_amdgcn_alignbyte(w1, w0, offset & 3u);
  out[1] = __builtin_amdgcn_alignbyte(w2, w1, offset & 3u);
}

// Q6_K, eight values at position p (a multiple of 8) of the block at slot + block_offset
// (2-byte aligned).  Four q's at a time are put together inside a word as bytes holding
// 4 (q - 32) in two's complement (q < 64: q << 2 stays inside its byte, toggling bit 7 subtracts
// 128), converted with sign extension and multiplied by (d * scale) / 4: the same real product
// as (d * scale) * (q - 32), rounded once.
__device__ __forceinline__ void decode_q6_k_words(const unsigned char *slot, uint32_t block_offset, uint32_t p,
                                                  float (&y)[8]) {
  const uint32_t half = p / 128, group = (p % 128) / 32, l = p % 32;
  uint32_t low[2], top[2];
  lds_piece(slot, block_offset + 64 * half + l + 32 * (group & 1u), low);
  lds_piece(slot, block_offset + 128 + 32 * half + l, top);
  const int scale = (int)(int8_t)slot[block_offset + 192 + 8 * half + 2 * group + l / 16];
  const float d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + block_offset + 208));
  const float step = (d * (float)scale) * 0.25f;
  const uint32_t low_shift = (group >> 1) * 4, high_shift = group * 2;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t nibbles = (low[w] >> low_shift) & 0x0F0F0F0Fu, pairs = (top[w] >> high_shift) & 0x03030303u;
    const uint32_t q = ((nibbles << 2) | (pairs << 6)) ^ 0x80808080u;
#pragma unroll
    for (int t = 0; t < 4; ++t) y[4 * w + t] = step * (float)(int)(signed char)(q >> (8 * t));
  }
}

// Q4_K, eight values at position p (a multiple of 8) of the block at slot + block_offset
// (8-byte aligned: the header is read as four words, the quants as two).
__device__ __forceinline__ void decode_q4_k_words(const unsigned char *slot, uint32_t block_offset, uint32_t p,
                                                  float (&y)[8]) {
  const uint32_t *head = reinterpret_cast<const uint32_t *>(slot + block_offset);
  const uint32_t h0 = head[0], s0 = head[1], s1 = head[2], s2 = head[3];
  const float d = f16_to_f32((uint16_t)h0), dmin = f16_to_f32((uint16_t)(h0 >> 16));
  const uint32_t sub = p / 32, within = p % 32, chunk = sub / 2;
  // scales[i] for i < 4 in s0, 4..7 in s1, 8..11 in s2
  const uint32_t at = 8 * (sub % 4);
  uint32_t sc, m;
  if (sub < 4) {
    sc = (s0 >> at) & 63u;
    m = (s1 >> at) & 63u;
  } else {
    sc = ((s2 >> at) & 0xFu) | (((s0 >> (at + 6)) & 3u) << 4);
    m = ((s2 >> (at + 4)) & 0xFu) | (((s1 >> (at + 6)) & 3u) << 4);
  }
  const float step = d * (float)sc, offset = dmin * (float)m;
  const uint32_t *q = reinterpret_cast<const uint32_t *>(slot + block_offset + 16 + 32 * chunk + within);
  const uint32_t shift = (sub & 1u) * 4;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t nibbles = (q[w] >> shift) & 0x0F0F0F0Fu;
#pragma unroll
    for (int t = 0; t < 4; ++t) y[4 * w + t] = step * (float)((nibbles >> (8 * t)) & 0xFFu) - offset;
  }
}

}  // namespace
}  // namespace hyle_hip
