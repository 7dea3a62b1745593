// How a wave reads rows of 2048 n GGUF values (Q4_K, Q6_K, Q8_0) made of whole 16-byte vectors,
// shared by the matrix-vector kernels of gguf_matvec.hip (exact weights times f32 activations)
// and gguf_matvec_q8.hip (integer dot products with 8-bit activation blocks): which bytes of a
// span of 2048 values a lane decodes (Lines<kind>::lane_of), where those values sit in the row
// of activations (position), the f32 dot product of the first kernel (dot), and the row of
// 16-byte vectors a wave keeps in flight (LinesRow).
#pragma once

#include "device_common.h"
#include "gguf_decode.h"

namespace hyle_hip {
namespace {

constexpr uint32_t kWavesPerBlock = kBlockThreads / kWaveLanes;

template <int kKind> struct Lines;

// sum over the four bytes of word (int8 each) times x[0..3], added to sum
__device__ __forceinline__ float dot_signed_bytes(uint32_t word, const float *x, float sum) {
#pragma unroll
  for (int t = 0; t < 4; ++t) sum = __builtin_fmaf((float)(int)(signed char)(word >> (8 * t)), x[t], sum);
  return sum;
}
// The same for unsigned bytes.  The empty asm keeps the compiler from looking through the word
// to the mask that made it: it would otherwise extract every nibble with a bit-field
// instruction of its own before converting, two instructions per value instead of one.
__device__ __forceinline__ float dot_bytes(uint32_t word, const float *x, float sum) {
  asm("" : "+v"(word));
#pragma unroll
  for (int t = 0; t < 4; ++t) sum = __builtin_fmaf((float)((word >> (8 * t)) & 0xFFu), x[t], sum);
  return sum;
}

// Q6_K.  2048 values are 16 halves of 128, four lanes per half.  Lane (half, j) owns positions
// l = 8 j .. 8 j + 7 of each of the half's four groups (l, l + 32, l + 64, l + 96): 8 bytes of
// ql[64 h + l], 8 of ql[64 h + 32 + l], 8 of qh[32 h + l], the half's eight scales and d.
// Four six-bit quants are put together inside a 32-bit word as bytes holding 4 (q - 32) in
// two's complement (q < 64, so q << 2 stays inside its byte, and bit 7 is the sign once the
// upper bit of the qh field is toggled), which one converting instruction per value
// sign-extends; the factor 1/4 goes into the group's scale.
template <> struct Lines<1> {
  static constexpr int kPassVectors = 105;
  struct Lane {
    uint32_t low, top, scales, d, j;
  };
  static __device__ __forceinline__ Lane lane_of(uint32_t pass, uint32_t lane) {
    const uint32_t half_index = pass * 16 + lane / 4, j = lane % 4;
    const uint32_t block = (half_index / 2) * 210, half = half_index % 2;
    return Lane{block + 64 * half + 8 * j, block + 128 + 32 * half + 8 * j, block + 192 + 8 * half, block + 208, j};
  }
  // where the lane's e-th activation (e = 8 g + t) sits in x
  static __device__ __forceinline__ uint32_t position(uint32_t pass, uint32_t lane, uint32_t e) {
    return pass * 2048 + (lane / 4) * 128 + 32 * (e / 8) + 8 * (lane % 4) + e % 8;
  }
  static __device__ __forceinline__ float dot(const unsigned char *slot, const Lane &at, const float (&x)[32],
                                              const float (&)[4]) {
    uint32_t lows[2], highs[2], tops[2], scales[2];
    lds_piece(slot, at.low, lows);
    lds_piece(slot, at.low + 32, highs);
    lds_piece(slot, at.top, tops);
    lds_piece(slot, at.scales, scales);
    const float d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + at.d)) * 0.25f;
    float group[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      // Toggling the upper bit of every two-bit field of qh subtracts 32 from each q modulo 64;
      // as bit 7 of a byte that holds 4 q it makes the byte 4 (q - 32) as an int8.
      const uint32_t low = lows[w], high = highs[w], top = tops[w] ^ 0xAAAAAAAAu;
      // bytes of 4 q: bits 2..5 from a nibble of ql, bits 6..7 from two bits of qh
      const uint32_t q0 = ((low << 2) & 0x3C3C3C3Cu) | ((top << 6) & 0xC0C0C0C0u);
      const uint32_t q1 = ((high << 2) & 0x3C3C3C3Cu) | ((top << 4) & 0xC0C0C0C0u);
      const uint32_t q2 = ((low >> 2) & 0x3C3C3C3Cu) | ((top << 2) & 0xC0C0C0C0u);
      const uint32_t q3 = ((high >> 2) & 0x3C3C3C3Cu) | (top & 0xC0C0C0C0u);
      group[0] = dot_signed_bytes(q0, &x[4 * w], group[0]);
      group[1] = dot_signed_bytes(q1, &x[8 + 4 * w], group[1]);
      group[2] = dot_signed_bytes(q2, &x[16 + 4 * w], group[2]);
      group[3] = dot_signed_bytes(q3, &x[24 + 4 * w], group[3]);
    }
    // scales[2 g + l / 16] of this half, l / 16 = j / 2
    float total = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t word = scales[g / 2] >> (16 * (g % 2) + 8 * (at.j / 2));
      total = __builtin_fmaf(d * (float)(int)(signed char)word, group[g], total);
    }
    return total;
  }
};

// Q4_K.  2048 values are 8 blocks of four 32-byte chunks; a chunk's low nibbles are sub-block
// 2 c, its high nibbles sub-block 2 c + 1.  A lane takes 8 quant bytes (16 values) of each of
// two blocks: piece i * 64 + lane, i = 0, 1, is block piece / 16, chunk (lane % 16) / 4, bytes
// 8 (lane % 4) .. + 7; every byte is read by one lane, the 16-byte header by the 16 lanes of
// its block.  Blocks are 16-byte aligned in LDS.
template <> struct Lines<0> {
  static constexpr int kPassVectors = 72;
  struct Lane {
    uint32_t header[2], quants[2];
    // the one scale factor this lane works out for the 16 lanes of its block (see dot)
    uint32_t main_shift, main_mask, top_shift, top_mask;
    bool main_in_s2, minimum;
    int source;  // lane of the block's sixteen that holds d * sc of this lane's first sub-block
  };
  static __device__ __forceinline__ Lane lane_of(uint32_t pass, uint32_t lane) {
    Lane at;
    const uint32_t chunk = (lane % 16) / 4;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t block = pass * 8 + (i * 64 + lane) / 16;
      at.header[i] = block * 144;
      at.quants[i] = block * 144 + 16 + 32 * chunk + 8 * (lane % 4);
    }
    // Lane u of a block's sixteen works out d * sc (u < 8) or -dmin * m (u >= 8) of sub-block
    // u % 8.  Sub-blocks 0..3 keep six bits of sc and m in scales[s] and scales[s + 4];
    // sub-blocks 4..7 keep four bits of each in scales[s + 4] and two more in the top of
    // scales[s - 4] and scales[s].  One expression serves all, with the lane's shifts and masks.
    const uint32_t sub = lane % 8;
    at.minimum = (lane % 16) >= 8;
    at.main_in_s2 = sub >= 4;
    at.main_shift = 8 * (sub % 4) + (sub >= 4 && at.minimum ? 4u : 0u);
    at.main_mask = sub < 4 ? 63u : 15u;
    at.top_shift = 8 * (sub % 4) + 6;
    at.top_mask = sub < 4 ? 0u : 3u;
    at.source = (int)((lane & ~15u) + 2 * chunk);
    return at;
  }
  // e = 16 i + 8 high + t
  static __device__ __forceinline__ uint32_t position(uint32_t pass, uint32_t lane, uint32_t e) {
    const uint32_t i = e / 16, high = (e / 8) % 2, t = e % 8;
    const uint32_t block = pass * 8 + (i * 64 + lane) / 16, chunk = (lane % 16) / 4;
    return block * 256 + 64 * chunk + 32 * high + 8 * (lane % 4) + t;
  }
  static __device__ __forceinline__ float dot(const unsigned char *slot, const Lane &at, const float (&x)[32],
                                              const float (&xsum)[4]) {
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const u32x4 head = *reinterpret_cast<const u32x4 *>(slot + at.header[i]);
      const uint32_t s0 = head.y, s1 = head.z, s2 = head.w;  // scales[0..3], [4..7], [8..11]
      const float d = f16_to_f32((uint16_t)head.x), dmin = f16_to_f32((uint16_t)(head.x >> 16));
      // this lane's factor, then the four this lane needs from its neighbours
      const uint32_t own = at.minimum ? s1 : s0;
      const uint32_t bits = (((at.main_in_s2 ? s2 : own) >> at.main_shift) & at.main_mask) |
                            (((own >> at.top_shift) & at.top_mask) << 4);
      const float factor = (at.minimum ? -dmin : d) * (float)bits;
      const float step_low = __shfl(factor, at.source), step_high = __shfl(factor, at.source + 1);
      const float offset_low = __shfl(factor, at.source + 8), offset_high = __shfl(factor, at.source + 9);
      const uint32_t *q = reinterpret_cast<const uint32_t *>(slot + at.quants[i]);
      float low = 0.0f, high = 0.0f;
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const uint32_t word = q[w];
        low = dot_bytes(word & 0x0F0F0F0Fu, &x[16 * i + 4 * w], low);
        high = dot_bytes((word >> 4) & 0x0F0F0F0Fu, &x[16 * i + 8 + 4 * w], high);
      }
      total = __builtin_fmaf(step_low, low, total);
      total = __builtin_fmaf(offset_low, xsum[2 * i], total);
      total = __builtin_fmaf(step_high, high, total);
      total = __builtin_fmaf(offset_high, xsum[2 * i + 1], total);
    }
    return total;
  }
};

// Q8_0.  2048 values are 64 blocks of 34 bytes {f16 d; i8 q[32]}: one block per lane.  Blocks
// are 2-byte aligned, so the 32 quants are taken from nine aligned words with a per-lane funnel
// shift; each byte is already the int8 the converting instruction wants.
template <> struct Lines<2> {
  static constexpr int kPassVectors = 136;
  struct Lane {
    uint32_t block, words, shift;
  };
  static __device__ __forceinline__ Lane lane_of(uint32_t pass, uint32_t lane) {
    const uint32_t block = pass * 2176 + 34 * lane, quants = block + 2;
    return Lane{block, quants & ~3u, quants & 3u};
  }
  static __device__ __forceinline__ uint32_t position(uint32_t pass, uint32_t lane, uint32_t e) {
    return pass * 2048 + 32 * lane + e;
  }
  static __device__ __forceinline__ float dot(const unsigned char *slot, const Lane &at, const float (&x)[32],
                                              const float (&)[4]) {
    const uint32_t *words = reinterpret_cast<const uint32_t *>(slot + at.words);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = words[i];
    const float d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + at.block));
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum = dot_signed_bytes(__builtin_amdgcn_alignbyte(w[i + 1], w[i], at.shift), &x[4 * i], sum);
    return d * sum;
  }
};

constexpr int kLinesDepth = 4;  // rows of a wave whose bytes are in flight

template <int kKind, int kPasses> struct LinesRow {
  static constexpr int kVectors = kPasses * Lines<kKind>::kPassVectors;  // 16-byte vectors in a row
  static constexpr int kLoads = (kVectors + kWaveLanes - 1) / kWaveLanes;
  static constexpr int kSlotBytes = kLoads * kWaveLanes * 16;            // LDS bytes of one wave
  u32x4 v[kLoads];
  // `vectors`: how many of the row's vectors exist (fewer than kVectors for a last, shorter span)
  static __device__ __forceinline__ LinesRow load(const unsigned char *row, uint32_t lane, uint32_t vectors = kVectors) {
    LinesRow r;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t wanted = lane + i * kWaveLanes;  // past the row: its last vector again (parked in LDS, never read)
      r.v[i] = load16_stream(row, wanted < vectors ? wanted : vectors - 1);
    }
    return r;
  }
};

}  // namespace
}  // namespace hyle_hip
