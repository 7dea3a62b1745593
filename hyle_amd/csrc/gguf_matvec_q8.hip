// y[m][n] = MatMul(x, W) for a GGUF weight (Q8_0, Q4_K, Q6_K; logical [K, N]) and a few activation
// rows, computed the way the reference's ggml CPU route computes it: each activation row is first
// quantised to 8-bit blocks (Q8_0 blocks of 32 for a Q8_0 weight, Q8_K blocks of 256 for Q4_K and
// Q6_K), block dot products are integers, and the scales are applied in f32.
//
// ggml's source is not in the reference tree.  The arithmetic follows the restatement the
// reference's own tests hold of it:
//   Q8_0 activation block   scale = f16(RN(max / 127)), code = RNE(RN(x * RN(127 / max)))
//       (tests/compute_models/dspark_original_shared_reference.h:147-185, the AVX form)
//   Q8_K activation block   the first element of largest magnitude, sign kept, gives
//       inverse = RN(-127 / max); code = min(127, RNE(RN(x * inverse))); scale = RN(1 / inverse)
//       (tests/compute_models/qwen27_original_nextn_reference.h:144-167)
//   product                 sum over 32-wide groups of w.scale * a.scale * (w.codes . a.codes)
//       [+ w.minimum * a.scale * (w.offsets . a.codes) for Q4_K], integer dots
//       (tests/compute_models/qwen27_original_nextn_reference.h:94-130, 216-244)
// The integer parts are exact here; the f32 products and sums differ from ggml's only in their
// order, which the reference's tests allow for with gamma(K / 4 + 65, 2^-24) * sum |terms|.
//
// Q6_K and Q8_0 rows are read exactly as in gguf_matvec.hip (whole 16-byte vectors through
// wave-private LDS, four spans of 2048 values in flight per wave, gguf_lines.h).  The activation
// codes of a lane's 32 positions are eight 32-bit words per activation row, so a weight word of four
// quants meets them in one v_dot4c_i32_i8, and decoding a span once serves every activation row:
//   Q6_K  four quants are assembled per word as int8 bytes 4 (q - 32); a 16-value group's dot is
//         multiplied by its int8 scale as an integer; one conversion and (d / 4) * a.scale close
//         the half block
//   Q8_0  the bytes are the int8 quants; d * a.scale closes the block
// Q4_K blocks are whole 16-byte vectors, so its rows go from global memory straight into the
// operands of 16 x 16 x 64 int8 matrix instructions, sixteen weight rows per wave
// (gguf_matvec_q8_tiles): nibbles are already bytes 0..15; sc * dot and m * (sum of activation
// codes) stay integers; d * a.scale and dmin * a.scale close the block.
#include <type_traits>

#include "device_common.h"
#include "gguf_decode.h"
#include "gguf_lines.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

// a * b + c for factors that fit 24 signed bits (v_mad_i32_i24; a full 32-bit multiply is four
// times slower)
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }

__device__ __forceinline__ int dot4(uint32_t weights, uint32_t codes, int sum) {
  return __builtin_amdgcn_sdot4((int)weights, (int)codes, sum, false);
}

// The element of largest magnitude of a block spread over kLanes adjacent lanes; among equal
// magnitudes the one at the lowest position of the row wins (ggml walks the block in order and
// replaces its candidate only on a strictly larger magnitude).
struct LaneMax {
  float magnitude, value;
  uint32_t position;
  template <int kCtrl> __device__ __forceinline__ LaneMax moved() const {
    return {dpp_move<kCtrl>(magnitude), dpp_move<kCtrl>(value), (uint32_t)dpp_move<kCtrl>((int)position)};
  }
  __device__ __forceinline__ LaneMax shuffled_xor(int mask) const {
    return {__shfl_xor(magnitude, mask, kWaveLanes), __shfl_xor(value, mask, kWaveLanes),
            (uint32_t)__shfl_xor((int)position, mask, kWaveLanes)};
  }
};
__device__ __forceinline__ LaneMax first_largest(LaneMax a, LaneMax b) {
  if (a.magnitude != b.magnitude) return a.magnitude > b.magnitude ? a : b;
  return a.position <= b.position ? a : b;
}
template <int kLanes> __device__ __forceinline__ LaneMax block_largest(LaneMax mine) {
  if constexpr (kLanes == 1) return mine;
  else return group_reduce<kLanes>(mine, [](LaneMax a, LaneMax b) { return first_largest(a, b); });
}

__device__ __forceinline__ uint32_t code_of(float scaled) {
  int code = (int)__builtin_rintf(scaled);  // nearest, ties to even
  code = code > 127 ? 127 : code;
  return (uint32_t)code & 0xFFu;
}

// What a lane holds of one activation row for one span of 2048 values: the codes of its 32
// positions (word e / 4, byte e % 4) and the scale of the activation block they belong to.
struct LaneCodes {
  uint32_t codes[8];
  float scale;
};

// Quantises the lane's share of span `span` of the activation row at `x` (k values of type TX).
// Every lane of a wave calls it; lanes that share an activation block agree on its scale through
// a cross-lane maximum.
// `live`: the lane's positions exist (a Q8_0 row's last span may be short: lanes past it read the
// row's first values and come back with zero codes and a zero scale).
template <int kKind, class TX>
__device__ __forceinline__ LaneCodes quantise_span(const void *x, size_t row_offset, uint32_t span, uint32_t lane, bool live = true) {
  using Kind = Lines<kKind>;
  // the lane's positions come in runs of eight neighbours (Lines<kind>::position), each a whole
  // 16-byte vector of a narrow type or two of f32: x starts on a 16-byte boundary (run_m)
  float values[32];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const size_t at = row_offset + (live ? Kind::position(span, lane, 8 * g) : (uint32_t)(8 * g));
    if constexpr (Traits<TX>::kVec == 8) {
      float piece[8];
      Traits<TX>::unpack(load16(x, at / 8), piece);
#pragma unroll
      for (int t = 0; t < 8; ++t) values[8 * g + t] = piece[t];
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float piece[4];
        Traits<TX>::unpack(load16(x, at / 4 + h), piece);
#pragma unroll
        for (int t = 0; t < 4; ++t) values[8 * g + 4 * h + t] = piece[t];
      }
    }
  }
  LaneCodes out;
  // Q8_0: the lane's 32 values are one block.  Q6_K: eight lanes share a block of 256.
  constexpr int kLanesPerBlock = kKind == 1 ? 8 : 1;
  LaneMax mine{0.0f, 0.0f, 0u};
#pragma unroll
  for (int e = 0; e < 32; ++e) {  // positions rise with e, so ">" keeps the first
    const float magnitude = __builtin_fabsf(values[e]);
    if (magnitude > mine.magnitude) mine = LaneMax{magnitude, values[e], Kind::position(span, lane, e)};
  }
  if (mine.magnitude == 0.0f) mine.position = 0xFFFFFFFFu;  // no candidate: any lane with one goes first
  LaneMax top = block_largest<kLanesPerBlock>(mine);
  if (!live) top.magnitude = 0.0f;
  float factor = 0.0f, stored = 0.0f;
  if (top.magnitude != 0.0f) {
    if constexpr (kKind == 2) {
      stored = f16_to_f32(f32_to_f16(top.magnitude / 127.0f));
      factor = 127.0f / top.magnitude;
    } else {
      factor = -127.0f / top.value;
      stored = 1.0f / factor;
    }
  }
  out.scale = stored;
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    uint32_t word = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) word |= code_of(values[4 * w + t] * factor) << (8 * t);
    out.codes[w] = top.magnitude != 0.0f ? word : 0u;
  }
  return out;
}

// The span's bytes decoded once into words of four int8 quants, then met with each activation row.
template <int kKind> struct SpanDot;

template <> struct SpanDot<1> {  // Q6_K
  uint32_t q[4][2];
  int scale[4];
  float step;  // d / 4
  __device__ __forceinline__ void decode(const unsigned char *slot, const Lines<1>::Lane &at) {
    uint32_t lows[2], highs[2], tops[2], scales[2];
    lds_piece(slot, at.low, lows);
    lds_piece(slot, at.low + 32, highs);
    lds_piece(slot, at.top, tops);
    lds_piece(slot, at.scales, scales);
    step = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + at.d)) * 0.25f;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const uint32_t low = lows[w], high = highs[w], top = tops[w] ^ 0xAAAAAAAAu;
      q[0][w] = ((low << 2) & 0x3C3C3C3Cu) | ((top << 6) & 0xC0C0C0C0u);
      q[1][w] = ((high << 2) & 0x3C3C3C3Cu) | ((top << 4) & 0xC0C0C0C0u);
      q[2][w] = ((low >> 2) & 0x3C3C3C3Cu) | ((top << 2) & 0xC0C0C0C0u);
      q[3][w] = ((high >> 2) & 0x3C3C3C3Cu) | (top & 0xC0C0C0C0u);
    }
#pragma unroll
    for (int g = 0; g < 4; ++g)
      scale[g] = (int)(signed char)(scales[g / 2] >> (16 * (g % 2) + 8 * (at.j / 2)));
  }
  __device__ __forceinline__ float against(const LaneCodes &a) const {
    int total = 0;
#pragma unroll
    for (int g = 0; g < 4; ++g) total = mad24(scale[g], dot4(q[g][0], a.codes[2 * g], dot4(q[g][1], a.codes[2 * g + 1], 0)), total);
    return (step * a.scale) * (float)total;
  }
};

// Sums of kCount values over the wave, jointly: log2(kCount) exchange steps halve the values a
// lane carries (lane l ends with value l % kCount summed over its group of kCount lanes), the
// remaining steps add the groups.  Every lane with l % kCount == i returns the total of v[i].
template <int kCount> __device__ __forceinline__ float joint_sum(float (&v)[kCount], uint32_t lane) {
  static_assert(kCount == 1 || kCount == 2 || kCount == 4 || kCount == 8, "joint sums of 1, 2, 4 or 8 values");
  int live = kCount;
#pragma unroll
  for (int step = 1; step < kCount; step *= 2) {
    const bool upper = (lane & (uint32_t)step) != 0;
    live /= 2;
#pragma unroll
    for (int i = 0; i < live; ++i) {
      const float keep = upper ? v[2 * i + 1] : v[2 * i], give = upper ? v[2 * i] : v[2 * i + 1];
      v[i] = keep + __shfl_xor(give, step, kWaveLanes);
    }
  }
  float mine = v[0];
#pragma unroll
  for (int step = kCount; step < kWaveLanes; step *= 2) mine += __shfl_xor(mine, step, kWaveLanes);
  return mine;
}

// Six-bit sc (or m) of sub-block j from the twelve scale bytes of a Q4_K block, s0 = bytes 0..3,
// s1 = 4..7, s2 = 8..11: sub-blocks 0..3 keep them whole in bytes j and j + 4, sub-blocks 4..7 keep
// four bits in a nibble of byte j + 4 and two more in the top of byte j - 4 (sc) or j (m).
__device__ __forceinline__ int q4k_six_bits(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t j, bool minimum) {
  const uint32_t shift = 8 * (j % 4), own = minimum ? s1 : s0;
  if (j < 4) return (int)((own >> shift) & 63u);
  return (int)(((s2 >> (shift + (minimum ? 4u : 0u))) & 15u) | (((own >> (shift + 6)) & 3u) << 4));
}

template <> struct SpanDot<2> {  // Q8_0
  uint32_t q[8];
  float d;
  __device__ __forceinline__ void decode(const unsigned char *slot, const Lines<2>::Lane &at) {
    const uint32_t *words = reinterpret_cast<const uint32_t *>(slot + at.words);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = words[i];
    d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + at.block));
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = __builtin_amdgcn_alignbyte(w[i + 1], w[i], at.shift);
  }
  __device__ __forceinline__ float against(const LaneCodes &a) const {
    int total = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) total = dot4(q[i], a.codes[i], total);
    return (d * a.scale) * (float)total;
  }
};

// LDS of a block: for every (activation row, span) the 64 lanes' LaneCodes, stored as
// [word][lane] so that a wave reads each word of its lanes from consecutive banks.
constexpr uint32_t kCodeWords = 8 + 1;  // codes, scale
__device__ __forceinline__ void park(uint32_t *staged, uint32_t pair, uint32_t lane, const LaneCodes &c) {
  uint32_t *at = staged + (size_t)pair * kCodeWords * kWaveLanes + lane;
#pragma unroll
  for (int w = 0; w < 8; ++w) at[w * kWaveLanes] = c.codes[w];
  at[8 * kWaveLanes] = f32_bits(c.scale);
}
__device__ __forceinline__ LaneCodes fetch(const uint32_t *staged, uint32_t pair, uint32_t lane) {
  const uint32_t *at = staged + (size_t)pair * kCodeWords * kWaveLanes + lane;
  LaneCodes c;
#pragma unroll
  for (int w = 0; w < 8; ++w) c.codes[w] = at[w * kWaveLanes];
  c.scale = bits_f32(at[8 * kWaveLanes]);
  return c;
}

// kM activation rows (rows past m repeat the last one and are not stored); kRegisters: one span
// per row (K = 2048), the lane's codes live in registers for the whole kernel.
template <int kKind, class TX, int kM, bool kRegisters>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_q8_lines(const unsigned char *weights, const void *x,
                                                                      void *y, uint32_t rows, uint64_t row_stride,
                                                                      uint32_t spans, uint32_t m) {
  using Row = LinesRow<kKind, 1>;
  using Kind = Lines<kKind>;
  constexpr uint32_t kSpanBytes = Kind::kPassVectors * 16;
  __shared__ __align__(16) unsigned char slots[kWavesPerBlock][Row::kSlotBytes];
  extern __shared__ __align__(16) uint32_t staged[];  // [m * spans][kCodeWords][64]
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  const uint32_t k = spans * 2048;
  // every wave quantises its share of the (activation row, span) pairs; the block then shares them
  for (uint32_t pair = wave; pair < m * spans; pair += kWavesPerBlock)
    park(staged, pair, lane, quantise_span<kKind, TX>(x, (size_t)(pair / spans) * k, pair % spans, lane));
  __syncthreads();
  LaneCodes held[kRegisters ? kM : 1];
  if constexpr (kRegisters) {
#pragma unroll
    for (int r = 0; r < kM; ++r) held[r] = fetch(staged, (uint32_t)r < m ? (uint32_t)r : m - 1, lane);
  }
  unsigned char *slot = slots[wave];
  const typename Kind::Lane at = Kind::lane_of(0, lane);
  const uint32_t stride = gridDim.x * kWavesPerBlock;
  const uint32_t first = blockIdx.x * kWavesPerBlock + wave;
  if (first >= rows) return;  // no barrier follows
  const uint32_t own_rows = (rows - first + stride - 1) / stride;
  const uint64_t segments = (uint64_t)own_rows * spans;
  // the stream of loads runs kLinesDepth segments ahead of the stream of decodes
  uint32_t load_row = first, load_span = 0;
  uint64_t loaded = 0;
  auto next_load = [&]() {
    // past the wave's last segment: its first row again, a valid address whose bytes go unused
    const bool live = loaded < segments;
    const unsigned char *source = weights + (size_t)(live ? load_row : first) * row_stride +
                                  (size_t)(live ? load_span : 0u) * kSpanBytes;
    ++loaded;
    if (++load_span == spans) {
      load_span = 0;
      load_row += stride;
    }
    return Row::load(source, lane);
  };
  Row ring[kLinesDepth];
#pragma unroll
  for (int d = 0; d < kLinesDepth; ++d) ring[d] = next_load();
  uint32_t row = first, span = 0;
  float totals[kM] = {};
  // value b * kM + r of a batch is activation row r against the batch's b-th weight row
  constexpr int kBatch = kM >= 4 ? 1 : 4 / kM;
  float pending[kBatch * kM] = {};
  int filled = 0;
  auto flush = [&](uint32_t first_row, int count) {
    const float mine = joint_sum<kBatch * kM>(pending, lane);
    const uint32_t b = (lane % (uint32_t)(kBatch * kM)) / (uint32_t)kM, r = lane % (uint32_t)kM;
    if (lane < (uint32_t)(kBatch * kM) && (int)b < count && r < m)
      Traits<TX>::store(y, (size_t)r * rows + first_row + b * stride, mine);
#pragma unroll
    for (int i = 0; i < kBatch * kM; ++i) pending[i] = 0.0f;
  };
  for (uint64_t done = 0; done < segments; done += kLinesDepth) {
#pragma unroll
    for (int d = 0; d < kLinesDepth; ++d) {
      if (done + d >= segments) break;
#pragma unroll
      for (int i = 0; i < Row::kLoads; ++i)
        *reinterpret_cast<u32x4 *>(slot + (size_t)(lane + i * kWaveLanes) * 16) = ring[d].v[i];
      ring[d] = next_load();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      SpanDot<kKind> decoded;
      decoded.decode(slot, at);
#pragma unroll
      for (int r = 0; r < kM; ++r) {
        if constexpr (kRegisters) {
          totals[r] += decoded.against(held[r]);
        } else {
          const uint32_t pair = ((uint32_t)r < m ? (uint32_t)r : m - 1) * spans + span;
          totals[r] += decoded.against(fetch(staged, pair, lane));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (++span == spans) {
        // the row is complete: park its kM totals; kBatch rows are summed over the wave together
#pragma unroll
        for (int r = 0; r < kM; ++r) {
          pending[filled * kM + r] = totals[r];
          totals[r] = 0.0f;
        }
        span = 0;
        row += stride;
        if (++filled == kBatch) {
          flush(row - (uint32_t)kBatch * stride, filled);
          filled = 0;
        }
      }
    }
  }
  if (filled != 0) flush(row - (uint32_t)filled * stride, filled);
}

// One activation row, one to six spans: a wave of the block per span.  The wave quantises its own
// span of x straight into registers (nothing is parked in LDS and no barrier precedes the first
// row), walks the block's rows at its span and leaves its share of each row in LDS, where the
// first wave adds the spans' shares in span order.
//
// tail_lanes: how many lanes of the last span's wave have a block of the row (64 unless the row is
// a Q8_0 row whose width is a multiple of 256 but not of 2048: a lane is a block of 32 values
// there, and the last span then holds 8, 16, ... 56 blocks in 17, 34, ... 119 whole vectors).
template <int kKind, class TX, int kSpans, bool kShort>
__global__ __launch_bounds__(kSpans * kWaveLanes) void gguf_matvec_q8_spans(const unsigned char *weights, const void *x, void *y,
                                                                          uint32_t rows, uint64_t row_stride, uint32_t tail_lanes) {
  static_assert(!kShort || kKind == 2, "only Q8_0 rows have short last spans");
  using Row = LinesRow<kKind, 1>;
  using Kind = Lines<kKind>;
  constexpr uint32_t kSpanBytes = Kind::kPassVectors * 16;
  __shared__ __align__(16) unsigned char slots[kSpans][Row::kSlotBytes];
  __shared__ float shares[kSpans][kLinesDepth];
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t span = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  unsigned char *slot = slots[span];
  const typename Kind::Lane at = Kind::lane_of(0, lane);
  const uint32_t stride = gridDim.x, first = blockIdx.x;  // first < rows: the grid has at most `rows` blocks
  const unsigned char *mine = weights + (size_t)span * kSpanBytes;
  // (whole spans: constants, and the compiler drops what depends on them)
  const uint32_t live_lanes = kShort && span == (uint32_t)kSpans - 1 ? tail_lanes : (uint32_t)kWaveLanes;
  const bool live = !kShort || lane < live_lanes;
  const uint32_t vectors = kShort ? (live_lanes * 34u + 15u) / 16u : (uint32_t)Kind::kPassVectors;
  Row ring[kLinesDepth];
#pragma unroll
  for (int d = 0; d < kLinesDepth; ++d) {
    const uint64_t wanted = (uint64_t)first + (uint64_t)d * stride;
    ring[d] = Row::load(mine + (size_t)(wanted < rows ? (uint32_t)wanted : first) * row_stride, lane, vectors);
  }
  const LaneCodes held = quantise_span<kKind, TX>(x, 0, span, lane, live);  // while the first rows are on their way
  for (uint64_t base = first; base < rows; base += (uint64_t)kLinesDepth * stride) {
    float totals[kLinesDepth] = {};
#pragma unroll
    for (int d = 0; d < kLinesDepth; ++d) {
      const uint64_t row = base + (uint64_t)d * stride;
      if (row >= rows) break;
#pragma unroll
      for (int i = 0; i < Row::kLoads; ++i)
        *reinterpret_cast<u32x4 *>(slot + (size_t)(lane + i * kWaveLanes) * 16) = ring[d].v[i];
      const uint64_t wanted = row + (uint64_t)kLinesDepth * stride;
      ring[d] = Row::load(mine + (size_t)(wanted < rows ? (uint32_t)wanted : first) * row_stride, lane, vectors);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      SpanDot<kKind> decoded;
      decoded.decode(slot, at);
      const float mine_of_row = decoded.against(held);
      totals[d] = live ? mine_of_row : 0.0f;  // a lane past a short last span decoded bytes that are not the row's
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    static_assert(kLinesDepth == 4, "the joint sum is taken over four rows");
    const float share = joint_sum<kLinesDepth>(totals, lane);  // lane l < 4: row l over the wave
    if constexpr (kSpans == 1) {
      const uint64_t row = base + (uint64_t)lane * stride;
      if (lane < (uint32_t)kLinesDepth && row < rows) Traits<TX>::store(y, (size_t)row, share);
    } else {
      if (lane < (uint32_t)kLinesDepth) shares[span][lane] = share;
      __syncthreads();
      const uint64_t row = base + (uint64_t)lane * stride;
      if (span == 0 && lane < (uint32_t)kLinesDepth && row < rows) {
        float whole = shares[0][lane];
#pragma unroll
        for (int other = 1; other < kSpans; ++other) whole += shares[other][lane];
        Traits<TX>::store(y, (size_t)row, whole);
      }
      __syncthreads();
    }
  }
}

// ---- several activation rows: the integer dots on the matrix unit ------------------------------
// v_mfma_i32_4x4x4i8 is sixteen independent 4 x 4 x 4 products, one per quad of lanes: lane q of a
// quad gives row q of A (four int8 along k) and column q of B, and gets column q of D back, one
// register per row.  With A = four weight rows at the same four positions and B = four activation
// rows' codes at those positions, one instruction is the sixteen four-value dots that the vector
// unit would take with sixteen v_dot4c.  So the four lanes of a quad decode four *different*
// weight rows (the four a wave keeps in flight) at the *same* positions, each for one activation
// row: lane (c, q) walks the 32-value shares of lanes 4 c .. 4 c + 3 of the one-row-per-wave
// layout, on weight row q, against the codes of activation row q.  The decode of a weight row is
// done once whatever the number of activation rows; what a group of 16 costs per lane beyond it is
// two matrix instructions and four scale multiplies, for four rows by four activation rows.
typedef int i32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ i32x4 quad_dots(uint32_t weights, uint32_t codes, i32x4 sum) {
  return __builtin_amdgcn_mfma_i32_4x4x4i8((int)weights, (int)codes, sum, 0, 0, 0);
}
// lane i of the caller's quad
template <int kLane> __device__ __forceinline__ int quad_lane(int v) { return dpp_move<kLane * 0x55>(v); }
template <int kLane> __device__ __forceinline__ float quad_lane(float v) { return dpp_move<kLane * 0x55>(v); }
// sum over the sixteen quads of the wave, lane q of each: every lane ends with its column's total
__device__ __forceinline__ float quads_sum(float v) {
  v += dpp_move<0x1B>(dpp_move<kDppHalfMirror>(v));  // lane ^ 4: half-row mirror, then quad reversal
  v += dpp_move<0x128>(v);                           // lane ^ 8: row_ror 8
  v += __shfl_xor(v, 16, kWaveLanes);
  v += __shfl_xor(v, 32, kWaveLanes);
  return v;
}

// One decoded 32-value share of this lane's weight row against the codes `a` of the same
// positions of this lane's activation row.  The codes go in as A and the weights as B, so the
// lane gets its own weight row back against the quad's four activation rows: sums[i] gains
// activation row i's part, and the weight row's scales are the lane's own.
template <int kKind> struct QuadDot;
template <> struct QuadDot<1> {  // Q6_K
  static __device__ __forceinline__ void add(const SpanDot<1> &w, const LaneCodes &a, float (&sums)[4]) {
    int total[4] = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const i32x4 zero = {0, 0, 0, 0};
      const i32x4 dots = quad_dots(a.codes[2 * g + 1], w.q[g][1], quad_dots(a.codes[2 * g], w.q[g][0], zero));
#pragma unroll
      for (int i = 0; i < 4; ++i) total[i] = mad24(w.scale[g], dots[i], total[i]);
    }
    sums[0] += (w.step * quad_lane<0>(a.scale)) * (float)total[0];
    sums[1] += (w.step * quad_lane<1>(a.scale)) * (float)total[1];
    sums[2] += (w.step * quad_lane<2>(a.scale)) * (float)total[2];
    sums[3] += (w.step * quad_lane<3>(a.scale)) * (float)total[3];
  }
};
template <> struct QuadDot<2> {  // Q8_0
  static __device__ __forceinline__ void add(const SpanDot<2> &w, const LaneCodes &a, float (&sums)[4]) {
    i32x4 dots = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i) dots = quad_dots(a.codes[i], w.q[i], dots);
    sums[0] += (w.d * quad_lane<0>(a.scale)) * (float)dots[0];
    sums[1] += (w.d * quad_lane<1>(a.scale)) * (float)dots[1];
    sums[2] += (w.d * quad_lane<2>(a.scale)) * (float)dots[2];
    sums[3] += (w.d * quad_lane<3>(a.scale)) * (float)dots[3];
  }
};

// kSets sets of four activation rows (rows past m repeat the last one and are not stored);
// kRegisters: one span per row (K = 2048), the lane's codes live in registers for the whole kernel.
// A wave takes weight rows first + n * stride four at a time, span by span.
template <int kKind, class TX, int kSets, bool kRegisters>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_q8_quads(const unsigned char *weights, const void *x,
                                                                      void *y, uint32_t rows, uint64_t row_stride,
                                                                      uint32_t spans, uint32_t m) {
  using Row = LinesRow<kKind, 1>;
  using Kind = Lines<kKind>;
  constexpr uint32_t kSpanBytes = Kind::kPassVectors * 16;
  // the four lanes of a quad read the same offsets of four slots at once: 32 bytes between the
  // slots' starts (mod 128) put them on different LDS banks
  constexpr int kSlotStride = Row::kSlotBytes + 32;
  __shared__ __align__(16) unsigned char slots[kWavesPerBlock][4][kSlotStride];
  extern __shared__ __align__(16) uint32_t staged[];  // [m * spans][kCodeWords][64]
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  const uint32_t quad = lane / 4, own = lane % 4;  // positions of lanes 4 quad .. + 3; weight row and activation row `own`
  const uint32_t k = spans * 2048;
  for (uint32_t pair = wave; pair < m * spans; pair += kWavesPerBlock)
    park(staged, pair, lane, quantise_span<kKind, TX>(x, (size_t)(pair / spans) * k, pair % spans, lane));
  __syncthreads();
  uint32_t token[kSets];
#pragma unroll
  for (int set = 0; set < kSets; ++set) token[set] = min(own + 4u * set, m - 1);
  LaneCodes held[kRegisters ? kSets * 4 : 1];
  if constexpr (kRegisters) {
#pragma unroll
    for (int set = 0; set < kSets; ++set)
#pragma unroll
      for (int t = 0; t < 4; ++t) held[set * 4 + t] = fetch(staged, token[set], 4 * quad + t);
  }
  typename Kind::Lane at[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) at[t] = Kind::lane_of(0, 4 * quad + t);
  const unsigned char *own_slot = slots[wave][own];
  const uint32_t stride = gridDim.x * kWavesPerBlock;
  const uint32_t first = blockIdx.x * kWavesPerBlock + wave;
  if (first >= rows) return;  // no barrier follows
  const uint32_t own_rows = (rows - first + stride - 1) / stride;
  const uint32_t batches = (own_rows + 3) / 4;
  // the loads of the next (batch, span) are in flight while this one is decoded
  auto load_batch = [&](uint32_t batch, uint32_t span, Row (&into)[4]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t n = 4 * batch + d;
      // past the wave's last row: its first row again, a valid address whose bytes go unused
      const unsigned char *source = weights + (size_t)(n < own_rows ? first + n * stride : first) * row_stride +
                                    (size_t)(n < own_rows ? span : 0u) * kSpanBytes;
      into[d] = Row::load(source, lane);
    }
  };
  Row ring[4];
  load_batch(0, 0, ring);
  float sums[kSets][4] = {};
  for (uint32_t batch = 0; batch < batches; ++batch) {
    for (uint32_t span = 0; span < spans; ++span) {
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int i = 0; i < Row::kLoads; ++i)
          *reinterpret_cast<u32x4 *>(slots[wave][d] + (size_t)(lane + i * kWaveLanes) * 16) = ring[d].v[i];
      {
        const bool last_span = span + 1 == spans;
        const uint32_t next_batch = last_span ? batch + 1 : batch;
        load_batch(next_batch < batches ? next_batch : 0u, last_span ? 0u : span + 1, ring);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        SpanDot<kKind> decoded;
        decoded.decode(own_slot, at[t]);
#pragma unroll
        for (int set = 0; set < kSets; ++set) {
          if constexpr (kRegisters) QuadDot<kKind>::add(decoded, held[set * 4 + t], sums[set]);
          else QuadDot<kKind>::add(decoded, fetch(staged, token[set] * spans + span, 4 * quad + t), sums[set]);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    // the four rows are complete: lane (0, q) stores its weight row against every activation row
#pragma unroll
    for (int set = 0; set < kSets; ++set)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float total = quads_sum(sums[set][i]);
        sums[set][i] = 0.0f;
        const uint32_t n = 4 * batch + own, r = (uint32_t)i + 4u * set;
        if (quad == 0 && n < own_rows && r < m) Traits<TX>::store(y, (size_t)r * rows + first + n * stride, total);
      }
  }
}

// ---- Q4_K: the sub-block dots on the matrix unit --------------------------------------------------
// v_mfma_i32_16x16x64_i8: lane (c, p) = c + 16 p gives sixteen int8 of row c of A and of column c of
// B at k-slots 16 p .. 16 p + 15, and gets D[4 p .. 4 p + 3][c] back.  Here a column is a weight row
// (sixteen per wave) and B is its nibbles: a lane loads its operands straight from global memory,
// 16 quant bytes at a time (a Q4_K block is nine 16-byte vectors: the header, then eight chunks).
// In a group of four blocks lane (c, p) takes chunk 4 i + p of block b of row c, whose low nibbles
// are sixteen values of sub-block 4 i + 2 (p / 2) and whose high nibbles are sixteen of the next
// one.  What the vector unit does per 32 weights is three instructions of nibble masking.
//
// The rows of A keep the 32-value sub-blocks apart: a row carries activation codes at the k-slots
// whose weights belong to its sub-block and zeros elsewhere, so that D[row][c] is one integer
// sub-block dot of weight row c.
//   One activation row: the sixteen rows are four sub-blocks of each of the group's four blocks;
//   instruction (b, i, nibble) feeds rows 4 b + 2 (p / 2) + nibble of the accumulator of half i, and
//   after the four blocks lane (c, p) holds the eight sub-block dots of block p of its row.
//   Four activation rows (eight: two sets): the sixteen rows are four sub-blocks of four activation
//   rows; instruction (i, nibble) of a block feeds rows 4 t + 2 (p / 2) + nibble, and after the
//   block lane (c, p) holds its eight sub-block dots against activation row p.
// Either way one lane per (weight row, block, activation row) extracts the block's six-bit factors,
// multiplies them in as integers and closes the block in f32.
//
// A lane's share of an A operand is nonzero for one instruction in eight (in two): its sixteen
// codes sit in LDS in their natural order behind a row of zeros, and the lane reads every operand
// at "its base for this instruction + what the instruction adds for all lanes", where the base is
// its codes' for the instruction that wants them and the row of zeros' for the others.  The block
// quantises the activation rows once while its first weight bytes are on their way.
constexpr uint32_t kTileRows = 16;  // weight rows of a wave

struct TileGroup {  // what a lane holds of four blocks of its weight row
  u32x4 head;          // of block `part` of the group
  u32x4 quants[4][2];  // chunk 4 i + part of block b
};

// Shared memory of a block: zeros [K] | codes [tokens][K] | sums [tokens][blocks][8] | scales [tokens][blocks] |
// shares [waves][64][tokens / 4 or 1]
__host__ __device__ inline size_t tile_shared_bytes(uint32_t tokens, uint32_t blocks) {
  return (size_t)(1 + tokens) * blocks * 256 + (size_t)tokens * blocks * (32 + 4) +
         (size_t)kWavesPerBlock * kWaveLanes * (tokens >= 4 ? tokens / 4 : 1) * 4;
}

// Block barrier that orders LDS accesses only: the weight loads issued before it stay in flight.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Half a wave quantises an activation block of 256 values (Q8_K), eight values per lane.
struct TileValues {
  u32x4 raw[2];
};
template <class TX> __device__ __forceinline__ TileValues tile_fetch(const void *x, size_t first, uint32_t u) {
  TileValues out;
  if constexpr (Traits<TX>::kVec == 8) {
    out.raw[0] = load16(x, first / 8 + u);
    out.raw[1] = out.raw[0];
  } else {
    out.raw[0] = load16(x, first / 4 + 2 * (size_t)u);
    out.raw[1] = load16(x, first / 4 + 2 * (size_t)u + 1);
  }
  return out;
}
template <class TX>
__device__ __forceinline__ void tile_quantise(const TileValues &fetched, uint32_t u, unsigned char *codes, int *sums,
                                              float *scale) {
  float values[8];
  if constexpr (Traits<TX>::kVec == 8) {
    Traits<TX>::unpack(fetched.raw[0], values);
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float piece[4];
      Traits<TX>::unpack(fetched.raw[h], piece);
#pragma unroll
      for (int e = 0; e < 4; ++e) values[4 * h + e] = piece[e];
    }
  }
  LaneMax mine{0.0f, 0.0f, 0u};
#pragma unroll
  for (int e = 0; e < 8; ++e) {  // positions rise with e, so ">" keeps the first
    const float magnitude = __builtin_fabsf(values[e]);
    if (magnitude > mine.magnitude) mine = LaneMax{magnitude, values[e], 8 * u + (uint32_t)e};
  }
  if (mine.magnitude == 0.0f) mine.position = 0xFFFFFFFFu;
  const LaneMax top = block_largest<32>(mine);
  float factor = 0.0f, stored = 0.0f;
  if (top.magnitude != 0.0f) {
    factor = -127.0f / top.value;
    stored = 1.0f / factor;
  }
  uint32_t words[2];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) word |= code_of(values[4 * w + e] * factor) << (8 * e);
    words[w] = top.magnitude != 0.0f ? word : 0u;
  }
  int sum = dot4(0x01010101u, words[0], dot4(0x01010101u, words[1], 0));
  sum += dpp_move<kDppSwap1>(sum);
  sum += dpp_move<kDppSwap2>(sum);  // the four lanes of a 32-value sub-block
  uint32_t *at = reinterpret_cast<uint32_t *>(codes) + 2 * u;
  at[0] = words[0];
  at[1] = words[1];
  if (u % 4 == 0) sums[u / 4] = sum;
  if (u == 0) *scale = stored;
}

// The sixteen six-bit factors of a block: sc[s] and mn[s] of sub-block s.
struct TileFactors {
  int sc[8], mn[8];
  float d, dmin;
  __device__ __forceinline__ explicit TileFactors(const u32x4 &h) {
#pragma unroll
    for (uint32_t s = 0; s < 8; ++s) {
      sc[s] = q4k_six_bits(h.y, h.z, h.w, s, false);
      mn[s] = q4k_six_bits(h.y, h.z, h.w, s, true);
    }
    d = f16_to_f32((uint16_t)h.x);
    dmin = f16_to_f32((uint16_t)(h.x >> 16));
  }
  // dots[i][r]: sub-block 4 i + r against the activation block whose sub-block sums are `sum`
  __device__ __forceinline__ float close(const i32x4 (&dots)[2], const int *sum, float scale) const {
    int scaled = 0, minima = 0;
#pragma unroll
    for (uint32_t s = 0; s < 8; ++s) {
      scaled = mad24(sc[s], dots[s / 4][s % 4], scaled);
      minima = mad24(mn[s], sum[s], minima);
    }
    return scale * (d * (float)scaled - dmin * (float)minima);
  }
};

// `blocks` >= 4 Q4_K blocks per row.  kSets == 0: one activation row; kSets == 1, 2: four or eight
// (rows past m repeat the last one and are not stored).  1 << split_log2 waves share a tile of
// sixteen weight rows: wave w of them walks the groups w, w + split, ... and the first adds the
// shares in wave order.
template <class TX, int kSets, bool kOneBatch>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_q8_tiles(const unsigned char *weights, const void *x, void *y,
                                                                      uint32_t rows, uint64_t row_stride, uint32_t blocks,
                                                                      uint32_t m, uint32_t split_log2) {
  constexpr uint32_t kTokens = kSets == 0 ? 1 : 4 * kSets;
  constexpr int kTotals = kSets == 0 ? 1 : kSets;
  extern __shared__ __align__(16) unsigned char shared[];
  const uint32_t k = blocks * 256;
  unsigned char *codes = shared + k;  // behind the row of zeros
  int *sums = reinterpret_cast<int *>(shared + (size_t)(1 + kTokens) * k);
  float *scales = reinterpret_cast<float *>(sums + (size_t)kTokens * blocks * 8);
  float *shares = scales + (size_t)kTokens * blocks;
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  const uint32_t column = lane % 16, part = lane / 16;
  const uint32_t split = 1u << split_log2, member = wave & (split - 1);
  const uint32_t row = ((blockIdx.x * kWavesPerBlock + wave) >> split_log2) * kTileRows + column;
  // rows past the last repeat it (valid addresses) and are not stored
  const unsigned char *mine = weights + (size_t)(row < rows ? row : rows - 1) * row_stride;
  const uint32_t groups = (blocks + 3) / 4;
  // A row's last group starts at its fourth block from the end: when the row is not a whole number
  // of groups it overlaps the one before, and the blocks they share are skipped.
  auto start_of = [&](uint32_t g) { return 4 * g + 4 <= blocks ? 4 * g : blocks - 4; };
  const unsigned char *heads = mine + part * 144, *chunks = mine + 16 + part * 16;
  auto load_group = [&](uint32_t g) {
    TileGroup out;
    const size_t start = (size_t)start_of(g) * 144;
    out.head = load16(heads + start, 0);
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b)
#pragma unroll
      for (uint32_t i = 0; i < 2; ++i) out.quants[b][i] = load16(chunks + start, b * 9 + 4 * i);
    return out;
  };
  auto clamped = [&](uint32_t g) { return g < groups ? g : groups - 1; };
  // activation blocks go round the block's eight half waves, four (eight) of a half wave's loads in flight;
  // the first round is asked for before the weights: loads return in order
  constexpr uint32_t kHalves = kBlockThreads / 32, kBatch = kSets == 2 ? 8 : 4;  // (eight activation rows of 2048 values are 64 blocks)
  const uint32_t half = threadIdx.x / 32, u = threadIdx.x % 32;
  const uint32_t units = kTokens * blocks;
  auto fetch_batch = [&](uint32_t first, TileValues (&fetched)[kBatch]) {
#pragma unroll
    for (uint32_t j = 0; j < kBatch; ++j) {
      const uint32_t unit = first + j * kHalves < units ? first + j * kHalves : units - 1;
      const uint32_t token = unit / blocks, block = unit - token * blocks;
      fetched[j] = tile_fetch<TX>(x, (size_t)(token < m ? token : m - 1) * k + (size_t)block * 256, u);
    }
  };
  auto quantise_batch = [&](uint32_t first, const TileValues (&fetched)[kBatch]) {
#pragma unroll
    for (uint32_t j = 0; j < kBatch; ++j) {
      const uint32_t unit = first + j * kHalves;
      if (unit < units) tile_quantise<TX>(fetched[j], u, codes + (size_t)unit * 256, sums + (size_t)unit * 8, scales + unit);
    }
  };
  TileValues fetched[kBatch];
  fetch_batch(half, fetched);
  TileGroup ring[2];
  ring[0] = load_group(clamped(member));
  ring[1] = load_group(clamped(member + split));
  for (uint32_t at = threadIdx.x * 16; at < k; at += kBlockThreads * 16) *reinterpret_cast<u32x4 *>(shared + at) = u32x4{0u, 0u, 0u, 0u};
  quantise_batch(half, fetched);
  if constexpr (!kOneBatch) {  // more activation blocks than one round takes: the rest wait for the weights before them
    for (uint32_t first = half + kHalves * kBatch; first < units; first += kHalves * kBatch) {
      fetch_batch(first, fetched);
      quantise_batch(first, fetched);
    }
  }
  lds_barrier();
  float totals[kTotals] = {};
  if constexpr (kSets == 0) {
    // rows of A: 4 b + 2 (part / 2) + nibble.  The lane's codes (block column / 4 of the group, nibble
    // column % 2, if column / 2 and part / 2 agree in their low bit) go to instruction (b, nibble).
    uint32_t base[4][2];
    {
      const bool faces = ((column >> 1) & 1u) == (part >> 1);
      const uint32_t own = k + (column / 4) * 256 + (part >> 1) * 64 + (column & 1u) * 32 + (part & 1u) * 16;
#pragma unroll
      for (uint32_t b = 0; b < 4; ++b)
#pragma unroll
        for (uint32_t nibble = 0; nibble < 2; ++nibble) base[b][nibble] = faces && column / 4 == b && (column & 1u) == nibble ? own : 0u;
    }
    auto work = [&](const TileGroup &held, uint32_t g, auto whole) {
      constexpr bool kWhole = decltype(whole)::value;  // the usual group, none of its blocks skipped: no branch in it
      const uint32_t start = start_of(g), skipped = kWhole ? 0u : 4 * g - start;
      i32x4 dots[2] = {i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}};
#pragma unroll
      for (uint32_t b = 0; b < 4; ++b) {
        if (!kWhole && b < skipped) continue;  // the same for the whole wave
#pragma unroll
        for (uint32_t i = 0; i < 2; ++i) {
          const u32x4 q = held.quants[b][i];
          const u32x4 nibbles[2] = {q & 0x0F0F0F0Fu, (q >> 4) & 0x0F0F0F0Fu};
#pragma unroll
          for (uint32_t nibble = 0; nibble < 2; ++nibble) {
            const u32x4 operand = *reinterpret_cast<const u32x4 *>(shared + base[b][nibble] + start * 256 + i * 128);
            dots[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)operand, (i32x4)nibbles[nibble], dots[i], 0, 0, 0);
          }
        }
      }
      if (kWhole || part >= skipped) {  // block start + part of the lane's row
        const uint32_t block = start + part;
        totals[0] += TileFactors(held.head).close(dots, sums + (size_t)block * 8, scales[block]);
      }
    };
    auto step = [&](const TileGroup &held, uint32_t g) {
      if (4 * g + 4 <= blocks) work(held, g, std::true_type{});
      else work(held, g, std::false_type{});
    };
    if (member + 2 * split >= groups) {
      // at most two groups, both in flight: straight-line code, every block starts as soon as its bytes are there
      step(ring[0], member);
      if (member + split < groups) step(ring[1], member + split);
    } else {
      for (uint32_t g = member; g < groups; g += 2 * split) {
#pragma unroll
        for (uint32_t slot = 0; slot < 2; ++slot) {
          const uint32_t now = g + slot * split;
          if (now >= groups) break;
          step(ring[slot], now);
          if (now + 2 * split < groups) ring[slot] = load_group(now + 2 * split);  // the other slot's bytes are in flight
        }
      }
    }
    totals[0] += __shfl_xor(totals[0], 16, kWaveLanes);
    totals[0] += __shfl_xor(totals[0], 32, kWaveLanes);
  } else {
    // rows of A: 4 t + 2 (part / 2) + nibble for activation row t of a set.  The lane's codes
    // (activation row column / 4, nibble column % 2, if column / 2 and part / 2 agree in their low
    // bit) go to the instructions of that nibble.
    uint32_t base[kSets][2];
    {
      const bool faces = ((column >> 1) & 1u) == (part >> 1);
#pragma unroll
      for (uint32_t set = 0; set < (uint32_t)kSets; ++set) {
        const uint32_t own = k * (1 + 4 * set + column / 4) + (part >> 1) * 64 + (column & 1u) * 32 + (part & 1u) * 16;
#pragma unroll
        for (uint32_t nibble = 0; nibble < 2; ++nibble) base[set][nibble] = faces && (column & 1u) == nibble ? own : 0u;
      }
    }
    auto work = [&](const TileGroup &held, uint32_t g, auto whole) {
      constexpr bool kWhole = decltype(whole)::value;
      const uint32_t start = start_of(g), skipped = kWhole ? 0u : 4 * g - start;
#pragma unroll
      for (uint32_t b = 0; b < 4; ++b) {
        if (!kWhole && b < skipped) continue;  // the same for the whole wave
        const uint32_t block = start + b;
        i32x4 dots[kSets][2];
#pragma unroll
        for (int set = 0; set < kSets; ++set) dots[set][0] = dots[set][1] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (uint32_t i = 0; i < 2; ++i) {
          const u32x4 q = held.quants[b][i];
          const u32x4 nibbles[2] = {q & 0x0F0F0F0Fu, (q >> 4) & 0x0F0F0F0Fu};
#pragma unroll
          for (uint32_t nibble = 0; nibble < 2; ++nibble) {
#pragma unroll
            for (int set = 0; set < kSets; ++set) {
              const u32x4 operand = *reinterpret_cast<const u32x4 *>(shared + base[set][nibble] + block * 256 + i * 128);
              dots[set][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)operand, (i32x4)nibbles[nibble], dots[set][i], 0, 0, 0);
            }
          }
        }
        // the header of block b is with lane (column, b); the lane closes the block against activation row part of every set
        const int from = (int)(column + 16 * b);
        const TileFactors factors(u32x4{(uint32_t)__shfl((int)held.head.x, from, kWaveLanes), (uint32_t)__shfl((int)held.head.y, from, kWaveLanes),
                                        (uint32_t)__shfl((int)held.head.z, from, kWaveLanes), (uint32_t)__shfl((int)held.head.w, from, kWaveLanes)});
#pragma unroll
        for (int set = 0; set < kSets; ++set) {
          const uint32_t unit = (4 * (uint32_t)set + part) * blocks + block;
          totals[set] += factors.close(dots[set], sums + (size_t)unit * 8, scales[unit]);
        }
      }
    };
    auto step = [&](const TileGroup &held, uint32_t g) {
      if (4 * g + 4 <= blocks) work(held, g, std::true_type{});
      else work(held, g, std::false_type{});
    };
    if (member + 2 * split >= groups) {
      // at most two groups, both in flight: straight-line code, every block starts as soon as its bytes are there
      step(ring[0], member);
      if (member + split < groups) step(ring[1], member + split);
    } else {
      for (uint32_t g = member; g < groups; g += 2 * split) {
#pragma unroll
        for (uint32_t slot = 0; slot < 2; ++slot) {
          const uint32_t now = g + slot * split;
          if (now >= groups) break;
          step(ring[slot], now);
          if (now + 2 * split < groups) ring[slot] = load_group(now + 2 * split);  // the other slot's bytes are in flight
        }
      }
    }
  }
  if (split_log2 != 0) {
#pragma unroll
    for (int t = 0; t < kTotals; ++t) shares[((size_t)wave * kWaveLanes + lane) * kTotals + t] = totals[t];
    lds_barrier();
    if (member != 0) return;
#pragma unroll
    for (int t = 0; t < kTotals; ++t)
      for (uint32_t other = 1; other < split; ++other) totals[t] += shares[((size_t)(wave + other) * kWaveLanes + lane) * kTotals + t];
  }
  if (row < rows) {
    if constexpr (kSets == 0) {
      if (part == 0) Traits<TX>::store(y, (size_t)row, totals[0]);
    } else {
#pragma unroll
      for (uint32_t set = 0; set < (uint32_t)kSets; ++set)
        if (4 * set + part < m) Traits<TX>::store(y, (size_t)(4 * set + part) * rows + row, totals[set]);
    }
  }
}

inline const char *kind_word(int kind) { return kind == 0 ? "q4_k" : (kind == 1 ? "q6_k" : "q8_0"); }
// gguf_matvec_q8_<form>/<format>[/<detail>]
template <int kKind, int kSets, bool kRegisters> struct QuadsTag {
  static std::string text() {
    return std::string("gguf_matvec_q8_quads/") + kind_word(kKind) + "/" + std::to_string(4 * kSets) + "-tokens" + (kRegisters ? "/registers" : "/lds");
  }
};
template <int kKind, int kM, bool kRegisters> struct LinesTag {
  static std::string text() {
    return std::string("gguf_matvec_q8_lines/") + kind_word(kKind) + "/" + std::to_string(kM) + "-tokens" + (kRegisters ? "/registers" : "/lds");
  }
};
template <int kKind, int kSpans, bool kShort> struct SpansTag {
  static std::string text() {
    return std::string("gguf_matvec_q8_spans/") + kind_word(kKind) + "/" + std::to_string(kSpans) + "-spans" + (kShort ? "/short" : "");
  }
};
template <int kSets, bool kOneBatch> struct TilesTag {
  static std::string text() {
    return "gguf_matvec_q8_tiles/q4_k/" + std::to_string(kSets == 0 ? 1 : 4 * kSets) + "-tokens" + (kOneBatch ? "" : "/long");
  }
};
template <int kKind, int kM> struct BlocksTag {
  static std::string text() { return std::string("gguf_matvec_q8_blocks/") + kind_word(kKind) + "/" + std::to_string(kM) + "-tokens"; }
};

// ---- any whole number of blocks per row, rows at any even byte stride ---------------------------
// The kernels above want rows of 2048 n values made of whole 16-byte vectors.  The reference's own
// projection shapes are wider than that (K = 128, 1024, 5120, 7168, 17408;
// tests/compute_models/cpu_c5_gguf_inputs.h:231-314), and a GGUF row of Q6_K or Q8_0 blocks starts on a
// 16-byte boundary only when K is a multiple of 2048 or 256.  Here every block first quantises the
// activation rows into LDS in their natural order (int8 codes [m][K], one f32 scale per activation
// block), then a wave walks its weight rows 1024 values at a time: the aligned 16-byte vectors that
// cover the step's bytes go through a wave-private LDS slot (the next step's are in flight
// meanwhile), sixteen lanes take each run of 256 values -- the pieces of the K-quant block, or eight
// Q8_0 blocks, two lanes each -- from aligned LDS words and a funnel shift by the step's byte
// offset, and meet the codes of the same positions with v_dot4c_i32_i8.  Same integer dots and f32
// closing products as the span kernels; only the order of the f32 sums differs.
template <int kWords> __device__ __forceinline__ void lds_words(const unsigned char *base, uint32_t offset, uint32_t (&out)[kWords]) {
  const uint32_t *words = reinterpret_cast<const uint32_t *>(base + (offset & ~3u));
  uint32_t w[kWords + 1];
#pragma unroll
  for (int i = 0; i <= kWords; ++i) w[i] = words[i];
#pragma unroll
  for (int i = 0; i < kWords; ++i) out[i] = __builtin_amdgcn_alignbyte(w[i + 1], w[i], offset & 3u);
}

template <int kKind> struct BlocksGeometry;
template <> struct BlocksGeometry<0> {  // Q4_K
  static constexpr uint32_t kRunBytes = 144, kActivationBlock = 256;
};
template <> struct BlocksGeometry<1> {  // Q6_K
  static constexpr uint32_t kRunBytes = 210, kActivationBlock = 256;
};
template <> struct BlocksGeometry<2> {  // Q8_0: a run of 256 values is eight blocks of 34 bytes
  static constexpr uint32_t kRunBytes = 272, kActivationBlock = 32;
};
constexpr int kBlocksDepth = 4;  // steps of a wave whose bytes are in flight
template <int kKind> struct BlocksStep {
  static constexpr uint32_t kBytes = 4 * BlocksGeometry<kKind>::kRunBytes;   // 1024 values of a row
  static constexpr int kLoads = (int)((kBytes + 14 + 15) / 16 + kWaveLanes - 1) / kWaveLanes;
  static constexpr uint32_t kSlotBytes = kLoads * kWaveLanes * 16;
};

// One lane's sixteen values of a run of 256 (run `at` bytes into the slot) against the codes of the
// same positions of one activation row; `codes` points at the row's codes of this run.
template <int kKind> struct RunDot;
template <> struct RunDot<0> {  // lane u: chunk u / 4, quant bytes 8 (u % 4) .. + 7: low nibbles sub-block 2 c, high 2 c + 1
  uint32_t low[2], high[2];
  int sc_low, sc_high, m_low, m_high;
  float d, dmin;
  uint32_t first;  // position of the lane's low-nibble values inside the run
  __device__ __forceinline__ void decode(const unsigned char *slot, uint32_t at, uint32_t u) {
    const uint32_t chunk = u / 4;
    uint32_t head[4], quants[2];
    lds_words<4>(slot, at, head);
    lds_words<2>(slot, at + 16 + 32 * chunk + 8 * (u % 4), quants);
    d = f16_to_f32((uint16_t)head[0]);
    dmin = f16_to_f32((uint16_t)(head[0] >> 16));
    // sub-blocks 2 c and 2 c + 1 sit in one half of the table (both below 4 or both from 4 on), in
    // neighbouring bytes: one branch per lane, the same in every step
    const uint32_t shift = 16 * (chunk % 2);
    if (chunk < 2) {  // six bits whole: sc in scales[j], m in scales[j + 4]
      const uint32_t sc = head[1] >> shift, mn = head[2] >> shift;
      sc_low = (int)(sc & 63u);
      sc_high = (int)((sc >> 8) & 63u);
      m_low = (int)(mn & 63u);
      m_high = (int)((mn >> 8) & 63u);
    } else {  // four bits in a nibble of scales[j + 4], two more in the top of scales[j - 4] (sc) or scales[j] (m)
      const uint32_t main = head[3] >> shift, sc_top = head[1] >> shift, m_top = head[2] >> shift;
      sc_low = (int)((main & 15u) | ((sc_top >> 2) & 48u));
      sc_high = (int)(((main >> 8) & 15u) | ((sc_top >> 10) & 48u));
      m_low = (int)(((main >> 4) & 15u) | ((m_top >> 2) & 48u));
      m_high = (int)(((main >> 12) & 15u) | ((m_top >> 10) & 48u));
    }
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      low[w] = quants[w] & 0x0F0F0F0Fu;
      high[w] = (quants[w] >> 4) & 0x0F0F0F0Fu;
    }
    first = 64 * chunk + 8 * (u % 4);
  }
  __device__ __forceinline__ float against(const unsigned char *codes, float a_scale) const {
    const uint32_t *lo = reinterpret_cast<const uint32_t *>(codes + first);
    const uint32_t *hi = reinterpret_cast<const uint32_t *>(codes + first + 32);
    const uint32_t c0 = lo[0], c1 = lo[1], c2 = hi[0], c3 = hi[1];
    const int lows = dot4(low[0], c0, dot4(low[1], c1, 0)), highs = dot4(high[0], c2, dot4(high[1], c3, 0));
    const int sum_low = dot4(0x01010101u, c0, dot4(0x01010101u, c1, 0)), sum_high = dot4(0x01010101u, c2, dot4(0x01010101u, c3, 0));
    const int scaled = mad24(sc_low, lows, __mul24(sc_high, highs));
    const int minima = mad24(m_low, sum_low, __mul24(m_high, sum_high));
    return a_scale * (d * (float)scaled - dmin * (float)minima);
  }
};
template <> struct RunDot<1> {  // lane u: half u / 8, positions 4 j .. 4 j + 3 (j = u % 8) of the half's four groups of 32
  uint32_t q[4];
  int scale[4];
  float step;  // d / 4
  uint32_t first;
  __device__ __forceinline__ void decode(const unsigned char *slot, uint32_t at, uint32_t u) {
    const uint32_t half = u / 8, j = u % 8;
    uint32_t a[1], b[1], t[1], scales[2];
    lds_words<1>(slot, at + 64 * half + 4 * j, a);
    lds_words<1>(slot, at + 64 * half + 32 + 4 * j, b);
    lds_words<1>(slot, at + 128 + 32 * half + 4 * j, t);
    lds_words<2>(slot, at + 192 + 8 * half, scales);
    step = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + at + 208)) * 0.25f;
    const uint32_t top = t[0] ^ 0xAAAAAAAAu;  // q - 32 modulo 64: bytes of 4 (q - 32) as int8
    q[0] = ((a[0] << 2) & 0x3C3C3C3Cu) | ((top << 6) & 0xC0C0C0C0u);
    q[1] = ((b[0] << 2) & 0x3C3C3C3Cu) | ((top << 4) & 0xC0C0C0C0u);
    q[2] = ((a[0] >> 2) & 0x3C3C3C3Cu) | ((top << 2) & 0xC0C0C0C0u);
    q[3] = ((b[0] >> 2) & 0x3C3C3C3Cu) | (top & 0xC0C0C0C0u);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t byte = 2 * g + j / 4;  // scales[8 half + 2 g + l / 16], l = 4 j
      scale[g] = (int)(signed char)(scales[byte / 4] >> (8 * (byte % 4)));
    }
    first = 128 * half + 4 * j;
  }
  __device__ __forceinline__ float against(const unsigned char *codes, float a_scale) const {
    int total = 0;
#pragma unroll
    for (int g = 0; g < 4; ++g)
      total = mad24(scale[g], dot4(q[g], *reinterpret_cast<const uint32_t *>(codes + first + 32 * g), 0), total);
    return (step * a_scale) * (float)total;
  }
};
template <> struct RunDot<2> {  // lane u: block u / 2 of the run's eight, quants 16 (u % 2) .. + 15
  uint32_t q[4];
  float d;
  uint32_t first;
  __device__ __forceinline__ void decode(const unsigned char *slot, uint32_t at, uint32_t u) {
    const uint32_t block = at + 34 * (u / 2);
    lds_words<4>(slot, block + 2 + 16 * (u % 2), q);
    d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + block));
    first = 16 * u;
  }
  __device__ __forceinline__ float against(const unsigned char *codes, float a_scale) const {
    const uint32_t *c = reinterpret_cast<const uint32_t *>(codes + first);
    int total = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) total = dot4(q[i], c[i], total);
    return (d * a_scale) * (float)total;
  }
};

// staged: int8 codes [m][k], then f32 scales [m][k / activation block].  kM: activation rows
// served at once (rows past m repeat the last one and are not stored).  kVectorX: x starts on a
// 16-byte boundary, so its rows (K is a multiple of 32) are read as whole vectors.
template <int kKind, class TX, int kM, bool kVectorX>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_q8_blocks(const unsigned char *weights, const void *x, void *y,
                                                                       uint32_t rows, uint64_t row_stride, uint32_t k,
                                                                       uint32_t m) {
  using Geometry = BlocksGeometry<kKind>;
  using Step = BlocksStep<kKind>;
  constexpr uint32_t kActivationBlock = Geometry::kActivationBlock;
  constexpr int kQuantiseLanes = kActivationBlock / 8;  // a lane quantises eight neighbouring values
  __shared__ __align__(16) unsigned char slots[kWavesPerBlock][Step::kSlotBytes];
  extern __shared__ __align__(16) uint32_t staged[];
  unsigned char *codes = reinterpret_cast<unsigned char *>(staged);
  float *scales = reinterpret_cast<float *>(codes + (size_t)m * k);  // k is a multiple of 32: aligned
  const uint32_t activation_blocks = k / kActivationBlock;
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);

  // ---- what the wave walks: its rows, 1024 values (a step) at a time ---------------------------
  const uint32_t stride = gridDim.x * kWavesPerBlock;
  const uint32_t first = blockIdx.x * kWavesPerBlock + wave;
  unsigned char *slot = slots[wave];
  const uint32_t runs = (k + 255) / 256;           // runs of 256 values in a row (the last one of a Q8_0 row may be short)
  const uint32_t steps = (runs + 3) / 4;
  const uint64_t row_bytes = (uint64_t)(k / kActivationBlock) * (kKind == 2 ? 34u : Geometry::kRunBytes);
  const uint32_t run = lane / 16, u = lane % 16;
  const uint32_t own_rows = first < rows ? (rows - first + stride - 1) / stride : 0u;
  const uint64_t segments = (uint64_t)own_rows * steps;  // (row, step) pairs of this wave, in order

  // The aligned 16-byte vectors that cover one step of one row; lanes past them repeat the last
  // one.  The stream of loads runs kBlocksDepth steps ahead of the stream of decodes; past the
  // wave's last step it reads the wave's first one again, a valid address whose bytes go unused.
  uint32_t load_row = first, load_step = 0;
  uint64_t loaded = 0;
  auto next_load = [&](u32x4 (&into)[Step::kLoads], uint32_t *shift) {
    const bool live = loaded < segments;
    const uint32_t row = live ? load_row : first, step = live ? load_step : 0u;
    ++loaded;
    if (++load_step == steps) {
      load_step = 0;
      load_row += stride;
    }
    const uint64_t begin = (uint64_t)row * row_stride + (uint64_t)step * Step::kBytes;
    const uint64_t left = row_bytes - (uint64_t)step * Step::kBytes;
    const uint32_t bytes = left < Step::kBytes ? (uint32_t)left : Step::kBytes;
    const uintptr_t address = reinterpret_cast<uintptr_t>(weights) + begin;
    const uint32_t off = (uint32_t)(address & 15u);
    const u32x4 *vectors = reinterpret_cast<const u32x4 *>(address - off);
    const uint32_t needed = (off + bytes + 15) / 16;
#pragma unroll
    for (int i = 0; i < Step::kLoads; ++i) {
      const uint32_t wanted = lane + i * kWaveLanes;
      into[i] = __builtin_nontemporal_load(vectors + (wanted < needed ? wanted : needed - 1));
    }
    *shift = off;
  };
  u32x4 ring[kBlocksDepth][Step::kLoads];
  uint32_t shifts[kBlocksDepth] = {};
  if (segments != 0) {  // the wave's first steps are on their way while the block quantises the activations
#pragma unroll
    for (int d = 0; d < kBlocksDepth; ++d) next_load(ring[d], &shifts[d]);
  }

  // ---- the activation rows, quantised once per block ------------------------------------------
  // A thread takes eight neighbouring values at a time (one 16-byte vector of a narrow type, two of
  // f32, when x allows vector loads), the next eight already on their way.
  auto fetch_values = [&](uint32_t r, uint32_t p, float (&values)[8]) {
    const bool inside = p < k;
    const size_t at = (size_t)r * k + (inside ? p : 0u);  // a thread past the row reads its start and keeps nothing
    if constexpr (kVectorX) {
      if constexpr (Traits<TX>::kVec == 8) {
        Traits<TX>::unpack(load16(x, at / 8), values);
      } else {
        float half[4];
        Traits<TX>::unpack(load16(x, at / 4), half);
#pragma unroll
        for (int e = 0; e < 4; ++e) values[e] = half[e];
        Traits<TX>::unpack(load16(x, at / 4 + 1), half);
#pragma unroll
        for (int e = 0; e < 4; ++e) values[4 + e] = half[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) values[e] = Traits<TX>::load(x, at + e);
    }
    if (!inside) {
#pragma unroll
      for (int e = 0; e < 8; ++e) values[e] = 0.0f;
    }
  };
  const uint32_t pieces = (k + kBlockThreads * 8 - 1) / (kBlockThreads * 8);  // per activation row
  const uint32_t turns = m * pieces;
  float ahead[8];
  if (turns != 0) fetch_values(0, threadIdx.x * 8, ahead);
  for (uint32_t turn = 0; turn < turns; ++turn) {
    const uint32_t r = turn / pieces, p = (turn % pieces) * (kBlockThreads * 8) + threadIdx.x * 8;
    const bool inside = p < k;  // the same for all lanes that share an activation block
    float values[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) values[e] = ahead[e];
    if (turn + 1 < turns)
      fetch_values((turn + 1) / pieces, ((turn + 1) % pieces) * (kBlockThreads * 8) + threadIdx.x * 8, ahead);
    LaneMax mine{0.0f, 0.0f, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e) {  // positions rise with e, so ">" keeps the first
      const float magnitude = __builtin_fabsf(values[e]);
      if (magnitude > mine.magnitude) mine = LaneMax{magnitude, values[e], p + e};
    }
    if (mine.magnitude == 0.0f) mine.position = 0xFFFFFFFFu;  // no candidate: any lane with one goes first
    const LaneMax top = block_largest<kQuantiseLanes>(mine);
    float factor = 0.0f, stored = 0.0f;
    if (top.magnitude != 0.0f) {
      if constexpr (kKind == 2) {
        stored = f16_to_f32(f32_to_f16(top.magnitude / 127.0f));
        factor = 127.0f / top.magnitude;
      } else {
        factor = -127.0f / top.value;
        stored = 1.0f / factor;
      }
    }
    uint32_t words[2] = {0u, 0u};
    if (top.magnitude != 0.0f) {
#pragma unroll
      for (int e = 0; e < 8; ++e) words[e / 4] |= code_of(values[e] * factor) << (8 * (e % 4));
    }
    if (inside) {
      uint32_t *to = reinterpret_cast<uint32_t *>(codes + (size_t)r * k + p);
      to[0] = words[0];
      to[1] = words[1];
      if (p % kActivationBlock == 0) scales[r * activation_blocks + p / kActivationBlock] = stored;
    }
  }
  __syncthreads();
  if (own_rows == 0) return;  // no barrier follows
  if (steps == 0) {  // K = 0: every product is an empty sum
    for (uint32_t row = first; row < rows; row += stride)
      if (lane < m) Traits<TX>::store(y, (size_t)lane * rows + row, 0.0f);
    return;
  }

  // ---- the weight rows ----------------------------------------------------------------------
  uint32_t row = first, step = 0;
  float totals[kM] = {};
  for (uint64_t done = 0; done < segments; done += kBlocksDepth) {
#pragma unroll
    for (int d = 0; d < kBlocksDepth; ++d) {
      if (done + d >= segments) break;
#pragma unroll
      for (int i = 0; i < Step::kLoads; ++i) *reinterpret_cast<u32x4 *>(slot + (size_t)(lane + i * kWaveLanes) * 16) = ring[d][i];
      const uint32_t at = shifts[d] + run * Geometry::kRunBytes;
      next_load(ring[d], &shifts[d]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const uint32_t run_index = step * 4 + run;
      const uint32_t position = run_index * 256 + (kKind == 2 ? 16 * u : 0u);  // of the lane's first value (K-quants: of its run)
      const bool live = position < k;
      RunDot<kKind> decoded;
      decoded.decode(slot, at, u);
      if (!live) decoded.first = 0;  // a lane past the row reads the row's first codes and adds nothing
      const uint32_t run_codes = live ? run_index * 256 : 0u;
      const uint32_t scale_index = live ? (kKind == 2 ? run_index * 8 + u / 2 : run_index) : 0u;
#pragma unroll
      for (int r = 0; r < kM; ++r) {
        const uint32_t token = (uint32_t)r < m ? (uint32_t)r : m - 1;
        const float part = decoded.against(codes + (size_t)token * k + run_codes, scales[token * activation_blocks + scale_index]);
        totals[r] += live ? part : 0.0f;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (++step == steps) {  // the row is complete
#pragma unroll
        for (int r = 0; r < kM; ++r) {
          const float whole = group_sum<kWaveLanes>(totals[r]);
          if (lane == 0 && (uint32_t)r < m) Traits<TX>::store(y, (size_t)r * rows + row, whole);
          totals[r] = 0.0f;
        }
        step = 0;
        row += stride;
      }
    }
  }
}

// Bytes of LDS one activation row takes in gguf_matvec_q8_blocks.
inline size_t blocks_row_bytes(int kind, uint32_t k) { return (size_t)k + (size_t)(k / (kind == 2 ? 32u : 256u)) * sizeof(float); }
constexpr size_t kBlocksSharedBudget = 56 * 1024;  // beside the waves' row slots (at most 8 KiB) in a block's 64 KiB

template <int kKind, class TX>
hipError_t run_blocks(const MatVecParams &p, const void *w, const void *x, void *y, int compute_units, hipStream_t s) {
  const size_t per_row = blocks_row_bytes(kKind, p.k);
  uint32_t fit = per_row == 0 ? 8u : (uint32_t)(kBlocksSharedBudget / per_row);
  if (fit == 0) return hipErrorInvalidValue;  // the plan declines such K
  fit = fit >= 8 ? 8 : (fit >= 4 ? 4 : (fit >= 2 ? 2 : 1));
  const uint32_t wanted = (uint32_t)((p.rows + kWavesPerBlock - 1) / kWavesPerBlock);
  const uint32_t machine = (uint32_t)(compute_units > 0 ? compute_units : 256) * 3u;  // three blocks per compute unit
  const dim3 grid(wanted < machine ? wanted : machine);
  const unsigned char *in = static_cast<const unsigned char *>(w);
  // activation rows in groups that fit LDS together; every group walks the weight again
  for (uint32_t done = 0; done < p.m; done += fit) {
    const uint32_t m = p.m - done < fit ? p.m - done : fit;
    const void *xs = static_cast<const char *>(x) + (size_t)done * p.k * Traits<TX>::kSize;
    void *ys = static_cast<char *>(y) + (size_t)done * p.rows * Traits<TX>::kSize;
    const size_t shared = m * per_row;
    const bool vector_x = (reinterpret_cast<uintptr_t>(xs) & 15u) == 0;
#define HYLE_BLOCKS(M)                                                                                                          \
  note_variant<BlocksTag<kKind, M>>();                                                                                          \
  if (vector_x)                                                                                                                 \
    hipLaunchKernelGGL((gguf_matvec_q8_blocks<kKind, TX, M, true>), grid, dim3(kBlockThreads), shared, s, in, xs, ys,          \
                       (uint32_t)p.rows, p.row_stride, p.k, m);                                                                 \
  else                                                                                                                          \
    hipLaunchKernelGGL((gguf_matvec_q8_blocks<kKind, TX, M, false>), grid, dim3(kBlockThreads), shared, s, in, xs, ys,         \
                       (uint32_t)p.rows, p.row_stride, p.k, m)
    if (m == 1) { HYLE_BLOCKS(1); }
    else if (m == 2) { HYLE_BLOCKS(2); }
    else if (m <= 4) { HYLE_BLOCKS(4); }
    else { HYLE_BLOCKS(8); }
#undef HYLE_BLOCKS
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  return hipSuccess;
}

template <int kKind, class TX>
hipError_t run_quads(const MatVecParams &p, const void *w, const void *x, void *y, uint32_t spans, dim3 grid,
                     size_t shared, hipStream_t s) {
  const unsigned char *in = static_cast<const unsigned char *>(w);
#define HYLE_QUADS(SETS, REGISTERS)                                                                             \
  note_variant<QuadsTag<kKind, SETS, REGISTERS>>();                                                                 \
  hipLaunchKernelGGL((gguf_matvec_q8_quads<kKind, TX, SETS, REGISTERS>), grid, dim3(kBlockThreads), shared, s, in, x, \
                     y, (uint32_t)p.rows, p.row_stride, spans, p.m)
  // Which forms a shape can reach follows from what fits a block's LDS beside the four row slots per
  // wave (run_m): one set of four tokens for every format, with the codes in registers when K = 2048
  // two sets only for Q6_K at K = 2048 (codes in registers); Q8_0's wider slots leave no room for a
  // second set.  (Q4_K takes the tile kernel.)
  const bool registers = spans == 1;
  if (p.m <= 4) {
    if (registers) { HYLE_QUADS(1, true); }
    else { HYLE_QUADS(1, false); }
  } else if constexpr (kKind == 1) {
    if (!registers) return hipErrorInvalidValue;
    HYLE_QUADS(2, true);
  } else {
    return hipErrorInvalidValue;
  }
#undef HYLE_QUADS
  return hipGetLastError();
}

template <int kKind, class TX, int kM>
hipError_t run_registers(const MatVecParams &p, const void *w, const void *x, void *y, uint32_t spans, dim3 grid,
                         size_t shared, hipStream_t s) {
  const unsigned char *in = static_cast<const unsigned char *>(w);
  // One span per row with the codes in registers is reached by Q8_0 with 5 to 8 tokens only (every
  // other K = 2048 shape takes the span or the quad kernel); the form that fetches the codes from
  // LDS serves any number of spans.
  if constexpr (kKind == 2 && kM == 8) {
    if (spans == 1) {
      note_variant<LinesTag<kKind, kM, true>>();
      hipLaunchKernelGGL((gguf_matvec_q8_lines<kKind, TX, kM, true>), grid, dim3(kBlockThreads), shared, s, in, x, y,
                         (uint32_t)p.rows, p.row_stride, spans, p.m);
      return hipGetLastError();
    }
  }
  note_variant<LinesTag<kKind, kM, false>>();
  hipLaunchKernelGGL((gguf_matvec_q8_lines<kKind, TX, kM, false>), grid, dim3(kBlockThreads), shared, s, in, x, y,
                     (uint32_t)p.rows, p.row_stride, spans, p.m);
  return hipGetLastError();
}

// One activation row: a wave per span.  Eight waves per compute unit measured best or equal in
// 25 of 27 shapes (three formats, K = 2048 ... 12288, 1024 ... 151936 rows: 0-30 % below the
// kernel that parks the codes in LDS first).
template <int kKind, class TX>
hipError_t run_spans(const MatVecParams &p, const void *w, const void *x, void *y, uint32_t spans, uint32_t tail_lanes,
                     int compute_units, hipStream_t s) {
  const uint32_t units = (uint32_t)(compute_units > 0 ? compute_units : 256);
  const uint32_t most = units * (spans <= 8 ? 8u / spans : 1u);
  const dim3 blocks((uint32_t)p.rows < most ? (uint32_t)p.rows : most);
  const unsigned char *in = static_cast<const unsigned char *>(w);
  const uint32_t rows = (uint32_t)p.rows;
#define HYLE_SPANS(N, SHORT)                                                                                             \
  note_variant<SpansTag<kKind, N, SHORT>>();                                                                             \
  hipLaunchKernelGGL((gguf_matvec_q8_spans<kKind, TX, N, SHORT>), blocks, dim3(N * kWaveLanes), 0, s, in, x, y, rows,      \
                     p.row_stride, tail_lanes)
  if (tail_lanes == kWaveLanes) {
    switch (spans) {
      case 1: HYLE_SPANS(1, false); break;
      case 2: HYLE_SPANS(2, false); break;
      case 3: HYLE_SPANS(3, false); break;
      case 4: HYLE_SPANS(4, false); break;
      case 5: HYLE_SPANS(5, false); break;
      case 6: HYLE_SPANS(6, false); break;
      default: return hipErrorInvalidValue;  // whole rows of more spans take the kernel that parks the codes
    }
  } else if constexpr (kKind == 2) {
    switch (spans) {
      case 1: HYLE_SPANS(1, true); break;
      case 2: HYLE_SPANS(2, true); break;
      case 3: HYLE_SPANS(3, true); break;
      case 4: HYLE_SPANS(4, true); break;
      case 5: HYLE_SPANS(5, true); break;
      case 6: HYLE_SPANS(6, true); break;
      case 7: HYLE_SPANS(7, true); break;
      case 8: HYLE_SPANS(8, true); break;
      case 9: HYLE_SPANS(9, true); break;
      default: return hipErrorInvalidValue;
    }
  } else {
    return hipErrorInvalidValue;
  }
#undef HYLE_SPANS
  return hipGetLastError();
}

// Q4_K on the matrix unit: K a whole number of blocks, rows and activations made of whole 16-byte
// vectors, the codes of every activation row within a block's 64 KiB of LDS.
inline uint32_t tile_tokens(uint32_t m) { return m <= 1 ? 1 : (m <= 4 ? 4 : 8); }
inline bool tiles_serve(const MatVecParams &p, const void *w, const void *x) {
  return p.k >= 1024 && p.k % 256 == 0 && p.m <= 8 && p.row_stride % 16 == 0 &&
         ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0 &&
         tile_shared_bytes(tile_tokens(p.m), p.k / 256) <= 64 * 1024;
}
template <class TX, int kSets>
hipError_t run_tiles_m(const MatVecParams &p, const void *w, const void *x, void *y, int compute_units, hipStream_t s) {
  const uint32_t blocks = p.k / 256, groups = (blocks + 3) / 4;
  const uint32_t tiles = (uint32_t)((p.rows + kTileRows - 1) / kTileRows);
  // few rows: up to four waves share a tile, each walking every second or fourth group of four blocks,
  // until there are eight waves per compute unit
  const uint64_t wanted = 8ull * (uint64_t)(compute_units > 0 ? compute_units : 256);
  uint32_t split_log2 = 0;
  while (split_log2 < 2 && (2u << split_log2) <= groups && ((uint64_t)tiles << split_log2) < wanted) ++split_log2;
  const uint32_t waves = tiles << split_log2;
  const size_t shared = tile_shared_bytes(kSets == 0 ? 1 : 4 * kSets, blocks);
  const dim3 grid((waves + kWavesPerBlock - 1) / kWavesPerBlock);
  const unsigned char *in = static_cast<const unsigned char *>(w);
  // at most 32 activation blocks in all (64 with eight rows): one round of the block's half waves, no loop around it
  if ((kSets == 0 ? 1u : 4u * kSets) * blocks <= (kSets == 2 ? 64u : 32u)) {
    note_variant<TilesTag<kSets, true>>();
    hipLaunchKernelGGL((gguf_matvec_q8_tiles<TX, kSets, true>), grid, dim3(kBlockThreads), shared, s, in, x, y, (uint32_t)p.rows,
                       p.row_stride, blocks, p.m, split_log2);
  } else {
    note_variant<TilesTag<kSets, false>>();
    hipLaunchKernelGGL((gguf_matvec_q8_tiles<TX, kSets, false>), grid, dim3(kBlockThreads), shared, s, in, x, y, (uint32_t)p.rows,
                       p.row_stride, blocks, p.m, split_log2);
  }
  return hipGetLastError();
}
template <class TX>
hipError_t run_tiles(const MatVecParams &p, const void *w, const void *x, void *y, int compute_units, hipStream_t s) {
  if (p.m <= 1) return run_tiles_m<TX, 0>(p, w, x, y, compute_units, s);
  if (p.m <= 4) return run_tiles_m<TX, 1>(p, w, x, y, compute_units, s);
  return run_tiles_m<TX, 2>(p, w, x, y, compute_units, s);
}

template <int kKind, class TX>
hipError_t run_m(const MatVecParams &p, const void *w, const void *x, void *y, int compute_units, hipStream_t s) {
  if constexpr (kKind == 0) {
    // Q4_K: the matrix unit, or block by block
    if (tiles_serve(p, w, x)) return run_tiles<TX>(p, w, x, y, compute_units, s);
    return run_blocks<kKind, TX>(p, w, x, y, compute_units, s);
  } else {
  if constexpr (kKind == 2) {
    // Q8_0, one activation row, a width of 256 n that is no multiple of 2048 (8 blocks are 17 whole
    // vectors): the span kernel with a short last span, up to nine spans
    const uint32_t whole = (p.k + 2047) / 2048;
    if (p.m == 1 && p.k >= 1024 && p.k % 256 == 0 && p.k % 2048 != 0 && whole <= 9 && p.row_stride % 16 == 0 &&
        ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0)
      return run_spans<kKind, TX>(p, w, x, y, whole, (p.k % 2048) / 32, compute_units, s);
  }
  // the span kernels: rows of 2048 n values made of whole 16-byte vectors, activations on a 16-byte
  // boundary, codes of every activation row in LDS beside the waves' row buffers (12 KiB); everything
  // else walks block by block
  if (p.k == 0 || p.k % 2048 != 0 || p.row_stride % 16 != 0 ||
      ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15u) != 0 ||
      gguf_matvec_q8_shared_bytes(p.m, p.k) + 12 * 1024 > 64 * 1024)
    return run_blocks<kKind, TX>(p, w, x, y, compute_units, s);
  const uint32_t spans = p.k / 2048;
  const uint32_t wanted = (uint32_t)((p.rows + kWavesPerBlock - 1) / kWavesPerBlock);
  const uint32_t machine = (uint32_t)(compute_units > 0 ? compute_units : 256) * 3u;  // three blocks per compute unit
  const dim3 grid(wanted < machine ? wanted : machine);
  const size_t shared = gguf_matvec_q8_shared_bytes(p.m, p.k);
  {
    // several activation rows: the quad form, if its four row slots per wave fit beside the codes
    const size_t slots = (size_t)kWavesPerBlock * 4 * (LinesRow<kKind, 1>::kSlotBytes + 32);
    // (a second set of four rows only for Q6_K with its codes in registers, K = 2048)
    const bool sets = p.m <= 4 || (kKind == 1 && spans == 1);
    if (p.m >= 2 && sets && slots + shared <= 64 * 1024) return run_quads<kKind, TX>(p, w, x, y, spans, grid, shared, s);
  }
  if (p.m == 1 && spans <= 6) return run_spans<kKind, TX>(p, w, x, y, spans, kWaveLanes, compute_units, s);
  if (p.m == 1) return run_registers<kKind, TX, 1>(p, w, x, y, spans, grid, shared, s);
  if (p.m == 2) return run_registers<kKind, TX, 2>(p, w, x, y, spans, grid, shared, s);
  if (p.m <= 4) return run_registers<kKind, TX, 4>(p, w, x, y, spans, grid, shared, s);
  return run_registers<kKind, TX, 8>(p, w, x, y, spans, grid, shared, s);
  }
}

template <class TX>
hipError_t run_kind(const MatVecParams &p, const void *w, const void *x, void *y, int compute_units, hipStream_t s) {
  switch (p.kind) {
    case 0: return run_m<0, TX>(p, w, x, y, compute_units, s);
    case 1: return run_m<1, TX>(p, w, x, y, compute_units, s);
    default: return run_m<2, TX>(p, w, x, y, compute_units, s);
  }
}

}  // namespace

size_t gguf_matvec_q8_shared_bytes(uint32_t m, uint32_t k) {
  return (size_t)m * (k / 2048) * kCodeWords * kWaveLanes * sizeof(uint32_t);
}

bool gguf_matvec_q8_serves(int kind, uint32_t k) { return blocks_row_bytes(kind, k) <= kBlocksSharedBudget; }

uint32_t gguf_matvec_q8_dispatches(int kind, uint32_t m, uint32_t k, uint64_t row_stride) {
  if (m == 0 || k == 0) return 1;
  if (kind == 0) {
    if (k >= 1024 && k % 256 == 0 && m <= 8 && row_stride % 16 == 0 && tile_shared_bytes(tile_tokens(m), k / 256) <= 64 * 1024) return 1;
  } else if (k % 2048 == 0 && row_stride % 16 == 0 && gguf_matvec_q8_shared_bytes(m, k) + 12 * 1024 <= 64 * 1024) {
    return 1;
  }
  uint32_t fit = (uint32_t)(kBlocksSharedBudget / blocks_row_bytes(kind, k));
  fit = fit >= 8 ? 8 : (fit >= 4 ? 4 : (fit >= 2 ? 2 : 1));
  return (m + fit - 1) / fit;
}

// K a whole number of blocks with one activation row's codes within LDS (gguf_matvec_q8_serves),
// rows at an even address and stride, M <= 8 (the plan checks all three).
hipError_t launch_gguf_matvec_q8(Elem x_type, const MatVecParams &p, const void *weights, const void *x, void *y,
                                 int compute_units, hipStream_t stream) {
  if (p.rows == 0 || p.m == 0) return hipSuccess;
  switch (x_type) {
    case Elem::kF32: return run_kind<F32>(p, weights, x, y, compute_units, stream);
    case Elem::kF16: return run_kind<F16>(p, weights, x, y, compute_units, stream);
    case Elem::kBF16: return run_kind<BF16>(p, weights, x, y, compute_units, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
