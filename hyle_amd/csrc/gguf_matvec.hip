// y[m][n] = sum over k of w[n][k] * x[m][k] for a GGUF weight (Q8_0, Q4_K or Q6_K rows of K
// values, logical [K, N]) and a few activation rows x [M, K], M <= 8: the matrix-vector product
// of token-by-token decoding, where the quantised bytes are read once and never written back as
// bf16.  w is the exact f32 decode (the arithmetic of gguf_decode.h), products and sums are f32.
//
// This is the arithmetic of MatMul(x, W) with the weight's values taken exactly.  ggml, which
// serves this operation in the reference (src/compute_provider_ggml*/), quantises the activation
// row to 8-bit blocks first and multiplies integers; its result differs from the exact product
// by that quantisation and is not reproduced here.
//
// The block first converts x to f32 in LDS.  Each wave then walks its rows (one to eight of
// them, so that tall weights share the x staging among more rows) reading the weight bytes straight from
// global memory, laid out over the lanes so that every byte is read once and neighbouring lanes
// read neighbouring bytes:
//   Q4_K  32 lanes per block: lane i takes the four quant bytes 4 i .. 4 i + 3 (eight values: the
//         low nibbles belong to sub-block 2 c, the high ones to 2 c + 1, c = i / 8);
//   Q6_K  16 lanes per block: lane (h, g) takes four neighbouring bytes of ql[64 h + l],
//         ql[64 h + l + 32] and qh[32 h + l], l = 4 g (sixteen values; single bytes and 64 lanes
//         per block when the row starts at an odd address);
//   Q8_0  8 lanes per block: lane i takes quants 4 i .. 4 i + 3.
// Block headers (scales) are read by every lane that needs them; those loads hit the same
// cache line.  A wave reduction leaves the row's M results.
//
// The shapes decoding spends its bytes on -- a single activation row against rows of 2048 n
// values made of whole 16-byte vectors -- have kernels of their own further down (rows read as
// whole cache lines, x in registers or LDS).  Those factor the scale out of each group of values
// that share it, y = sum of scale * (sum of q x): the same real number as the sum over exactly
// decoded weights, with different f32 roundings; every form is held to 1e-5 * sum |w x| of the
// exact product.
#include "device_common.h"
#include "gguf_decode.h"
#include "gguf_lines.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

__device__ __forceinline__ float f16_at(const unsigned char *p) {
  return f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}
// Four bytes from an address that is 4-byte aligned when `aligned`, else byte by byte.
__device__ __forceinline__ uint32_t word_at(const unsigned char *p, bool aligned) {
  if (aligned) return __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p));
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

template <int kM> struct Acc {
  float v[kM];
};

// acc[r] += sum_j w[j] * x[r][at + j * stride]
template <int kM, int kCount>
__device__ __forceinline__ void fold(Acc<kM> &acc, const float (&w)[kCount], const float *xs, uint32_t k, uint32_t m,
                                     uint32_t at, uint32_t stride) {
#pragma unroll
  for (int r = 0; r < kM; ++r) {
    if ((uint32_t)r < m) {
      const float *xr = xs + (size_t)r * k + at;
#pragma unroll
      for (int j = 0; j < kCount; ++j) acc.v[r] += w[j] * xr[j * stride];
    }
  }
}

template <int kM>
__device__ __forceinline__ void row_q4_k(const unsigned char *row, uint32_t k, bool aligned, const float *xs,
                                         uint32_t m, uint32_t lane, Acc<kM> &acc) {
  const uint32_t blocks = k / 256, i = lane % 32, chunk = i / 8;
#pragma unroll 4
  for (uint32_t b = lane / 32; b < blocks; b += 2) {
    const unsigned char *blk = row + (size_t)b * 144;
    // the 16 header bytes {f16 d, f16 dmin, scales[12]} as four words, the lane's quants as one
    const uint32_t head[4] = {word_at(blk, aligned), word_at(blk + 4, aligned), word_at(blk + 8, aligned),
                              word_at(blk + 12, aligned)};
    const uint32_t q = word_at(blk + 16 + 4 * i, aligned);
    const float d = f16_to_f32((uint16_t)head[0]), dmin = f16_to_f32((uint16_t)(head[0] >> 16));
    auto scale_byte = [&](uint32_t index) {  // scales[index], index 0..11
      return (head[1 + index / 4] >> (8 * (index % 4))) & 0xFFu;
    };
    float w[4];
#pragma unroll
    for (int high = 0; high < 2; ++high) {
      const uint32_t sub = 2 * chunk + high;
      uint32_t sc, mn;
      if (sub < 4) {
        sc = scale_byte(sub) & 63u;
        mn = scale_byte(sub + 4) & 63u;
      } else {
        sc = (scale_byte(sub + 4) & 0xFu) | ((scale_byte(sub - 4) >> 6) << 4);
        mn = (scale_byte(sub + 4) >> 4) | ((scale_byte(sub) >> 6) << 4);
      }
      const float step = d * (float)sc, offset = dmin * (float)mn;
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = step * (float)((q >> (8 * j + 4 * high)) & 0xFu) - offset;
      fold<kM, 4>(acc, w, xs, k, m, b * 256 + 32 * sub + (i % 8) * 4, 1);
    }
  }
}

template <int kM>
__device__ __forceinline__ void row_q6_k(const unsigned char *row, uint32_t k, const float *xs, uint32_t m,
                                         uint32_t lane, Acc<kM> &acc) {
  const uint32_t blocks = k / 256, half = lane / 32, l = lane % 32;
#pragma unroll 4
  for (uint32_t b = 0; b < blocks; ++b) {
    const unsigned char *blk = row + (size_t)b * 210;
    const uint32_t low = blk[64 * half + l], high = blk[64 * half + l + 32], top = blk[128 + 32 * half + l];
    const signed char *sc = reinterpret_cast<const signed char *>(blk + 192 + 8 * half + l / 16);
    const float d = f16_at(blk + 208);
    float w[4];
    w[0] = d * (float)sc[0] * (float)((int)((low & 0xFu) | ((top & 3u) << 4)) - 32);
    w[1] = d * (float)sc[2] * (float)((int)((high & 0xFu) | (((top >> 2) & 3u) << 4)) - 32);
    w[2] = d * (float)sc[4] * (float)((int)((low >> 4) | (((top >> 4) & 3u) << 4)) - 32);
    w[3] = d * (float)sc[6] * (float)((int)((high >> 4) | (((top >> 6) & 3u) << 4)) - 32);
    fold<kM, 4>(acc, w, xs, k, m, b * 256 + 128 * half + l, 32);
  }
}

// Q6_K with 2-byte loads (blocks of a row that starts at an even address are 2-byte aligned):
// 16 lanes per block, lane (h, g) takes l = 4 g .. 4 g + 3 of half h: two bytes at a time of
// ql[64 h + l], ql[64 h + l + 32] and qh[32 h + l], sixteen values in all.
__device__ __forceinline__ uint32_t pair_at(const unsigned char *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(p));
}
template <int kM>
__device__ __forceinline__ void row_q6_k_pairs(const unsigned char *row, uint32_t k, const float *xs, uint32_t m,
                                               uint32_t lane, Acc<kM> &acc) {
  const uint32_t blocks = k / 256, within = lane % 16, half = within / 8, l = (within % 8) * 4;
#pragma unroll 2
  for (uint32_t b = lane / 16; b < blocks; b += 4) {
    const unsigned char *blk = row + (size_t)b * 210;
    const unsigned char *ql = blk + 64 * half + l, *qh = blk + 128 + 32 * half + l;
    const uint32_t low = pair_at(ql) | (pair_at(ql + 2) << 16);
    const uint32_t high = pair_at(ql + 32) | (pair_at(ql + 34) << 16);
    const uint32_t top = pair_at(qh) | (pair_at(qh + 2) << 16);
    const signed char *sc = reinterpret_cast<const signed char *>(blk + 192 + 8 * half + l / 16);
    const float d = f16_to_f32((uint16_t)pair_at(blk + 208));
    const float step[4] = {d * (float)sc[0], d * (float)sc[2], d * (float)sc[4], d * (float)sc[6]};
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // position l + j of each of the four groups
      const uint32_t lo = (low >> (8 * j)) & 0xFFu, hi = (high >> (8 * j)) & 0xFFu, tp = (top >> (8 * j)) & 0xFFu;
      float w[4];
      w[0] = step[0] * (float)((int)((lo & 0xFu) | ((tp & 3u) << 4)) - 32);
      w[1] = step[1] * (float)((int)((hi & 0xFu) | (((tp >> 2) & 3u) << 4)) - 32);
      w[2] = step[2] * (float)((int)((lo >> 4) | (((tp >> 4) & 3u) << 4)) - 32);
      w[3] = step[3] * (float)((int)((hi >> 4) | (((tp >> 6) & 3u) << 4)) - 32);
      fold<kM, 4>(acc, w, xs, k, m, b * 256 + 128 * half + l + j, 32);
    }
  }
}

template <int kM>
__device__ __forceinline__ void row_q8_0(const unsigned char *row, uint32_t k, const float *xs, uint32_t m,
                                         uint32_t lane, Acc<kM> &acc) {
  const uint32_t blocks = k / 32, part = (lane % 8) * 4;
#pragma unroll 4
  for (uint32_t b = lane / 8; b < blocks; b += 8) {
    const unsigned char *blk = row + (size_t)b * 34;
    const float d = f16_at(blk);
    float w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = (float)(signed char)blk[2 + part + j] * d;
    fold<kM, 4>(acc, w, xs, k, m, b * 32 + part, 1);
  }
}

// ---------------------------------------------------------------------------------
// One activation row against Q4_K, Q6_K or Q8_0 rows of 2048 values made of whole 16-byte
// vectors (longer rows: the variant further down): the projections of a decoded token.
//
// Every cache line is requested once: the wave reads a row as whole 16-byte vectors (lane i
// takes vectors i, i + 64, ...: 2048 values are 72, 105 or 136 vectors), keeps the four rows still in
// flight in registers, and hands the bytes to the lanes that decode them through a region of
// LDS that only this wave touches.  (Reading each lane's pieces straight from memory asks for
// every line several times while it is still on its way; the address unit and those waits then
// set the time: 89 us for Q6_K [2048 -> 151936] against 54 us.)  LDS executes one wave's
// instructions in order, so the stores of a row and the loads that follow need no barrier, and
// the next row is stored only after this row's loads were issued.  LDS is read as naturally
// aligned words (an unaligned read stalls).  The grid is sized to the machine, not to the
// weight: wave w of W takes rows w, w + W, ...
//
// A lane decodes the same 32 positions of every 2048 values of every row, so its activations
// stay in registers.  Values that share a scale are summed against x first and scaled once:
//   Q6_K  y = sum over groups of (d * scale) * sum (q - 32) x
//   Q4_K  y = sum over sub-blocks of (d * sc) * sum q x - (dmin * m) * sum x
//   Q8_0  y = sum over blocks of d * sum q x
// with f32 products and sums (the sums of x are per lane and computed once).  About 135 vector
// instructions per row and lane remain for Q6_K, which on 256 compute units is about 40 us for
// 151,936 rows: the kernels are bound by that arithmetic.
template <int kKind, class TX, int kPasses>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_lines(const unsigned char *weights, const void *x, void *y,
                                                                   uint32_t rows, uint64_t row_stride) {
  using Row = LinesRow<kKind, kPasses>;
  using Kind = Lines<kKind>;
  __shared__ __align__(16) unsigned char slots[kWavesPerBlock][Row::kSlotBytes];
  const uint32_t lane = threadIdx.x % kWaveLanes;
  // the wave's number as a scalar, so that row addresses are scalar too
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  unsigned char *slot = slots[wave];
  float xs[kPasses][32], xsum[kPasses][4];
  typename Kind::Lane at[kPasses];
#pragma unroll
  for (int pass = 0; pass < kPasses; ++pass) {
    at[pass] = Kind::lane_of(pass, lane);
#pragma unroll
    for (int e = 0; e < 32; ++e) xs[pass][e] = Traits<TX>::load(x, Kind::position(pass, lane, e));
#pragma unroll
    for (int part = 0; part < 4; ++part) {
      xsum[pass][part] = 0.0f;
#pragma unroll
      for (int t = 0; t < 8; ++t) xsum[pass][part] += xs[pass][8 * part + t];
    }
  }
  const uint32_t stride = gridDim.x * kWavesPerBlock;
  const uint32_t first = blockIdx.x * kWavesPerBlock + wave;
  if (first >= rows) return;
  // A row past the end is replaced by the wave's first row: a valid address whose bytes go
  // unused (loads inside a branch wait for each other: measured, 7.5 against 6.7 us for 6144 rows).
  Row ring[kLinesDepth];
#pragma unroll
  for (int d = 0; d < kLinesDepth; ++d) {
    const uint64_t wanted = (uint64_t)first + (uint64_t)d * stride;
    const uint32_t row = wanted < rows ? (uint32_t)wanted : first;
    ring[d] = Row::load(weights + (size_t)row * row_stride, lane);
  }
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
      const uint32_t following = wanted < rows ? (uint32_t)wanted : first;
      ring[d] = Row::load(weights + (size_t)following * row_stride, lane);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int pass = 0; pass < kPasses; ++pass) totals[d] += Kind::dot(slot, at[pass], xs[pass], xsum[pass]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    // The four rows are summed over the wave together: two exchanges leave lane l with the sum
    // of row l % 4 over its group of four lanes, four more add the sixteen groups.
    static_assert(kLinesDepth == 4, "the joint reduction is written for four rows");
    const bool odd = (lane & 1u) != 0, upper = (lane & 2u) != 0;
    const float pair01 = (odd ? totals[1] : totals[0]) + __shfl_xor(odd ? totals[0] : totals[1], 1);
    const float pair23 = (odd ? totals[3] : totals[2]) + __shfl_xor(odd ? totals[2] : totals[3], 1);
    float mine = (upper ? pair23 : pair01) + __shfl_xor(upper ? pair01 : pair23, 2);
#pragma unroll
    for (int step = 4; step < kWaveLanes; step *= 2) mine += __shfl_xor(mine, step);
    const uint64_t row = base + (uint64_t)lane * stride;
    if (lane < (uint32_t)kLinesDepth && row < rows) Traits<TX>::store(y, (size_t)row, mine);
  }
}

// One activation row against rows of kSpans spans of 2048 values, a wave of the block per span:
// the wave keeps its span of x in registers as the kernel above does (no staging of x through
// LDS, so a block starts on its rows at once, which is most of the time when a wave has only a
// row or two to walk: Q4_K [6144 -> 2048] has 2048 rows for 1024 compute-unit SIMDs), walks the
// block's rows span by span and leaves its share of each row in LDS, where the first wave adds
// the spans' shares in span order.
template <int kKind, class TX, int kSpans>
__global__ __launch_bounds__(kSpans * kWaveLanes) void gguf_matvec_spans(const unsigned char *weights, const void *x, void *y,
                                                                       uint32_t rows, uint64_t row_stride) {
  using Row = LinesRow<kKind, 1>;
  using Kind = Lines<kKind>;
  constexpr uint32_t kSpanBytes = Kind::kPassVectors * 16;
  __shared__ __align__(16) unsigned char slots[kSpans][Row::kSlotBytes];
  __shared__ float shares[kSpans][kLinesDepth];
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t span = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  unsigned char *slot = slots[span];
  float xs[32], xsum[4];
  const typename Kind::Lane at = Kind::lane_of(0, lane);
#pragma unroll
  for (int e = 0; e < 32; ++e) xs[e] = Traits<TX>::load(x, Kind::position(span, lane, e));
#pragma unroll
  for (int part = 0; part < 4; ++part) {
    xsum[part] = 0.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) xsum[part] += xs[8 * part + t];
  }
  const uint32_t stride = gridDim.x, first = blockIdx.x;  // first < rows: the grid has at most `rows` blocks
  const unsigned char *mine = weights + (size_t)span * kSpanBytes;
  Row ring[kLinesDepth];
#pragma unroll
  for (int d = 0; d < kLinesDepth; ++d) {
    const uint64_t wanted = (uint64_t)first + (uint64_t)d * stride;
    ring[d] = Row::load(mine + (size_t)(wanted < rows ? (uint32_t)wanted : first) * row_stride, lane);
  }
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
      ring[d] = Row::load(mine + (size_t)(wanted < rows ? (uint32_t)wanted : first) * row_stride, lane);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      totals[d] = Kind::dot(slot, at, xs, xsum);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    // as above: lane l < 4 ends with row l's sum over the wave
    static_assert(kLinesDepth == 4, "the joint reduction is written for four rows");
    const bool odd = (lane & 1u) != 0, upper = (lane & 2u) != 0;
    const float pair01 = (odd ? totals[1] : totals[0]) + __shfl_xor(odd ? totals[0] : totals[1], 1);
    const float pair23 = (odd ? totals[3] : totals[2]) + __shfl_xor(odd ? totals[2] : totals[3], 1);
    float share = (upper ? pair23 : pair01) + __shfl_xor(upper ? pair01 : pair23, 2);
#pragma unroll
    for (int step = 4; step < kWaveLanes; step *= 2) share += __shfl_xor(share, step);
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

// Two to eight activation rows (any K = 2048 n whose activations fit) and one row longer than six
// spans: the same walk over spans of 2048 values, with the
// activations as f32 in LDS instead of registers.  They are laid out [span][e / 4][lane][e % 4], so
// that a lane fetches its 32 values of a span with eight 16-byte reads that are contiguous across
// the wave; Q4_K's per-lane sums of x sit beside them.  A wave walks the spans of its rows one
// after another, four spans in flight, and closes a row with a wave reduction.
template <int kKind, class TX, int kM>
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec_lines_long(const unsigned char *weights, const void *x,
                                                                        void *y, uint32_t rows, uint64_t row_stride,
                                                                        uint32_t spans, uint32_t m) {
  using Row = LinesRow<kKind, 1>;
  using Kind = Lines<kKind>;
  constexpr uint32_t kSpanBytes = Kind::kPassVectors * 16;
  __shared__ __align__(16) unsigned char slots[kWavesPerBlock][Row::kSlotBytes];
  // x: m rows of spans * 2048 floats (an activation row after the other), then their sums: m * spans * 256
  extern __shared__ __align__(16) float staged[];
  const uint32_t k = spans * 2048;
  float *sums = staged + (size_t)m * k;
  for (uint32_t r = 0; r < m; ++r) {
    for (uint32_t i = threadIdx.x; i < k; i += kBlockThreads) {
      const uint32_t span = i / 2048, quad = (i % 2048) / 256, lane = (i / 4) % kWaveLanes, e = 4 * quad + i % 4;
      staged[(size_t)r * k + i] = Traits<TX>::load(x, (size_t)r * k + Kind::position(span, lane, e));
    }
  }
  __syncthreads();
  if constexpr (kKind == 0) {
    for (uint32_t i = threadIdx.x; i < m * spans * 256; i += kBlockThreads) {
      const uint32_t group = i / 256, lane = (i / 4) % kWaveLanes, part = i % 4;  // group = r * spans + span
      float sum = 0.0f;
      for (uint32_t t = 0; t < 8; ++t) {
        const uint32_t e = 8 * part + t;
        sum += staged[((group * 8 + e / 4) * kWaveLanes + lane) * 4 + e % 4];
      }
      sums[i] = sum;
    }
    __syncthreads();
  }
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
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
      // One call per activation row: the span's bytes are decoded by the same expressions each
      // time, which the compiler works out once and multiplies against every row of x.
#pragma unroll
      // (No branch around a call, or the sharing is lost: a row of x past the last one is
      // the last one again, worked on and never stored.)
      for (int r = 0; r < kM; ++r) {
        const uint32_t group = ((uint32_t)r < m ? (uint32_t)r : m - 1) * spans + span;
        float xs[32], xsum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int quad = 0; quad < 8; ++quad) {
          const float4 v = *reinterpret_cast<const float4 *>(staged + ((size_t)(group * 8 + quad) * kWaveLanes + lane) * 4);
          xs[4 * quad] = v.x, xs[4 * quad + 1] = v.y, xs[4 * quad + 2] = v.z, xs[4 * quad + 3] = v.w;
        }
        if constexpr (kKind == 0) {
          const float4 v = *reinterpret_cast<const float4 *>(sums + ((size_t)group * kWaveLanes + lane) * 4);
          xsum[0] = v.x, xsum[1] = v.y, xsum[2] = v.z, xsum[3] = v.w;
        }
        totals[r] += Kind::dot(slot, at, xs, xsum);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (++span == spans) {
#pragma unroll
        for (int r = 0; r < kM; ++r) {
          const float whole = group_sum<kWaveLanes>(totals[r]);
          if (lane == 0 && (uint32_t)r < m) Traits<TX>::store(y, (size_t)r * rows + row, whole);
          totals[r] = 0.0f;
        }
        span = 0;
        row += stride;
      }
    }
  }
}

template <int kKind, int kM, class TX>  // 0 = Q4_K, 1 = Q6_K, 2 = Q8_0
__global__ __launch_bounds__(kBlockThreads) void gguf_matvec(const unsigned char *weights, const void *x, void *y,
                                                             uint32_t rows, uint32_t k, uint64_t row_stride,
                                                             uint32_t m, uint32_t rows_per_wave) {
  extern __shared__ __align__(16) unsigned char shared[];
  float *xs = reinterpret_cast<float *>(shared);  // [m][k]
  for (uint32_t i = threadIdx.x; i < m * k; i += kBlockThreads) xs[i] = Traits<TX>::load(x, i);
  __syncthreads();
  const uint32_t lane = threadIdx.x % kWaveLanes, wave = threadIdx.x / kWaveLanes;
  const bool aligned = ((reinterpret_cast<uintptr_t>(weights) | row_stride) & 3u) == 0;
  const bool even = ((reinterpret_cast<uintptr_t>(weights) | row_stride) & 1u) == 0;
  for (uint32_t turn = 0; turn < rows_per_wave; ++turn) {
    const uint32_t row = (blockIdx.x * rows_per_wave + turn) * kWavesPerBlock + wave;
    if (row >= rows) break;
    const unsigned char *source = weights + (size_t)row * row_stride;
    Acc<kM> acc;
#pragma unroll
    for (int r = 0; r < kM; ++r) acc.v[r] = 0.0f;
    if constexpr (kKind == 0) row_q4_k<kM>(source, k, aligned, xs, m, lane, acc);
    else if constexpr (kKind == 1) {
      if (even) row_q6_k_pairs<kM>(source, k, xs, m, lane, acc);
      else row_q6_k<kM>(source, k, xs, m, lane, acc);
    }
    else row_q8_0<kM>(source, k, xs, m, lane, acc);
#pragma unroll
    for (int r = 0; r < kM; ++r) {
      const float total = group_sum<kWaveLanes>(acc.v[r]);
      if (lane == 0 && (uint32_t)r < m) Traits<TX>::store(y, (size_t)r * rows + row, total);
    }
  }
}

// Launch-shape labels: gguf_matvec_<form>/<format>/<detail>
inline const char *matvec_kind_word(int kind) { return kind == 0 ? "q4_k" : (kind == 1 ? "q6_k" : "q8_0"); }
template <int kKind> struct ExactLinesTag {
  static std::string text() { return std::string("gguf_matvec_lines/") + matvec_kind_word(kKind); }
};
template <int kKind, int kSpans> struct ExactSpansTag {
  static std::string text() { return std::string("gguf_matvec_spans/") + matvec_kind_word(kKind) + "/" + std::to_string(kSpans) + "-spans"; }
};
template <int kKind, int kM> struct ExactLongTag {
  static std::string text() { return std::string("gguf_matvec_lines_long/") + matvec_kind_word(kKind) + "/" + std::to_string(kM) + "-tokens"; }
};
template <int kKind, int kM> struct ExactGeneralTag {
  static std::string text() { return std::string("gguf_matvec_general/") + matvec_kind_word(kKind) + "/" + std::to_string(kM) + "-tokens"; }
};

template <int kKind, class TX>
hipError_t run_m(const MatVecParams &p, const void *w, const void *x, void *y, hipStream_t s) {
  // Rows per wave: one when there are few rows (every wave in flight at once), up to eight for
  // tall weights, so that the conversion of x into LDS is shared by more rows.
  uint32_t rows_per_wave = (uint32_t)(p.rows / (kWavesPerBlock * 4096));
  rows_per_wave = rows_per_wave < 1 ? 1 : (rows_per_wave > 8 ? 8 : rows_per_wave);
  const uint32_t rows_per_block = kWavesPerBlock * rows_per_wave;
  const dim3 grid(((uint32_t)p.rows + rows_per_block - 1) / rows_per_block), block(kBlockThreads);
  const size_t shared = (size_t)p.m * p.k * sizeof(float);
  const unsigned char *in = static_cast<const unsigned char *>(w);
  const uint32_t units = p.compute_units;
  {
    // one activation row over rows of 2048 n values made of whole 16-byte vectors
    const bool lines = ((reinterpret_cast<uintptr_t>(w) | p.row_stride) & 15u) == 0;
    if (p.m == 1 && lines && p.k == 2048) {
      const uint32_t wanted = (uint32_t)((p.rows + kWavesPerBlock - 1) / kWavesPerBlock);
      // three blocks per compute unit measured best (Q4_K [2048 -> 6144] 4.9 us and [2048 -> 151936]
      // 45.9 us, against 6.4 and 47.7 us with five; counts that are not a multiple of the
      // compute units leave some of them a block short and are slower)
      const dim3 machine(wanted < units * 3u ? wanted : units * 3u);
      note_variant<ExactLinesTag<kKind>>();
      hipLaunchKernelGGL((gguf_matvec_lines<kKind, TX, 1>), machine, block, 0, s, in, x, y, (uint32_t)p.rows,
                         p.row_stride);
      return hipGetLastError();
    }
    // several activation rows, or more spans: x in LDS, as long as it fits in a block's 64 KiB
    // beside the waves' row buffers
    const size_t staged = (size_t)p.m * (p.k / 2048) * (2048 + (kKind == 0 ? 256 : 0)) * sizeof(float);
    const size_t parked = (size_t)kWavesPerBlock * LinesRow<kKind, 1>::kSlotBytes;
    // one activation row, two to six spans: a wave per span, twelve waves per compute unit
    // (Q4_K [6144 -> 2048]: 4.8 us with 4 blocks of three waves per unit, 4.9 / 5.4 / 6.6 / 7.3 us
    // with 3 / 2 / 6 / 8; [4096 -> 14336]: 11.7 us with 6 blocks of two waves, 13.4 / 13.7 us with
    // 4 / 8; with the activations staged in LDS as below: 8.1 and 14.3 us, and 24 against 15 us
    // for [12288 -> 4096])
    if (p.m == 1 && lines && p.k % 2048 == 0 && p.k >= 4096 && p.k <= 12288) {
      const uint32_t spans = p.k / 2048;
      const uint32_t most = units * (12u / spans);
      const dim3 machine((uint32_t)p.rows < most ? (uint32_t)p.rows : most);
      const uint32_t rows = (uint32_t)p.rows;
      switch (spans) {
        case 2: note_variant<ExactSpansTag<kKind, 2>>(); hipLaunchKernelGGL((gguf_matvec_spans<kKind, TX, 2>), machine, dim3(2 * kWaveLanes), 0, s, in, x, y, rows, p.row_stride); break;
        case 3: note_variant<ExactSpansTag<kKind, 3>>(); hipLaunchKernelGGL((gguf_matvec_spans<kKind, TX, 3>), machine, dim3(3 * kWaveLanes), 0, s, in, x, y, rows, p.row_stride); break;
        case 4: note_variant<ExactSpansTag<kKind, 4>>(); hipLaunchKernelGGL((gguf_matvec_spans<kKind, TX, 4>), machine, dim3(4 * kWaveLanes), 0, s, in, x, y, rows, p.row_stride); break;
        case 5: note_variant<ExactSpansTag<kKind, 5>>(); hipLaunchKernelGGL((gguf_matvec_spans<kKind, TX, 5>), machine, dim3(5 * kWaveLanes), 0, s, in, x, y, rows, p.row_stride); break;
        default: note_variant<ExactSpansTag<kKind, 6>>(); hipLaunchKernelGGL((gguf_matvec_spans<kKind, TX, 6>), machine, dim3(6 * kWaveLanes), 0, s, in, x, y, rows, p.row_stride); break;
      }
      return hipGetLastError();
    }
    if (lines && p.k % 2048 == 0 && (p.k > 2048 || p.m > 1) && staged + parked <= 64 * 1024) {
      const uint32_t spans = p.k / 2048;
      const uint32_t wanted = (uint32_t)((p.rows + kWavesPerBlock - 1) / kWavesPerBlock);
      const dim3 machine(wanted < units * 3u ? wanted : units * 3u);
      if (p.m == 1) {
        // one activation row arrives here with seven spans or more: only Q6_K's then fit beside its row buffers
        if constexpr (kKind == 1) {
          note_variant<ExactLongTag<kKind, 1>>();
          hipLaunchKernelGGL((gguf_matvec_lines_long<kKind, TX, 1>), machine, block, staged, s, in, x, y,
                             (uint32_t)p.rows, p.row_stride, spans, p.m);
        } else {
          return hipErrorInvalidValue;
        }
      }
      else if (p.m == 2) {
        note_variant<ExactLongTag<kKind, 2>>();
        hipLaunchKernelGGL((gguf_matvec_lines_long<kKind, TX, 2>), machine, block, staged, s, in, x, y,
                           (uint32_t)p.rows, p.row_stride, spans, p.m);
      }
      else if (p.m <= 4) {
        note_variant<ExactLongTag<kKind, 4>>();
        hipLaunchKernelGGL((gguf_matvec_lines_long<kKind, TX, 4>), machine, block, staged, s, in, x, y,
                           (uint32_t)p.rows, p.row_stride, spans, p.m);
      }
      else {
        note_variant<ExactLongTag<kKind, 8>>();
        hipLaunchKernelGGL((gguf_matvec_lines_long<kKind, TX, 8>), machine, block, staged, s, in, x, y,
                           (uint32_t)p.rows, p.row_stride, spans, p.m);
      }
      return hipGetLastError();
    }
  }
  if (p.m == 1) {
    note_variant<ExactGeneralTag<kKind, 1>>();
    hipLaunchKernelGGL((gguf_matvec<kKind, 1, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
  }
  else if (p.m <= 4) {
    note_variant<ExactGeneralTag<kKind, 4>>();
    hipLaunchKernelGGL((gguf_matvec<kKind, 4, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
  }
  else {
    note_variant<ExactGeneralTag<kKind, 8>>();
    hipLaunchKernelGGL((gguf_matvec<kKind, 8, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
  }
  return hipGetLastError();
}

template <class TX>
hipError_t run_kind(const MatVecParams &p, const void *w, const void *x, void *y, hipStream_t s) {
  switch (p.kind) {
    case 0: return run_m<0, TX>(p, w, x, y, s);
    case 1: return run_m<1, TX>(p, w, x, y, s);
    default: return run_m<2, TX>(p, w, x, y, s);
  }
}

}  // namespace

size_t gguf_matvec_shared_bytes(uint32_t m, uint32_t k) {
  return (size_t)m * k * sizeof(float);
}

hipError_t launch_gguf_matvec(Elem x_type, const MatVecParams &p, const void *weights, const void *x, void *y,
                              hipStream_t stream) {
  if (p.rows == 0 || p.m == 0) return hipSuccess;
  switch (x_type) {
    case Elem::kF32: return run_kind<F32>(p, weights, x, y, stream);
    case Elem::kF16: return run_kind<F16>(p, weights, x, y, stream);
    case Elem::kBF16: return run_kind<BF16>(p, weights, x, y, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
