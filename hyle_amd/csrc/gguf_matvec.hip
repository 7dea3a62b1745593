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
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr uint32_t kWavesPerBlock = kBlockThreads / kWaveLanes;

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
  if (p.m == 1)
    hipLaunchKernelGGL((gguf_matvec<kKind, 1, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
  else if (p.m <= 4)
    hipLaunchKernelGGL((gguf_matvec<kKind, 4, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
  else
    hipLaunchKernelGGL((gguf_matvec<kKind, 8, TX>), grid, block, shared, s, in, x, y, (uint32_t)p.rows, p.k,
                       p.row_stride, p.m, rows_per_wave);
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
