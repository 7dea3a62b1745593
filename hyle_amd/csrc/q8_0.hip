// q8_0.hip -- Q8_0 block dequant to bf16 fused with the per-row sum of squares,
// for gfx950.
//
// Block layout (src/compute_ops/low_precision.cc:28-29 of the reference; ggml
// block_q8_0): 34 bytes = little-endian fp16 scale d followed by 32 int8 quants.
// A weight [K, N] is stored as N physical rows of K/32 blocks
// (src/compute_ops/low_precision.cc:269-297).  Decode is y = (float)q * (float)d:
// an 8-bit by 11-bit significand product, exact in f32, so the bf16 store is one
// RN-even rounding and the result is bit-identical on every implementation.
//
// Blocks are only 2-byte aligned, so a wave parks its row in LDS with 16-byte global loads
// (every cache line requested once) and re-slices it there; output leaves as 16-byte bf16x8
// stores, 1 KiB of consecutive bf16 per store instruction of a wave.  Each row's sum of squares
// of the exact products is reduced with a wave64 butterfly.
//
// Three kernels: rows of K = 2048 n values made of whole 16-byte vectors take one wave per row
// with a region of LDS that only this wave touches and no block barrier (q8_0_lines: aligned
// 32-bit LDS words joined by byte-wise funnel shifts); other rows of whole vectors stage
// block-wide with 2-byte LDS reads (q8_0_rows); anything else reads bytes (q8_0_rows_bytes).
#include "device_common.h"
#include "gguf_decode.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr int kBlockBytes = 34;
constexpr int kBlockElems = 32;

// Requires row_bytes % 16 == 0, row_stride % 16 == 0 and a 16-byte aligned base.
constexpr int kMaxRowBytes = 8704;  // 256 blocks = 8192 elements

// Each wave owns `kRows` consecutive rows: all their global loads are issued first.
template <int kWaves, int kRows>
__global__ __launch_bounds__(kWaves *kWaveLanes) void q8_0_rows(const char *blocks, uint16_t *out,
                                                               float *sumsq, uint32_t rows,
                                                               uint32_t k, uint64_t row_stride,
                                                               uint32_t row_bytes) {
  extern __shared__ __attribute__((aligned(16))) char staged[];
  const uint32_t wave = threadIdx.x / kWaveLanes, lane = threadIdx.x % kWaveLanes;
  const uint32_t first_row = (blockIdx.x * kWaves + wave) * kRows;
  char *mine = staged + (size_t)wave * kRows * row_bytes;
  const uint32_t row_vectors = row_bytes / 16;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const uint32_t row = first_row + r;
    if (row < rows) {
      const char *src = blocks + (size_t)row * row_stride;
      for (uint32_t v = lane; v < row_vectors; v += kWaveLanes)
        reinterpret_cast<u32x4 *>(mine + (size_t)r * row_bytes)[v] = load16_stream(src, v);
    }
  }
  __syncthreads();
  const uint32_t out_vectors = k / 8;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const uint32_t row = first_row + r;
    float squares = 0.0f;
    if (row < rows) {
      const char *staged_row = mine + (size_t)r * row_bytes;
      // output vector j holds elements [8j, 8j+8): block j/4, quants 8*(j%4) ..
      for (uint32_t j = lane; j < out_vectors; j += kWaveLanes) {
        const char *block = staged_row + (size_t)(j / 4) * kBlockBytes;
        const float d = f16_to_f32(*reinterpret_cast<const uint16_t *>(block));
        const uint16_t *q = reinterpret_cast<const uint16_t *>(block + 2 + 8 * (j % 4));
        float y[8];
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          const uint32_t pair = q[h];
          y[2 * h] = (float)(int8_t)(pair & 0xFFu) * d;
          y[2 * h + 1] = (float)(int8_t)(pair >> 8) * d;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) squares = __builtin_fmaf(y[e], y[e], squares);
        store16_stream(out, (size_t)row * out_vectors + j, Traits<BF16>::pack(y));
      }
    }
    squares = group_sum<kWaveLanes>(squares);
    if (row < rows && lane == 0) sumsq[row] = squares;
  }
}

// Rows of K = 2048 n values, whole 16-byte vectors, 16-byte aligned: one wave per row, no barrier.
// A span of 2048 values is 64 blocks = 2176 bytes = 136 vectors: two per lane and a third for
// the first eight lanes (the others repeat the span's last vector, one request for all of them);
// plain loads: the non-temporal hint costs 10 % here, while the stores keep it.
// The vectors are parked in LDS that only this wave touches (LDS executes one wave's
// instructions in order); lane l then decodes output vectors l, l + 64, l + 128, l + 192 of
// the span: eight quants at a 2-byte aligned offset come out of three aligned words and two
// funnel shifts, the block's scale out of one 16-bit read.  The next span's loads are in flight
// while this one is decoded.
template <int kWaves>
__global__ __launch_bounds__(kWaves *kWaveLanes) void q8_0_lines(const unsigned char *blocks, void *out,
                                                                float *sumsq, uint32_t rows, uint32_t k,
                                                                uint64_t row_stride) {
  constexpr uint32_t kSpan = 2048;
  constexpr uint32_t kVectors = kSpan / kBlockElems * kBlockBytes / 16;  // 136
  constexpr int kLoads = (kVectors + kWaveLanes - 1) / kWaveLanes;       // 3
  __shared__ __align__(16) unsigned char slots[kWaves][kLoads * kWaveLanes * 16];
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
  const uint32_t row = blockIdx.x * kWaves + wave;
  if (row >= rows) return;
  unsigned char *slot = slots[wave];
  const unsigned char *source = blocks + (size_t)row * row_stride;
  const uint32_t steps = k / kSpan;
  uint32_t vec[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const uint32_t wanted = lane + i * kWaveLanes;
    vec[i] = wanted < kVectors ? wanted : kVectors - 1;
  }
  u32x4 raw[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) raw[i] = load16(source, vec[i]);
  float squares = 0.0f;
  for (uint32_t step = 0; step < steps; ++step) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) *reinterpret_cast<u32x4 *>(slot + (size_t)(lane + i * kWaveLanes) * 16) = raw[i];
    if (step + 1 < steps) {  // uniform across the wave
#pragma unroll
      for (int i = 0; i < kLoads; ++i) raw[i] = load16(source, (size_t)(step + 1) * kVectors + vec[i]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (uint32_t i = 0; i < kSpan / (kWaveLanes * 8); ++i) {
      const uint32_t j = i * kWaveLanes + lane;  // output vector of the span: block j / 4, quants 8 (j % 4) ..
      const uint32_t block_offset = (j / 4) * kBlockBytes;
      const float d = f16_to_f32(*reinterpret_cast<const uint16_t *>(slot + block_offset));
      uint32_t q[2];
      lds_piece(slot, block_offset + 2 + 8 * (j % 4), q);
      float y[8];
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int t = 0; t < 4; ++t) y[4 * w + t] = (float)(int)(signed char)(q[w] >> (8 * t)) * d;
#pragma unroll
      for (int e = 0; e < 8; ++e) squares = __builtin_fmaf(y[e], y[e], squares);
      store16_stream(out, ((size_t)row * k + (size_t)step * kSpan) / 8 + j, Traits<BF16>::pack(y));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  squares = group_sum<kWaveLanes>(squares);
  if (lane == 0) sumsq[row] = squares;
}

// Any k (multiple of 32), any stride or alignment: one wave per row, byte loads.
__global__ __launch_bounds__(kBlockThreads) void q8_0_rows_bytes(const uint8_t *blocks, uint16_t *out,
                                                                 float *sumsq, uint32_t rows,
                                                                 uint32_t k, uint64_t row_stride) {
  const uint32_t wave = threadIdx.x / kWaveLanes, lane = threadIdx.x % kWaveLanes;
  const uint32_t row = blockIdx.x * (kBlockThreads / kWaveLanes) + wave;
  const bool row_ok = row < rows;
  float squares = 0.0f;
  if (row_ok) {
    const uint8_t *src = blocks + (size_t)row * row_stride;
    for (uint32_t e = lane; e < k; e += kWaveLanes) {
      const uint8_t *block = src + (size_t)(e / kBlockElems) * kBlockBytes;
      const float d = f16_to_f32((uint16_t)(block[0] | ((uint16_t)block[1] << 8)));
      const float y = (float)(int8_t)block[2 + e % kBlockElems] * d;
      squares = __builtin_fmaf(y, y, squares);
      out[(size_t)row * k + e] = f32_to_bf16(y);
    }
  }
  squares = group_sum<kWaveLanes>(squares);
  if (row_ok && lane == 0) sumsq[row] = squares;
}

struct LinesTag {
  static std::string text() { return "q8_0_lines"; }
};
struct RowsTag {
  static std::string text() { return "q8_0_rows"; }
};
struct BytesTag {
  static std::string text() { return "q8_0_rows_bytes"; }
};

template <int kWaves, int kRows>
hipError_t run_rows(const Q8Params &p, const void *blocks, void *out, float *sumsq,
                    uint32_t row_bytes, hipStream_t stream) {
  const uint32_t rows = (uint32_t)p.rows;
  constexpr int kRowsPerBlock = kWaves * kRows;
  note_variant<RowsTag>();
  hipLaunchKernelGGL((q8_0_rows<kWaves, kRows>), dim3((rows + kRowsPerBlock - 1) / kRowsPerBlock),
                     dim3(kWaves * kWaveLanes), (size_t)kRowsPerBlock * row_bytes, stream,
                     static_cast<const char *>(blocks), static_cast<uint16_t *>(out), sumsq, rows, p.k,
                     p.row_stride, row_bytes);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_q8_0_dequant(const Q8Params &p, const void *blocks, void *out, float *sumsq,
                               bool vectorised, hipStream_t stream) {
  if (p.rows == 0) return hipSuccess;
  const uint32_t rows = (uint32_t)p.rows;
  const uint32_t row_bytes = p.k / kBlockElems * kBlockBytes;
  const bool fast = vectorised && row_bytes != 0 && row_bytes % 16 == 0 &&
                    p.row_stride % 16 == 0 && row_bytes <= kMaxRowBytes;
  if (fast && p.k % 2048 == 0) {
    // Measured on MI355X for W[6144 x 2048] (38.6 MB of traffic, buffers rotated): 6.7 us with
    // plain loads and non-temporal stores; 7.4 us with non-temporal loads too; 8.6 / 10.5 us with
    // plain stores; a wave that walks several rows with the next row in flight 7.3 - 9.3 us; the
    // block-staged kernel below 7.1 us.
    constexpr int kWaves = 4;
    note_variant<LinesTag>();
    hipLaunchKernelGGL((q8_0_lines<kWaves>), dim3((rows + kWaves - 1) / kWaves), dim3(kWaves * kWaveLanes), 0, stream,
                       static_cast<const unsigned char *>(blocks), out, sumsq, rows, p.k, p.row_stride);
    return hipGetLastError();
  }
  if (fast) {
    // Measured on MI355X for W[6144 x 2048]: 2, 4 or 8 waves per block with one row per wave
    // all take about 8 us; two or four rows per wave are slower (9 to 13 us).
    return run_rows<4, 1>(p, blocks, out, sumsq, row_bytes, stream);
  }
  constexpr int kWaves = kBlockThreads / kWaveLanes;
  note_variant<BytesTag>();
  hipLaunchKernelGGL(q8_0_rows_bytes, dim3((rows + kWaves - 1) / kWaves), dim3(kBlockThreads), 0,
                     stream, static_cast<const uint8_t *>(blocks), static_cast<uint16_t *>(out),
                     sumsq, rows, p.k, p.row_stride);
  return hipGetLastError();
}

}  // namespace hyle_hip
