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
// Blocks are only 2-byte aligned, so a wave stages its rows in LDS with 16-byte
// global loads and re-slices them with 2-byte LDS reads; output leaves as
// 16-byte bf16x8 stores.  Each row's sum of squares of the exact products is
// reduced with a wave64 butterfly.
#include "device_common.h"
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

template <int kWaves, int kRows>
hipError_t run_rows(const Q8Params &p, const void *blocks, void *out, float *sumsq,
                    uint32_t row_bytes, hipStream_t stream) {
  const uint32_t rows = (uint32_t)p.rows;
  constexpr int kRowsPerBlock = kWaves * kRows;
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
  if (fast) {
    // Measured on MI355X for W[6144 x 2048]: 2, 4 or 8 waves per block with one row per wave
    // all take about 8 us; two or four rows per wave are slower (9 to 13 us).
    return run_rows<4, 1>(p, blocks, out, sumsq, row_bytes, stream);
  }
  constexpr int kWaves = kBlockThreads / kWaveLanes;
  hipLaunchKernelGGL(q8_0_rows_bytes, dim3((rows + kWaves - 1) / kWaves), dim3(kBlockThreads), 0,
                     stream, static_cast<const uint8_t *>(blocks), static_cast<uint16_t *>(out),
                     sumsq, rows, p.k, p.row_stride);
  return hipGetLastError();
}

}  // namespace hyle_hip
