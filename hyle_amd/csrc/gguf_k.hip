// GGUF Q4_K and Q6_K rows -> bf16 [rows, k] plus the f32 row sums of squares of the exact f32
// values, the K-quant siblings of q8_0.hip.
//
// Geometry from the reference (src/compute_ops/low_precision.cc:22-27: 256 elements in 144 and
// 210 bytes); the decode is ggml's dequantize_row_q4_K / dequantize_row_q6_K, restated from the
// published block layouts, checked against the two readings of these formats the reference
// tree holds (third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38;
// tests/compute_models/qwen27_original_nextn_reference.h:74-86,262-287):
//   Q4_K  {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]}   y = (d * sc) * q - (dmin * m)
//   Q6_K  {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d}  y = (d * scale) * (q - 32)
// with separate f32 roundings for the products and the subtraction, as the source writes them.
//
// Two kernels.  Rows made of whole 16-byte vectors with K a multiple of 2048 (the usual case)
// take one wave per row, whole cache lines into wave-private LDS and word-wise decoding
// (k_quant_lines, measured 5.9 / 6.3 us for Q4_K / Q6_K [6144 x 2048] on MI355X).  Anything else
// takes the general kernel: a block of 256 threads takes four rows at a time, eight super-blocks
// of each (at most 1680 bytes) are staged in LDS per step with the widest loads the row's
// address allows, and a thread decodes eight neighbouring values from LDS bytes (10.7 / 12.3 us
// for the same shape).  Both store eight values as one 16-byte vector.
#include "device_common.h"
#include "gguf_decode.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr int kChunkBlocks = kBlockThreads * 8 / kSuper;  // super-blocks decoded per step: 8

// Bytes -> LDS with the widest loads the address allows (Q4_K rows of a 16-byte aligned tensor
// always take words; Q6_K blocks are only 2-byte aligned as a rule).
__device__ __forceinline__ void stage(unsigned char *to, const unsigned char *from, uint32_t bytes) {
  if (((reinterpret_cast<uintptr_t>(from) | bytes) & 3u) == 0) {
    for (uint32_t i = threadIdx.x; i < bytes / 4; i += kBlockThreads)
      reinterpret_cast<uint32_t *>(to)[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(from) + i);
  } else if (((reinterpret_cast<uintptr_t>(from) | bytes) & 1u) == 0) {
    for (uint32_t i = threadIdx.x; i < bytes / 2; i += kBlockThreads)
      reinterpret_cast<uint16_t *>(to)[i] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(from) + i);
  } else {
    for (uint32_t i = threadIdx.x; i < bytes; i += kBlockThreads) to[i] = from[i];
  }
}

// kRows rows per block: their chunks are staged together, so kRows times the bytes are in flight
// per barrier and each thread has kRows independent decodes.
template <int kKind, int kRows>  // 0 = Q4_K, 1 = Q6_K
__global__ __launch_bounds__(kBlockThreads) void k_quant_rows(const unsigned char *blocks, void *out,
                                                              float *sumsq, uint32_t rows, uint32_t k,
                                                              uint64_t row_stride) {
  constexpr uint32_t kBlockBytes = kKind == 0 ? 144 : 210;
  constexpr uint32_t kSlot = (kChunkBlocks * kBlockBytes + 15) / 16 * 16;
  __shared__ __align__(16) unsigned char staged[kRows][kSlot];
  __shared__ float joint[kRows][kBlockThreads / kWaveLanes];
  const uint32_t first_row = blockIdx.x * kRows;
  const uint32_t super_blocks = k / kSuper;
  float acc[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) acc[r] = 0.0f;
  for (uint32_t first = 0; first < super_blocks; first += kChunkBlocks) {
    const uint32_t count = min((uint32_t)kChunkBlocks, super_blocks - first);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const uint32_t row = min(first_row + r, rows - 1);  // a row past the end re-reads the last one
      stage(staged[r], blocks + (size_t)row * row_stride + (size_t)first * kBlockBytes, count * kBlockBytes);
    }
    __syncthreads();
    const uint32_t local = threadIdx.x * 8;  // position within the chunk
    if (local < count * kSuper) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const unsigned char *blk = staged[r] + (local / kSuper) * kBlockBytes;
        float y[8];
        if constexpr (kKind == 0) decode_q4_k(blk, local % kSuper, y);
        else decode_q6_k(blk, local % kSuper, y);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[r] = __builtin_fmaf(y[j], y[j], acc[r]);
        if (first_row + r < rows) {
          const size_t element = (size_t)(first_row + r) * k + (size_t)first * kSuper + local;
          store16_stream(out, element / 8, Traits<BF16>::pack(y));
        }
      }
    }
    __syncthreads();  // the next step overwrites the staging
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const float total = row_sum<kBlockThreads>(acc[r], joint[r]);
    if (threadIdx.x == 0 && first_row + r < rows) sumsq[first_row + r] = total;
  }
}

// Rows made of whole 16-byte vectors, K a multiple of 2048: one wave per row and no barrier.
// The wave reads 2048 values' worth of blocks (1152 or 1680 bytes) as 16-byte vectors, one per
// lane and request, so that every cache line is asked for once; parks them in a region of LDS
// that only this wave touches (LDS executes one wave's instructions in order); and each lane
// decodes eight neighbouring values at a time from aligned 32-bit words, so that a store
// instruction of the wave writes 1 KiB of consecutive bf16.  The next 2048 values are on their
// way while these are decoded.  The loads are plain ones: with the non-temporal hint the same
// kernel took 8.0 / 9.3 us instead of 5.9 / 6.3 us (the bf16 stores keep the hint).
template <int kKind>  // 0 = Q4_K, 1 = Q6_K
__global__ __launch_bounds__(kBlockThreads) void k_quant_lines(const unsigned char *blocks, void *out, float *sumsq,
                                                               uint32_t rows, uint32_t k, uint64_t row_stride) {
  constexpr uint32_t kBlockBytes = kKind == 0 ? 144 : 210;
  constexpr uint32_t kSpan = 2048;                                  // values per step
  constexpr uint32_t kVectors = kSpan / kSuper * kBlockBytes / 16;  // 72 or 105
  constexpr int kLoads = (kVectors + kWaveLanes - 1) / kWaveLanes;  // 2
  constexpr int kWaves = kBlockThreads / kWaveLanes;
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
  for (int i = 0; i < kLoads; ++i) {  // past the span: its last vector again (parked, never read)
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
    const uint32_t following = step + 1 < steps ? step + 1 : step;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) raw[i] = load16(source, (size_t)following * kVectors + vec[i]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (uint32_t i = 0; i < kSpan / (kWaveLanes * 8); ++i) {
      const uint32_t p = (i * kWaveLanes + lane) * 8;  // position within the span
      float y[8];
      if constexpr (kKind == 0) decode_q4_k_words(slot, (p / kSuper) * kBlockBytes, p % kSuper, y);
      else decode_q6_k_words(slot, (p / kSuper) * kBlockBytes, p % kSuper, y);
#pragma unroll
      for (int j = 0; j < 8; ++j) squares = __builtin_fmaf(y[j], y[j], squares);
      store16_stream(out, ((size_t)row * k + (size_t)step * kSpan + p) / 8, Traits<BF16>::pack(y));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  squares = group_sum<kWaveLanes>(squares);
  if (lane == 0) sumsq[row] = squares;
}

}  // namespace

namespace {
template <int kKind, bool kLines> struct KQuantTag {
  static std::string text() { return std::string(kLines ? "k_quant_lines/" : "k_quant_rows/") + (kKind == 0 ? "q4_k" : "q6_k"); }
};
}  // namespace

hipError_t launch_k_quant_dequant(const KQuantParams &p, const void *blocks, void *out, float *sumsq,
                                  hipStream_t stream) {
  if (p.rows == 0) return hipSuccess;
  const unsigned char *in = static_cast<const unsigned char *>(blocks);
  const bool lines = ((reinterpret_cast<uintptr_t>(blocks) | p.row_stride) & 15u) == 0 && p.k != 0 && p.k % 2048 == 0;
  if (lines) {
    constexpr int kWaves = kBlockThreads / kWaveLanes;
    const dim3 grid(((uint32_t)p.rows + kWaves - 1) / kWaves), block(kBlockThreads);
    if (p.kind == 0) note_variant<KQuantTag<0, true>>();
    else note_variant<KQuantTag<1, true>>();
    if (p.kind == 0)
      hipLaunchKernelGGL((k_quant_lines<0>), grid, block, 0, stream, in, out, sumsq, (uint32_t)p.rows, p.k,
                         p.row_stride);
    else
      hipLaunchKernelGGL((k_quant_lines<1>), grid, block, 0, stream, in, out, sumsq, (uint32_t)p.rows, p.k,
                         p.row_stride);
    return hipGetLastError();
  }
  constexpr int kRows = 4;
  const dim3 grid(((uint32_t)p.rows + kRows - 1) / kRows), block(kBlockThreads);
  if (p.kind == 0) note_variant<KQuantTag<0, false>>();
  else note_variant<KQuantTag<1, false>>();
  if (p.kind == 0)
    hipLaunchKernelGGL((k_quant_rows<0, kRows>), grid, block, 0, stream, in, out, sumsq, (uint32_t)p.rows, p.k,
                       p.row_stride);
  else
    hipLaunchKernelGGL((k_quant_rows<1, kRows>), grid, block, 0, stream, in, out, sumsq, (uint32_t)p.rows, p.k,
                       p.row_stride);
  return hipGetLastError();
}

}  // namespace hyle_hip
