// The row kernel of RMSNorm and LayerNorm and what its launchers share: included by norm.hip (the
// launch shapes that mask lanes and rows outside the tensor) and by norm_exact_rms.hip /
// norm_exact_layer.hip (the shapes that cover it exactly), which are separate files so that their
// many instantiations compile side by side.
#pragma once

#include <type_traits>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

template <class W, int kVec>
__device__ __forceinline__ void load_weight(const void *w, uint32_t vec, float (&out)[kVec]) {
  if constexpr (Traits<W>::kVec == kVec) {
    Traits<W>::unpack(load16(w, vec), out);
  } else {  // f32 parameters under a narrow input: two vectors per input vector
    float lo[4], hi[4];
    Traits<F32>::unpack(load16(w, 2 * (size_t)vec), lo);
    Traits<F32>::unpack(load16(w, 2 * (size_t)vec + 1), hi);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      out[j] = lo[j];
      out[4 + j] = hi[j];
    }
  }
}

enum : int { kPlain = 0, kScale = 1, kScaleBias = 2 };  // learned parameters of a launch

// `kRows` consecutive rows share one group of lanes.  Loads carry no branches (a lane outside
// the row, or a row outside the tensor, reads a clamped, valid address and zeroes the value).
// The rows are loaded one after another (the kVpl loads of a row together, the next row once
// they have arrived), the parameter vectors are fetched once for all rows, and every store
// follows the last load: a block reads in one phase and writes in another, which for tensors of
// a few tens of MB measured 10-15 % faster on MI355X than issuing all loads of a lane at once.
// `kExact` launches cover the tensor exactly (every lane a vector of every row of its group), so
// nothing is masked -- not even a group's second row by one comparison for the whole group: with
// that, LayerNorm over [8192, 2048] bf16 measured 14.5 us against 11.7 us -- and `kParameters` is
// fixed per instantiation: per element the bf16 LayerNorm is ten vector instructions instead of
// sixteen.  One such instruction per element is 0.44 us of every SIMD's time for 16.7 M
// elements, which the loads do not hide once all waves of a launch are resident together and
// move through their phases side by side.
template <class T, class W, int kLanes, int kVpl, int kThreads, int kRows, bool kLayer, int kParameters, bool kExact>
__global__ __launch_bounds__(kThreads) void norm_rows(const void *x, const void *w, const void *b,
                                                      void *y, uint32_t rows, uint32_t row_vectors,
                                                      float width, float epsilon) {
  constexpr int parameters = kParameters;
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kGroupsPerBlock = kThreads / kLanes;
  __shared__ float joint[kLayer ? 2 : 1][kRows][kThreads / kWaveLanes];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t first_row = (blockIdx.x * kGroupsPerBlock + threadIdx.x / kLanes) * kRows;

  u32x4 raw[kRows][kVpl];
  uint32_t vec[kVpl];
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    const uint32_t wanted = lane + k * kLanes;
    vec[k] = kExact || wanted < row_vectors ? wanted : row_vectors - 1;
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const uint32_t row = kExact || first_row + r < rows ? first_row + r : rows - 1;
    const size_t row_base = (size_t)row * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) raw[r][k] = load16_stream(x, row_base + vec[k]);
#pragma unroll
    for (int k = 0; k < kVpl; ++k) loads_issued(raw[r][k]);
  }
  float scale[kVpl][kVec], bias[kVpl][kVec];
  if constexpr (parameters != kPlain) {
#pragma unroll
    for (int k = 0; k < kVpl; ++k) load_weight<W, kVec>(w, vec[k], scale[k]);
  }
  if constexpr (kLayer && parameters == kScaleBias) {
#pragma unroll
    for (int k = 0; k < kVpl; ++k) load_weight<W, kVec>(b, vec[k], bias[k]);
  }
  // Row by row: measured on MI355X, reducing the statistics of both rows behind one barrier
  // is slower (RMSNorm over [8192, 2048] bf16: 13.5 us against 11.4 us).
  float v[kRows][kVpl][kVec];
  float inverse[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    bool ok[kVpl];
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      ok[k] = kExact || (first_row + r < rows && lane + k * kLanes < row_vectors);
      Traits<T>::unpack(raw[r][k], v[r][k]);
    }
    if constexpr (kLayer) {
      float sum = 0.0f;
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int j = 0; j < kVec; ++j) sum += ok[k] ? v[r][k][j] : 0.0f;
      const float mean = row_sum<kLanes>(sum, joint[1][r]) / width;
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[r][k][j] -= mean;
    }
    float squares = 0.0f;
#pragma unroll
    for (int k = 0; k < kVpl; ++k)
#pragma unroll
      for (int j = 0; j < kVec; ++j) {
        v[r][k][j] = ok[k] ? v[r][k][j] : 0.0f;
        squares = __builtin_fmaf(v[r][k][j], v[r][k][j], squares);
      }
    squares = row_sum<kLanes>(squares, joint[0][r]);
    inverse[r] = 1.0f / sqrtf(squares / width + epsilon);
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const uint32_t row = first_row + r;
    const size_t row_base = (size_t)row * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      if (kExact || (row < rows && lane + k * kLanes < row_vectors)) {
        float out[kVec];
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          out[j] = v[r][k][j] * inverse[r];
          if constexpr (kLayer && parameters == kScaleBias) out[j] = __builtin_fmaf(out[j], scale[k][j], bias[k][j]);
          else if constexpr (parameters != kPlain) out[j] = out[j] * scale[k][j];
        }
        store16_stream(y, row_base + vec[k], Traits<T>::pack(out));
      }
    }
  }
}

struct Bound {
  const void *x, *w, *b;
  void *y;
};

// <family>/<rms|layer>/<lanes>x<vectors per lane>/<threads per block>/<rows per lane group>[/<ragged|exact>]
template <bool kLayer, int kLanes, int kVpl, int kThreads, int kRows, int kForm> struct NormTag {  // kForm: 0 exact-only shape, 1 ragged, 2 exact
  static std::string text() {
    return std::string(kForm == 0 ? "norm_rows_exact/" : "norm_rows/") + (kLayer ? "layer/" : "rms/") + std::to_string(kLanes) + "x" +
           std::to_string(kVpl) + "/" + std::to_string(kThreads) + "/" + std::to_string(kRows) +
           (kForm == 1 ? "/ragged" : (kForm == 2 ? "/exact" : ""));
  }
};

// A launch shape used only when it covers the tensor exactly (no masked variant is built for it).
template <class T, class W, bool kLayer, int kLanes, int kVpl, int kThreads, int kRows>
bool run_exact(const NormParams &p, const Bound &io, int parameters, hipStream_t s) {
  constexpr int kRowsPerBlock = kThreads / kLanes * kRows;
  const uint32_t rows = (uint32_t)p.shape.rows, row_vectors = p.shape.width / Traits<T>::kVec;
  if (rows % kRowsPerBlock != 0 || row_vectors != (uint32_t)(kLanes * kVpl)) return false;
  note_variant<NormTag<kLayer, kLanes, kVpl, kThreads, kRows, 0>>();
  const dim3 grid(rows / kRowsPerBlock), block(kThreads);
  const float width = (float)p.shape.width;
  if (parameters == kPlain)
    hipLaunchKernelGGL((norm_rows<T, W, kLanes, kVpl, kThreads, kRows, kLayer, kPlain, true>), grid, block, 0, s, io.x, io.w,
                       io.b, io.y, rows, row_vectors, width, p.epsilon);
  else if (kLayer && parameters == kScaleBias)
    hipLaunchKernelGGL((norm_rows<T, W, kLanes, kVpl, kThreads, kRows, kLayer, kLayer ? kScaleBias : kScale, true>), grid, block,
                       0, s, io.x, io.w, io.b, io.y, rows, row_vectors, width, p.epsilon);
  else
    hipLaunchKernelGGL((norm_rows<T, W, kLanes, kVpl, kThreads, kRows, kLayer, kScale, true>), grid, block, 0, s, io.x, io.w,
                       io.b, io.y, rows, row_vectors, width, p.epsilon);
  return true;
}

}  // namespace

// Launches the shape that covers [rows, width] exactly, if there is one (norm_exact.h lists them:
// rows of 16 to 128 vectors in multiples of a block's rows, an even number of rows of 64 n, 128 n
// or 256 n vectors).  False: nothing was launched, take the masked shapes.
bool launch_norm_exact_rms(Elem type, const NormParams &p, const void *x, const void *w, void *y, hipStream_t stream);
bool launch_norm_exact_layer(Elem type, const NormParams &p, const void *x, const void *w, const void *b, void *y,
                             hipStream_t stream);

}  // namespace hyle_hip
