// norm.hip -- RMSNorm and LayerNorm over the last axis for gfx950.
//
// One pass over HBM: a row is split over `kLanes` lanes (a slice of a wave, a
// whole wave, or several waves of a block), each lane keeps its 16-byte
// vectors in registers, the row statistics are reduced with wave64 DPP
// butterflies (LDS only to join the waves of a row), then the same registers
// are scaled and stored.  In-place is safe: every load of a row retires before
// its first store.
//
// Arithmetic follows the reference
// (src/compute_provider_native/normalization.cc:41-80,
//  src/simd/math/activations.cc:124-175): f32 accumulation,
//   RMSNorm    inv = 1 / sqrt(sum(x^2) / n + eps), then (x * inv) * w
//   LayerNorm  mean = sum(x) / n, inv = 1 / sqrt(sum((x - mean)^2) / n + eps),
//              then fma((x - mean) * inv, scale, bias); scale alone multiplies
// with a true divide and square root and one RN-even store.
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
// nothing is masked, and `kParameters` is fixed per instantiation: per element the bf16 LayerNorm
// is ten vector instructions instead of sixteen.  One such instruction per element is 0.44 us of
// every SIMD's time for 16.7 M elements, which the loads do not hide once all waves of a launch
// are resident together and move through their phases side by side.
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

// Any width, any element alignment: one block per row, the row is re-read for each pass
// (the re-reads come from cache).
template <class T, class W, bool kLayer>
__global__ __launch_bounds__(kBlockThreads) void norm_generic(const void *x, const void *w, const void *b,
                                                              void *y, uint32_t width, float epsilon,
                                                              int parameters) {
  __shared__ float joint[2][kBlockThreads / kWaveLanes];
  const size_t base = (size_t)blockIdx.x * width;
  float mean = 0.0f;
  if constexpr (kLayer) {
    float sum = 0.0f;
    for (uint32_t i = threadIdx.x; i < width; i += kBlockThreads) sum += Traits<T>::load(x, base + i);
    mean = row_sum<kBlockThreads>(sum, joint[1]) / (float)width;
  }
  float squares = 0.0f;
  for (uint32_t i = threadIdx.x; i < width; i += kBlockThreads) {
    const float v = Traits<T>::load(x, base + i) - mean;
    squares = __builtin_fmaf(v, v, squares);
  }
  squares = row_sum<kBlockThreads>(squares, joint[0]);
  const float inverse = 1.0f / sqrtf(squares / (float)width + epsilon);
  // every read of this row is complete before its first store: an exact alias is safe
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < width; i += kBlockThreads) {
    float r = (Traits<T>::load(x, base + i) - mean) * inverse;
    if (kLayer && parameters == kScaleBias) r = __builtin_fmaf(r, Traits<W>::load(w, i), Traits<W>::load(b, i));
    else if (parameters != kPlain) r = r * Traits<W>::load(w, i);
    Traits<T>::store(y, base + i, r);
  }
}

struct Bound {
  const void *x, *w, *b;
  void *y;
};

template <class T, class W, bool kLayer, int kLanes, int kVpl, int kThreads = kBlockThreads, int kRows = 1>
hipError_t run_rows(const NormParams &p, const Bound &io, int parameters, hipStream_t s) {
  constexpr int kRowsPerBlock = kThreads / kLanes * kRows;
  const uint32_t rows = (uint32_t)p.shape.rows, row_vectors = p.shape.width / Traits<T>::kVec;
  const uint32_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  // Measured on MI355X for [8192, 2048] bf16: the unmasked LayerNorm runs 11.3-11.6 us against
  // 14.3 us masked; the unmasked RMSNorm is no faster than the masked one (11.4-12.0 us against
  // 11.2-11.6 us), so it is not instantiated.
  const bool exact = kLayer && rows % kRowsPerBlock == 0 && row_vectors == (uint32_t)(kLanes * kVpl);
  auto go = [&](auto parameters_tag, auto exact_tag) {
    hipLaunchKernelGGL((norm_rows<T, W, kLanes, kVpl, kThreads, kRows, kLayer, decltype(parameters_tag)::value,
                                  decltype(exact_tag)::value>),
                       dim3(blocks), dim3(kThreads), 0, s, io.x, io.w, io.b, io.y, rows, row_vectors,
                       (float)p.shape.width, p.epsilon);
  };
  auto by_shape = [&](auto parameters_tag) {
    if constexpr (kLayer) {
      if (exact) return go(parameters_tag, std::true_type{});
    }
    go(parameters_tag, std::false_type{});
  };
  if (parameters == kPlain) by_shape(std::integral_constant<int, kPlain>{});
  else if (kLayer && parameters == kScaleBias) by_shape(std::integral_constant<int, kLayer ? kScaleBias : kScale>{});
  else by_shape(std::integral_constant<int, kScale>{});
  return hipGetLastError();
}

template <class T, class W, bool kLayer>
hipError_t run(const NormParams &p, const Bound &io, bool vectorised, hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const uint32_t vectors = p.shape.width / kVec;
  const int parameters = !p.has_weight ? kPlain : (p.has_bias ? kScaleBias : kScale);
  if (vectorised && p.shape.width % kVec == 0 && vectors <= 8u * 1024u) {
    if (vectors <= 8) return run_rows<T, W, kLayer, 8, 1>(p, io, parameters, s);
    if (vectors <= 16) return run_rows<T, W, kLayer, 16, 1>(p, io, parameters, s);
    if (vectors <= 32) return run_rows<T, W, kLayer, 32, 1>(p, io, parameters, s);
    if (vectors <= 64) return run_rows<T, W, kLayer, 64, 1>(p, io, parameters, s);
    // Two vectors per lane, two rows per lane group and small blocks measured best on MI355X
    // for X[8192, 2048] bf16: 11.2 us, against 12.3-13.5 us for the same rows in blocks of
    // 256-1024 threads and 13.7-15.4 us for one vector per lane with four or eight rows.
    if (vectors <= 128) return run_rows<T, W, kLayer, 64, 2, 256, 2>(p, io, parameters, s);
    if (vectors <= 256) {
      // One wave per row (no barrier), two rows one after the other: the second row's loads are
      // in flight while the first is reduced, scaled and stored.  [8192, 2048] bf16 on MI355X:
      // LayerNorm 11.3 us in blocks of one wave (11.5-11.8 us in blocks of 2-8 waves, 12.2 us
      // with four rows per wave, 13.5 us with one, 14.3 us for two waves per row); RMSNorm
      // 11.2 us in blocks of four waves (11.6-11.9 us for two waves per row).
      if constexpr (kLayer) return run_rows<T, W, kLayer, 64, 4, 64, 2>(p, io, parameters, s);
      return run_rows<T, W, kLayer, 64, 4, 256, 2>(p, io, parameters, s);
    }
    if (vectors <= 512) return run_rows<T, W, kLayer, 256, 2, 256, 2>(p, io, parameters, s);
    if (vectors <= 1024) return run_rows<T, W, kLayer, 256, 4>(p, io, parameters, s);
    if (vectors <= 2048) return run_rows<T, W, kLayer, 256, 8>(p, io, parameters, s);
    if (vectors <= 4096) return run_rows<T, W, kLayer, 1024, 4, 1024>(p, io, parameters, s);
    return run_rows<T, W, kLayer, 1024, 8, 1024>(p, io, parameters, s);
  }
  hipLaunchKernelGGL((norm_generic<T, W, kLayer>), dim3((uint32_t)p.shape.rows), dim3(kBlockThreads), 0, s,
                     io.x, io.w, io.b, io.y, p.shape.width, p.epsilon, parameters);
  return hipGetLastError();
}

template <bool kLayer>
hipError_t run_typed(Elem type, const NormParams &p, const Bound &io, bool vectorised, hipStream_t stream) {
  switch (type) {
    case Elem::kF32: return run<F32, F32, kLayer>(p, io, vectorised, stream);
    case Elem::kF16:
      return p.weight_f32 ? run<F16, F32, kLayer>(p, io, vectorised, stream)
                          : run<F16, F16, kLayer>(p, io, vectorised, stream);
    case Elem::kBF16:
      return p.weight_f32 ? run<BF16, F32, kLayer>(p, io, vectorised, stream)
                          : run<BF16, BF16, kLayer>(p, io, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_norm(Elem type, const NormParams &p, const void *x, const void *w, const void *b,
                       void *y, bool vectorised, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  const Bound io{x, w, b, y};
  return p.layer ? run_typed<true>(type, p, io, vectorised, stream)
                 : run_typed<false>(type, p, io, vectorised, stream);
}

}  // namespace hyle_hip
