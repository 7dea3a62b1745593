// rmsnorm.hip -- RMSNorm over the last axis for gfx950.
//
// One pass over HBM: a row is split over `kLanes` lanes (a slice of a wave, a
// whole wave, or the four waves of a block), each lane keeps its 16-byte
// vectors in registers, the sum of squares is reduced with wave64 DPP
// butterflies (LDS only to join the four waves of a block), then the same
// registers are scaled and stored.  In-place is safe: every load of a row
// retires before its first store.
//
// Arithmetic follows the reference
// (src/compute_provider_native/normalization.cc:41-80,
//  src/simd/math/activations.cc:124-146): f32 accumulation,
// inv = 1 / sqrt(sum / n + eps) with a true divide and square root, then
// (x * inv) * w with one RN-even store.
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

template <int kLanes> __device__ __forceinline__ float row_sum(float v, float *joint) {
  if constexpr (kLanes <= kWaveLanes) {
    return group_sum<kLanes>(v);
  } else {
    static_assert(kLanes == kBlockThreads, "a row spans a slice of a wave, a wave, or the block");
    v = group_sum<kWaveLanes>(v);
    if ((threadIdx.x & (kWaveLanes - 1)) == 0) joint[threadIdx.x / kWaveLanes] = v;
    __syncthreads();
    return (joint[0] + joint[1]) + (joint[2] + joint[3]);
  }
}

template <class W, int kVec>
__device__ __forceinline__ void load_weight(const void *w, uint32_t vec, float (&out)[kVec]) {
  if constexpr (Traits<W>::kVec == kVec) {
    Traits<W>::unpack(load16(w, vec), out);
  } else {  // f32 weights under a narrow input: two vectors per input vector
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

template <class T, class W, int kLanes, int kVpl>
__global__ __launch_bounds__(kBlockThreads) void rms_norm_rows(const void *x, const void *w,
                                                               void *y, uint32_t rows,
                                                               uint32_t row_vectors, float width,
                                                               float epsilon, int has_weight) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kRowsPerBlock = kBlockThreads / kLanes;
  __shared__ float joint[4];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t row = blockIdx.x * kRowsPerBlock + threadIdx.x / kLanes;
  const bool row_ok = row < rows;
  const size_t row_base = (size_t)row * row_vectors;

  float v[kVpl][kVec];
  float scale[kVpl][kVec];
  float squares = 0.0f;
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    const uint32_t vec = lane + k * kLanes;
    if (row_ok && vec < row_vectors) {
      Traits<T>::unpack(load16_stream(x, row_base + vec), v[k]);
      if (has_weight) load_weight<W, kVec>(w, vec, scale[k]);
    } else {
#pragma unroll
      for (int j = 0; j < kVec; ++j) v[k][j] = 0.0f;
    }
  }
#pragma unroll
  for (int k = 0; k < kVpl; ++k)
#pragma unroll
    for (int j = 0; j < kVec; ++j) squares = __builtin_fmaf(v[k][j], v[k][j], squares);

  squares = row_sum<kLanes>(squares, joint);
  const float inverse = 1.0f / sqrtf(squares / width + epsilon);

#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    const uint32_t vec = lane + k * kLanes;
    if (row_ok && vec < row_vectors) {
      float r[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j) {
        r[j] = v[k][j] * inverse;
        if (has_weight) r[j] = r[j] * scale[k][j];
      }
      store16_stream(y, row_base + vec, Traits<T>::pack(r));
    }
  }
}

// Any width, any element alignment: one block per row, the row is read twice
// (the second read comes from cache).
template <class T, class W>
__global__ __launch_bounds__(kBlockThreads) void rms_norm_generic(const void *x, const void *w,
                                                                  void *y, uint32_t width,
                                                                  float epsilon, int has_weight) {
  __shared__ float joint[4];
  const size_t base = (size_t)blockIdx.x * width;
  float squares = 0.0f;
  for (uint32_t i = threadIdx.x; i < width; i += kBlockThreads) {
    const float v = Traits<T>::load(x, base + i);
    squares = __builtin_fmaf(v, v, squares);
  }
  squares = row_sum<kBlockThreads>(squares, joint);
  const float inverse = 1.0f / sqrtf(squares / (float)width + epsilon);
  for (uint32_t i = threadIdx.x; i < width; i += kBlockThreads) {
    float r = Traits<T>::load(x, base + i) * inverse;
    if (has_weight) r = r * Traits<W>::load(w, i);
    Traits<T>::store(y, base + i, r);
  }
}

template <class T, class W, int kLanes, int kVpl>
hipError_t run_rows(const NormParams &p, const void *x, const void *w, void *y, hipStream_t s) {
  constexpr int kRowsPerBlock = kBlockThreads / kLanes;
  const uint32_t rows = (uint32_t)p.shape.rows;
  const uint32_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  hipLaunchKernelGGL((rms_norm_rows<T, W, kLanes, kVpl>), dim3(blocks), dim3(kBlockThreads), 0, s, x,
                     w, y, rows, p.shape.width / Traits<T>::kVec, (float)p.shape.width, p.epsilon,
                     p.has_weight ? 1 : 0);
  return hipGetLastError();
}

template <class T, class W>
hipError_t run(const NormParams &p, const void *x, const void *w, void *y, bool vectorised,
               hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const uint32_t vectors = p.shape.width / kVec;
  if (vectorised && p.shape.width % kVec == 0 && vectors <= 8u * kBlockThreads) {
    if (vectors <= 8) return run_rows<T, W, 8, 1>(p, x, w, y, s);
    if (vectors <= 16) return run_rows<T, W, 16, 1>(p, x, w, y, s);
    if (vectors <= 32) return run_rows<T, W, 32, 1>(p, x, w, y, s);
    if (vectors <= 64) return run_rows<T, W, 64, 1>(p, x, w, y, s);
    if (vectors <= 128) return run_rows<T, W, 64, 2>(p, x, w, y, s);
    if (vectors <= 256) return run_rows<T, W, 64, 4>(p, x, w, y, s);
    if (vectors <= 512) return run_rows<T, W, 64, 8>(p, x, w, y, s);
    if (vectors <= 1024) return run_rows<T, W, 256, 4>(p, x, w, y, s);
    return run_rows<T, W, 256, 8>(p, x, w, y, s);
  }
  hipLaunchKernelGGL((rms_norm_generic<T, W>), dim3((uint32_t)p.shape.rows), dim3(kBlockThreads), 0,
                     s, x, w, y, p.shape.width, p.epsilon, p.has_weight ? 1 : 0);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_rms_norm(Elem type, const NormParams &p, const void *x, const void *w, void *y,
                           bool vectorised, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run<F32, F32>(p, x, w, y, vectorised, stream);
    case Elem::kF16:
      return p.weight_f32 ? run<F16, F32>(p, x, w, y, vectorised, stream)
                          : run<F16, F16>(p, x, w, y, vectorised, stream);
    case Elem::kBF16:
      return p.weight_f32 ? run<BF16, F32>(p, x, w, y, vectorised, stream)
                          : run<BF16, BF16>(p, x, w, y, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
