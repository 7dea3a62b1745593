// Row Softmax / LogSoftmax without a mask, in launch shapes that cover the tensor exactly: every
// lane holds whole vectors of every row of its group, so nothing is masked, and a lane group takes
// several rows one after the other, the later rows' loads in flight while the first is reduced,
// exponentiated and stored -- the shapes RMSNorm and LayerNorm use for the same reason
// (norm_exact.h).  Arithmetic and the invalid-row rule are those of softmax.hip; a NaN shows as an
// unordered pair and +inf as the row's maximum.  Results stored in 8 or 11 significand bits take
// their exponentials from one fused multiply-add into the hardware exp2.
//
// The exponentials keep a row's values in registers across three passes, so -- unlike the norms --
// at most four vectors per lane measured best where the width allows it.  MI355X, 67 MB per
// launch (a plain copy: 11.0 us), against the shapes of softmax.hip (one row per group, every
// element behind an in-the-row test, the residual form of exp for every type):
//   f32   [8192, 1024] 12.0 (12.7)  [4096, 2048] 10.7 (12.7)  [2048, 4096] 10.5 (13.1)  [1024, 8192] 11.5 (12.6)
//   bf16  [16384, 1024] 11.0 (13.6) [8192, 2048] 10.7 (13.9)  [4096, 4096] 10.6 (13.6)  [2048, 8192] 10.5 (14.2)
// 512 vectors per row: 128 lanes x 4 vectors, two rows 11.7 (bf16) / 10.9 (f32); 64 x 8 12.7 / 11.5;
// 256 x 2 12.0 / 12.0; one row per group 12.5 - 13.1 / 12.6 - 12.9.
#include "softmax_math.h"

namespace hyle_hip {
namespace {

// exp(t) * 2^32 for t <= 0, for results that are stored in 8 or 11 significand bits: one fused
// multiply-add into the hardware exp2 (about 1e-6 relative; -inf gives 0).  f32 storage keeps the
// form with the exact residual.
template <class T> __device__ __forceinline__ float exp_for(float t) {
  if constexpr (Traits<T>::kSize == 4) return exp_scaled(t);
  else return __builtin_amdgcn_exp2f(__builtin_fmaf(t, 1.44269504088896340736f, 32.0f));
}

template <class T, int kLanes, int kVpl, int kThreads, int kRows, bool kLog>
__global__ __launch_bounds__(kThreads) void softmax_rows_exact(const void *x, void *y, uint32_t row_vectors, float scale) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kWaves = kThreads / kWaveLanes;
  __shared__ float joint_max[kRows][kWaves], joint_sum[kRows][kWaves], joint_count[kRows][kWaves];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t first_row = (blockIdx.x * (kThreads / kLanes) + threadIdx.x / kLanes) * kRows;
  u32x4 raw[kRows][kVpl];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const size_t row_base = (size_t)(first_row + r) * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) raw[r][k] = load16_stream(x, row_base + lane + k * kLanes);
#pragma unroll
    for (int k = 0; k < kVpl; ++k) loads_issued(raw[r][k]);
  }
  float v[kRows][kVpl][kVec];
  float normaliser[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    float peak = -INFINITY;
    bool poisoned = false;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      Traits<T>::unpack(raw[r][k], v[r][k]);
#pragma unroll
      for (int j = 0; j < kVec; ++j) v[r][k][j] *= scale;
#pragma unroll
      for (int j = 0; j < kVec; j += 2) {
        poisoned = poisoned || __builtin_isunordered(v[r][k][j], v[r][k][j + 1]);
        peak = fmaxf(peak, fmaxf(v[r][k][j], v[r][k][j + 1]));
      }
    }
    // an infinite maximum of either sign marks the row: +inf poisoned, -inf nothing finite
    peak = row_max<kLanes>(poisoned ? INFINITY : peak, joint_max[r]);
    const bool invalid = __builtin_fabsf(peak) == INFINITY;
    float total = 0.0f, maxima = 0.0f;
#pragma unroll
    for (int k = 0; k < kVpl; ++k)
#pragma unroll
      for (int j = 0; j < kVec; ++j) {
        const float shifted = v[r][k][j] - peak;
        if constexpr (kLog) {  // the maxima are counted, not summed (src/compute_provider_cuda/reduction_kernel.cu:178-196)
          const bool at_peak = shifted == 0.0f;
          total += at_peak ? 0.0f : exp_for<T>(shifted);
          maxima += at_peak ? 1.0f : 0.0f;
          v[r][k][j] = shifted;
        } else {
          v[r][k][j] = exp_for<T>(shifted);
          total += v[r][k][j];
        }
      }
    total = row_sum<kLanes>(total, joint_sum[r]);  // = 2^32 * sum(exp)
    if constexpr (kLog) maxima = row_sum<kLanes>(maxima, joint_count[r]);
    normaliser[r] = kLog ? log1pf((maxima - 1.0f) + total * 2.3283064365386963e-10f) : 1.0f / total;
    if (invalid) normaliser[r] = __builtin_nanf("");
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const size_t row_base = (size_t)(first_row + r) * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      float out[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j) out[j] = kLog ? v[r][k][j] - normaliser[r] : v[r][k][j] * normaliser[r];
      store16_stream(y, row_base + lane + k * kLanes, Traits<T>::pack(out));
    }
  }
}

template <class T, int kLanes, int kVpl, int kThreads, int kRows>
bool run_exact(const SoftmaxParams &p, const void *x, void *y, hipStream_t s) {
  constexpr int kRowsPerBlock = kThreads / kLanes * kRows;
  const uint32_t rows = (uint32_t)p.shape.rows, row_vectors = p.shape.width / Traits<T>::kVec;
  if (rows % kRowsPerBlock != 0 || row_vectors != (uint32_t)(kLanes * kVpl)) return false;
  const dim3 grid(rows / kRowsPerBlock), block(kThreads);
  if (p.log) hipLaunchKernelGGL((softmax_rows_exact<T, kLanes, kVpl, kThreads, kRows, true>), grid, block, 0, s, x, y, row_vectors, p.scale);
  else hipLaunchKernelGGL((softmax_rows_exact<T, kLanes, kVpl, kThreads, kRows, false>), grid, block, 0, s, x, y, row_vectors, p.scale);
  return true;
}

template <class T>
bool run_exact_shape(const SoftmaxParams &p, const void *x, void *y, hipStream_t s) {
  constexpr uint32_t kVec = Traits<T>::kVec;
  if (p.shape.width % kVec != 0) return false;
  const uint32_t vectors = p.shape.width / kVec;
  switch (vectors) {
    case 16: return run_exact<T, 8, 2, 64, 4>(p, x, y, s);
    case 32: return run_exact<T, 16, 2, 64, 4>(p, x, y, s);
    case 64: return run_exact<T, 32, 2, 64, 4>(p, x, y, s);
    case 128: return run_exact<T, 64, 2, 64, 4>(p, x, y, s);
    case 192: return run_exact<T, 64, 3, 64, 2>(p, x, y, s);
    case 256: return run_exact<T, 128, 2, 128, 2>(p, x, y, s);
    case 320: return run_exact<T, 64, 5, 64, 2>(p, x, y, s);
    case 384: return run_exact<T, 128, 3, 128, 2>(p, x, y, s);
    case 448: return run_exact<T, 64, 7, 64, 2>(p, x, y, s);
    case 512: return run_exact<T, 128, 4, 128, 2>(p, x, y, s);
    case 640: return run_exact<T, 128, 5, 128, 2>(p, x, y, s);
    case 768: return run_exact<T, 256, 3, 256, 2>(p, x, y, s);
    case 896: return run_exact<T, 128, 7, 128, 2>(p, x, y, s);
    case 1024: return run_exact<T, 256, 4, 256, 2>(p, x, y, s);
    case 1280: return run_exact<T, 256, 5, 256, 2>(p, x, y, s);
    case 1536: return run_exact<T, 512, 3, 512, 2>(p, x, y, s);
    case 1792: return run_exact<T, 256, 7, 256, 2>(p, x, y, s);
    case 2048: return run_exact<T, 512, 4, 512, 2>(p, x, y, s);
    default: return false;
  }
}

}  // namespace

bool launch_softmax_exact(Elem type, const SoftmaxParams &p, const void *x, void *y, hipStream_t stream) {
  switch (type) {
    case Elem::kF32: return run_exact_shape<F32>(p, x, y, stream);
    case Elem::kF16: return run_exact_shape<F16>(p, x, y, stream);
    case Elem::kBF16: return run_exact_shape<BF16>(p, x, y, stream);
  }
  return false;
}

}  // namespace hyle_hip
