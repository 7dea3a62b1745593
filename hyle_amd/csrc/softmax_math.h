// What the row softmax kernels share (softmax.hip: any width and row count; softmax_exact.hip:
// launch shapes that cover the tensor exactly).
#pragma once

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

enum : int { kMaskNone = 0, kMaskAdditive = 1, kMaskBoolean = 2 };

// exp(t) * 2^32 for t <= 0.  t * log2(e) is taken as a rounded product plus its exact
// residual (one fma), so the hardware exp2 sees an argument good to about 2e-8 * |t|
// and the result stays within 2e-6 relative down to the subnormal range.
__device__ __forceinline__ float exp_scaled(float t) {
  constexpr float kLog2e = 1.44269504088896340736f;
  constexpr float kLn2 = 0.69314718055994530942f;
  t = fmaxf(t, -200.0f);  // exp(-200) * 2^32 is below every subnormal; also tames -inf
  const float hi = t * kLog2e;
  const float lo = __builtin_fmaf(t, kLog2e, -hi);
  const float p = __builtin_amdgcn_exp2f(hi + 32.0f);
  return __builtin_fmaf(p, lo * kLn2, p);
}

// NaN or +inf: the values that make a softmax row undefined
// (src/simd/math/activations.cc:181-186).
__device__ __forceinline__ bool poisons_row(float v) {
  return __builtin_amdgcn_class(v, 0x001 | 0x002 | 0x200);  // sNaN | qNaN | +inf
}


struct MaskRows {
  int32_t outer_rank;
  uint32_t outer_dims[kMaxRank];
  int64_t outer_strides[kMaxRank];
  int64_t inner_stride;
};

__device__ __forceinline__ int64_t mask_row_offset(const MaskRows &m, uint32_t row) {
  int64_t offset = 0;
  uint32_t rest = row;
  for (int axis = m.outer_rank - 1; axis >= 0; --axis) {
    const uint32_t extent = m.outer_dims[axis];
    offset += (int64_t)(rest % extent) * m.outer_strides[axis];
    rest /= extent;
  }
  return offset;
}

}  // namespace

// Rows in the launch shape that covers [rows, width] exactly, if there is one (a mask that has a
// value per column; `mask` is nullptr without one).  False: nothing was launched.
bool launch_softmax_exact(Elem type, const SoftmaxParams &p, const void *x, const void *mask, void *y, hipStream_t stream);

}  // namespace hyle_hip
