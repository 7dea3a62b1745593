// What the row softmax kernels share (softmax.hip: every mask, any width; softmax_exact.hip:
// unmasked rows in launch shapes that cover the tensor exactly).
#pragma once

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

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

}  // namespace

// Unmasked rows in the launch shape that covers [rows, width] exactly, if there is one.  False:
// nothing was launched.
bool launch_softmax_exact(Elem type, const SoftmaxParams &p, const void *x, void *y, hipStream_t stream);

}  // namespace hyle_hip
