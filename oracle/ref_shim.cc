// ref_shim.cc -- C-callable doorway onto the reference's own scalar semantic
// floor, used ONLY to validate oracle/hyle_oracle.c (test infrastructure).
//
// This file contains no arithmetic.  It includes the reference's headers where
// they lie (the Makefile passes -I<reference> -I<reference>/include) and
// forwards to the functions the reference compiles from
//   src/simd/math/activations.cc      (silu / swiglu / rms_norm / layer_norm / softmax)
//   include/hyle/simd/dtype.h         (f16 / bf16 codecs, header-only)
// The resulting library lives in oracle/_ref/ and is never committed.
#include <cstddef>
#include <cstdint>

#include "hyle/simd/dtype.h"
#include "src/simd/math/kernels.h"

namespace hs = hyle::simd;
namespace hd = hyle::simd::detail;

extern "C" {

float ref_f16_to_f32(std::uint16_t bits) {
  return hs::f16_to_f32(hs::float16_t::from_bits(bits));
}
std::uint16_t ref_f32_to_f16(float value) { return hs::f32_to_f16(value).bits; }
float ref_bf16_to_f32(std::uint16_t bits) {
  return hs::bf16_to_f32(hs::bfloat16_t::from_bits(bits));
}
std::uint16_t ref_f32_to_bf16(float value) {
  return hs::f32_to_bf16(value).bits;
}

// Bulk forms so exhaustive sweeps do not pay one foreign call per value.
void ref_f16_to_f32_n(const std::uint16_t *src, float *dst, std::size_t n) {
  for (std::size_t i = 0; i < n; ++i)
    dst[i] = hs::f16_to_f32(hs::float16_t::from_bits(src[i]));
}
void ref_f32_to_f16_n(const float *src, std::uint16_t *dst, std::size_t n) {
  for (std::size_t i = 0; i < n; ++i) dst[i] = hs::f32_to_f16(src[i]).bits;
}
void ref_f32_to_bf16_n(const float *src, std::uint16_t *dst, std::size_t n) {
  for (std::size_t i = 0; i < n; ++i) dst[i] = hs::f32_to_bf16(src[i]).bits;
}

void ref_silu_f32(const float *src, float *dst, std::size_t n) {
  hd::silu_f32_scalar(src, dst, n);
}
void ref_silu_f16(const std::uint16_t *src, std::uint16_t *dst, std::size_t n) {
  hd::silu_f16_scalar(reinterpret_cast<const hs::float16_t *>(src),
                      reinterpret_cast<hs::float16_t *>(dst), n);
}
void ref_silu_bf16(const std::uint16_t *src, std::uint16_t *dst,
                   std::size_t n) {
  hd::silu_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(src),
                       reinterpret_cast<hs::bfloat16_t *>(dst), n);
}

void ref_swiglu_f32(const float *gate, const float *value, float *dst,
                    std::size_t n) {
  hd::swiglu_f32_scalar(gate, value, dst, n);
}
void ref_swiglu_f16(const std::uint16_t *gate, const std::uint16_t *value,
                    std::uint16_t *dst, std::size_t n) {
  hd::swiglu_f16_scalar(reinterpret_cast<const hs::float16_t *>(gate),
                        reinterpret_cast<const hs::float16_t *>(value),
                        reinterpret_cast<hs::float16_t *>(dst), n);
}
void ref_swiglu_bf16(const std::uint16_t *gate, const std::uint16_t *value,
                     std::uint16_t *dst, std::size_t n) {
  hd::swiglu_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(gate),
                         reinterpret_cast<const hs::bfloat16_t *>(value),
                         reinterpret_cast<hs::bfloat16_t *>(dst), n);
}

// gelu / gelu_tanh / sigmoid / relu and the gated forms built on them
void ref_gelu_f32(const float *src, float *dst, std::size_t n) { hd::gelu_f32_scalar(src, dst, n); }
void ref_gelu_tanh_f32(const float *src, float *dst, std::size_t n) { hd::gelu_tanh_f32_scalar(src, dst, n); }
void ref_sigmoid_f32(const float *src, float *dst, std::size_t n) { hd::sigmoid_f32_scalar(src, dst, n); }
void ref_relu_f32(const float *src, float *dst, std::size_t n) { hd::relu_f32_scalar(src, dst, n); }
void ref_gelu_f16(const std::uint16_t *src, std::uint16_t *dst, std::size_t n) {
  hd::gelu_f16_scalar(reinterpret_cast<const hs::float16_t *>(src), reinterpret_cast<hs::float16_t *>(dst), n);
}
void ref_gelu_bf16(const std::uint16_t *src, std::uint16_t *dst, std::size_t n) {
  hd::gelu_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(src), reinterpret_cast<hs::bfloat16_t *>(dst), n);
}
void ref_gelu_tanh_f16(const std::uint16_t *src, std::uint16_t *dst, std::size_t n) {
  hd::gelu_tanh_f16_scalar(reinterpret_cast<const hs::float16_t *>(src), reinterpret_cast<hs::float16_t *>(dst), n);
}
void ref_gelu_tanh_bf16(const std::uint16_t *src, std::uint16_t *dst, std::size_t n) {
  hd::gelu_tanh_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(src), reinterpret_cast<hs::bfloat16_t *>(dst), n);
}
void ref_geglu_f32(const float *gate, const float *value, float *dst, std::size_t n) {
  hd::geglu_f32_scalar(gate, value, dst, n);
}
void ref_geglu_tanh_f32(const float *gate, const float *value, float *dst, std::size_t n) {
  hd::geglu_tanh_f32_scalar(gate, value, dst, n);
}
void ref_geglu_bf16(const std::uint16_t *gate, const std::uint16_t *value, std::uint16_t *dst, std::size_t n) {
  hd::geglu_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(gate), reinterpret_cast<const hs::bfloat16_t *>(value),
                        reinterpret_cast<hs::bfloat16_t *>(dst), n);
}
void ref_geglu_tanh_bf16(const std::uint16_t *gate, const std::uint16_t *value, std::uint16_t *dst, std::size_t n) {
  hd::geglu_tanh_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(gate), reinterpret_cast<const hs::bfloat16_t *>(value),
                             reinterpret_cast<hs::bfloat16_t *>(dst), n);
}

void ref_rms_norm_f32(const float *src, const float *weight, float *dst,
                      std::size_t n, float epsilon) {
  hd::rms_norm_f32_scalar(src, weight, dst, n, epsilon);
}
void ref_rms_norm_f16(const std::uint16_t *src, const std::uint16_t *weight,
                      std::uint16_t *dst, std::size_t n, float epsilon) {
  hd::rms_norm_f16_scalar(reinterpret_cast<const hs::float16_t *>(src),
                          reinterpret_cast<const hs::float16_t *>(weight),
                          reinterpret_cast<hs::float16_t *>(dst), n, epsilon);
}
void ref_rms_norm_bf16(const std::uint16_t *src, const std::uint16_t *weight,
                       std::uint16_t *dst, std::size_t n, float epsilon) {
  hd::rms_norm_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(src),
                           reinterpret_cast<const hs::bfloat16_t *>(weight),
                           reinterpret_cast<hs::bfloat16_t *>(dst), n, epsilon);
}

void ref_layer_norm_f32(const float *src, const float *scale, const float *bias, float *dst,
                        std::size_t n, float epsilon) {
  hd::layer_norm_f32_scalar(src, scale, bias, dst, n, epsilon);
}
void ref_layer_norm_f16(const std::uint16_t *src, const std::uint16_t *scale, const std::uint16_t *bias,
                        std::uint16_t *dst, std::size_t n, float epsilon) {
  hd::layer_norm_f16_scalar(reinterpret_cast<const hs::float16_t *>(src),
                            reinterpret_cast<const hs::float16_t *>(scale),
                            reinterpret_cast<const hs::float16_t *>(bias),
                            reinterpret_cast<hs::float16_t *>(dst), n, epsilon);
}
void ref_layer_norm_bf16(const std::uint16_t *src, const std::uint16_t *scale, const std::uint16_t *bias,
                         std::uint16_t *dst, std::size_t n, float epsilon) {
  hd::layer_norm_bf16_scalar(reinterpret_cast<const hs::bfloat16_t *>(src),
                             reinterpret_cast<const hs::bfloat16_t *>(scale),
                             reinterpret_cast<const hs::bfloat16_t *>(bias),
                             reinterpret_cast<hs::bfloat16_t *>(dst), n, epsilon);
}

void ref_softmax_f32(const float *src, float *dst, std::size_t n) {
  hd::softmax_f32_scalar(src, dst, n);
}
void ref_log_softmax_f32(const float *src, float *dst, std::size_t n) {
  hd::log_softmax_f32_scalar(src, dst, n);
}

}  // extern "C"
