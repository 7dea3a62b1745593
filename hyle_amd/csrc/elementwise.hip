// elementwise.hip -- Binary (broadcast), BinaryChain, Unary SiLU and SwiGLU for
// gfx950.  Pure streaming kernels: 128-bit global loads and stores, several
// independent vectors in flight per lane, f32 arithmetic, one rounding per
// stored value.
//
// Semantics follow the reference's CPU native provider:
//   Binary        src/compute_provider_native/elementwise.cc:102-169 (decode ->
//                 f32 op -> one RN-even store), broadcast offsets of
//                 src/compute_provider_native/native_plan.h:152-174
//   SiLU / SwiGLU src/simd/math/activations.cc:21-25,44-47,114-122
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr int kUnroll = 4;

// ---- scalar semantics --------------------------------------------------------
enum : int { kAdd = 0, kSub = 1, kMul = 2, kDiv = 3, kMin = 4, kMax = 5 };

template <int kKind> __device__ __forceinline__ float binary_apply(float x, float y) {
  if constexpr (kKind == kAdd) return x + y;
  else if constexpr (kKind == kSub) return x - y;
  else if constexpr (kKind == kMul) return x * y;
  else if constexpr (kKind == kDiv) return x / y;
  else if constexpr (kKind == kMin) return fminf(x, y);
  else return fmaxf(x, y);
}
__device__ __forceinline__ float binary_apply_rt(int kind, float x, float y) {
  switch (kind) {
    case kAdd: return x + y;
    case kSub: return x - y;
    case kMul: return x * y;
    case kDiv: return x / y;
    case kMin: return fminf(x, y);
    default: return fmaxf(x, y);
  }
}

// Exact form, operation for operation the reference's scalar floor
// (src/simd/math/activations.cc:21-25,44-47): used for f32 storage.
__device__ __forceinline__ float silu_exact(float x) {
  if (x == -INFINITY) return 0.0f;
  float s;
  if (x != x) {
    s = x;
  } else {
    const float e = expf(-fabsf(x));
    s = (x < 0.0f ? e : 1.0f) / (1.0f + e);
  }
  return x * s;
}

// Narrow storage keeps 8 (bf16) or 11 (f16) significand bits, so the sigmoid is
// evaluated as 1 / (1 + exp(-x)) with the hardware exp2 and reciprocal (about
// 1e-6 relative).  exp(-x) is carried scaled by 2^-32 so that it stays finite
// down to x = -110, where silu(x) itself underflows every storage type:
//   sigmoid = 2^-32 / (exp(-x) * 2^-32 + 2^-32).
// The final product is the ordinary one, so a sigmoid that underflowed to zero gives -0 for a
// negative x, as x * sigmoid(x) does in the reference; only x = -inf is singled out (+0 there,
// src/simd/math/activations.cc:44-47, instead of -inf * 0).
__device__ __forceinline__ float times_or_zero_at_minus_inf(float x, float factor) {
  const float product = x * factor;
  return x == -INFINITY ? 0.0f : product;
}
__device__ __forceinline__ float silu_fast(float x) {
  constexpr float kNegLog2e = -1.44269504088896340736f;
  constexpr float kTwoM32 = 2.3283064365386963e-10f;
  const float scaled = __builtin_amdgcn_exp2f(__builtin_fmaf(x, kNegLog2e, -32.0f));
  const float sigmoid = __builtin_amdgcn_rcpf(scaled + kTwoM32) * kTwoM32;
  return times_or_zero_at_minus_inf(x, sigmoid);
}

template <class T> __device__ __forceinline__ float silu_for(float x) {
  if constexpr (Traits<T>::kSize == 4) return silu_exact(x);
  else return silu_fast(x);
}

// Unary kinds (include/hyle/compute/operation.h:57-73) in the scalar forms of the reference:
// src/compute_provider_native/elementwise.cc:30-55 (neg, exp, log, sqrt, rsqrt, tanh, relu, silu),
// src/simd/math/activations.cc:21-47 (sigmoid, gelu, gelu_tanh, silu) and
// tests/compute_provider_native/elementwise_test.cc:43-82 (abs, softplus).
enum : int {
  kAbs = 0, kNeg, kExp, kLog, kSqrt, kRsqrt, kTanh, kSigmoid, kRelu, kGelu, kGeluTanh, kSiluKind, kSoftplus
};

__device__ __forceinline__ float sigmoid_exact(float x) {
  if (x != x) return x;
  const float e = expf(-fabsf(x));
  return x < 0.0f ? e / (1.0f + e) : 1.0f / (1.0f + e);
}
__device__ __forceinline__ float gelu_erf(float x) {
  if (x == -INFINITY) return 0.0f;
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float gelu_tanh(float x) {
  if (x == -INFINITY) return 0.0f;
  const float inner = 0.79788456080286535588f * x * __builtin_fmaf(0.044715f, x * x, 1.0f);
  return 0.5f * x * (1.0f + tanhf(inner));
}
// log1p(exp(x)); the reference evaluates it in double.  max(x, 0) + log1p(exp(-|x|)) is the
// same function without the overflow, good to a few units of f32 in the last place.
__device__ __forceinline__ float softplus(float x) {
  if (x != x) return x;
  return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x)));
}

// Forms for narrow storage (8 or 11 significand bits), built on the hardware exp2 and
// reciprocal like silu_fast; each is good to about 2e-7 of the result's scale, far inside half
// a unit of bf16 / f16, and none of them subtracts nearly equal numbers.
__device__ __forceinline__ float sigmoid_fast(float x) {
  constexpr float kNegLog2e = -1.44269504088896340736f;
  constexpr float kTwoM32 = 2.3283064365386963e-10f;
  const float scaled = __builtin_amdgcn_exp2f(__builtin_fmaf(x, kNegLog2e, -32.0f));
  return __builtin_amdgcn_rcpf(scaled + kTwoM32) * kTwoM32;
}
// 0.5 * (1 + tanh(u)) = sigmoid(2u): the tanh form of GELU without the cancelling 1 + tanh.
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float inner = 0.79788456080286535588f * x * __builtin_fmaf(0.044715f, x * x, 1.0f);
  return times_or_zero_at_minus_inf(x, sigmoid_fast(2.0f * inner));
}
// 1 - erf(z) for z >= 0 is poly(t) * exp(-z^2), t = 1 / (1 + p z) (Abramowitz and Stegun
// 7.1.26, absolute error 1.5e-7); the negative side of 1 + erf is that product itself.
__device__ __forceinline__ float gelu_erf_fast(float x) {
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.0f));
  float poly = __builtin_fmaf(t, 1.061405429f, -1.453152027f);
  poly = __builtin_fmaf(t, poly, 1.421413741f);
  poly = __builtin_fmaf(t, poly, -0.284496736f);
  poly = __builtin_fmaf(t, poly, 0.254829592f);
  const float tail = (poly * t) * __builtin_amdgcn_exp2f(-1.44269504088896340736f * z * z);
  const float one_plus_erf = x < 0.0f ? tail : 2.0f - tail;
  return times_or_zero_at_minus_inf(x, 0.5f * one_plus_erf);
}
template <class T> __device__ __forceinline__ float sigmoid_for(float x) {
  if constexpr (Traits<T>::kSize == 4) return sigmoid_exact(x);
  else return sigmoid_fast(x);
}
template <class T> __device__ __forceinline__ float gelu_for(float x) {
  if constexpr (Traits<T>::kSize == 4) return gelu_erf(x);
  else return gelu_erf_fast(x);
}
template <class T> __device__ __forceinline__ float gelu_tanh_for(float x) {
  if constexpr (Traits<T>::kSize == 4) return gelu_tanh(x);
  else return gelu_tanh_fast(x);
}

template <class T> __device__ __forceinline__ float unary_apply_rt(int kind, float x) {
  switch (kind) {
    case kAbs: return fabsf(x);
    case kNeg: return -x;
    case kExp: return expf(x);
    case kLog: return logf(x);
    case kSqrt: return sqrtf(x);
    case kRsqrt: return 1.0f / sqrtf(x);
    case kTanh: return tanhf(x);
    case kSigmoid: return sigmoid_for<T>(x);
    case kRelu: return x != x ? x : (x > 0.0f ? x : 0.0f);
    case kGelu: return gelu_for<T>(x);
    case kGeluTanh: return gelu_tanh_for<T>(x);
    case kSiluKind: return silu_for<T>(x);
    default: return softplus(x);
  }
}
template <int kKind> struct UnaryFn {
  static constexpr int kInputs = 1;
  template <class T> __device__ __forceinline__ float operator()(T, float x, float, float) const {
    return unary_apply_rt<T>(kKind, x);  // kKind is a constant: the switch folds away
  }
};
// GatedActivationKind (include/hyle/compute/operation.h:91-95): activation(gate) * value.
template <class T> __device__ __forceinline__ float gate_apply_rt(int activation, float g) {
  return activation == 0 ? silu_for<T>(g) : (activation == 1 ? gelu_for<T>(g) : gelu_tanh_for<T>(g));
}
template <int kActivation> struct GatedFn {
  static constexpr int kInputs = 2;
  template <class T> __device__ __forceinline__ float operator()(T, float g, float u, float) const {
    return gate_apply_rt<T>(kActivation, g) * u;
  }
};

template <int kKind> struct BinaryFn {
  static constexpr int kInputs = 2;
  template <class T> __device__ __forceinline__ float operator()(T, float x, float y, float) const {
    return binary_apply<kKind>(x, y);
  }
};
template <int kKind0, int kKind1> struct ChainFn {
  static constexpr int kInputs = 3;
  template <class T> __device__ __forceinline__ float operator()(T, float x, float y, float z) const {
    return binary_apply<kKind1>(Traits<T>::round(binary_apply<kKind0>(x, y)), z);
  }
};
struct SiluFn {
  static constexpr int kInputs = 1;
  template <class T> __device__ __forceinline__ float operator()(T, float x, float, float) const {
    return silu_for<T>(x);
  }
};
struct SwigluFn {
  static constexpr int kInputs = 2;
  template <class T> __device__ __forceinline__ float operator()(T, float g, float u, float) const {
    return silu_for<T>(g) * u;
  }
};
// One functor for the slow routes: the operation is a launch-uniform value.
struct RuntimeFn {
  EwOp op;
  int kind0, kind1;
  template <class T> __device__ __forceinline__ float operator()(T, float x, float y, float z) const {
    switch (op) {
      case EwOp::kBinary: return binary_apply_rt(kind0, x, y);
      case EwOp::kChain:
        return binary_apply_rt(kind1, Traits<T>::round(binary_apply_rt(kind0, x, y)), z);
      case EwOp::kSilu: return silu_for<T>(x);
      case EwOp::kUnary: return unary_apply_rt<T>(kind0, x);
      case EwOp::kGated: return gate_apply_rt<T>(kind0, x) * y;
      default: return silu_for<T>(x) * y;
    }
  }
};

// ---- flat vectorised kernel ----------------------------------------------------
// Operand addressing inside the flat kernels.  `period` is in elements: 0 = the
// operand is as long as the output, 1 = one value for every element, otherwise
// the operand repeats every `period` elements (a dense broadcast suffix).  The
// vectorised kernel needs period % vector width == 0 (`period_vec`).  Element
// counts are at most INT32_MAX, so 32-bit indices suffice.
struct Operand {
  const void *base;
  uint32_t period;
  uint32_t period_vec;
};

template <class T>
__device__ __forceinline__ float fetch1(const Operand &op, uint32_t e) {
  return Traits<T>::load(op.base, op.period ? e % op.period : e);
}

// ---- every input as long as the output -------------------------------------------------
// Each lane handles kUnroll vectors, kThreads apart.  Loads carry no branches (a lane past the
// end reads the last vector and drops it) and no load sits next to its first use:
// kSerial = false issues every load of the lane before the first value is consumed;
// kSerial = true takes the vectors one after another (the loads of vector k + 1 are issued
// while vector k is computed).  Either way the results stay in registers and all stores follow
// the last load, so a block reads in one phase and writes in another.
template <class T, class Fn, int kUnroll, int kThreads, bool kSerial>
__global__ __launch_bounds__(kThreads) void ew_full_vec(const void *a, const void *b, const void *c,
                                                        void *out, uint32_t vectors,
                                                        uint32_t elements, Fn fn) {
  constexpr int kVec = Traits<T>::kVec;
  const uint32_t first = blockIdx.x * (kUnroll * kThreads) + threadIdx.x;
  if (vectors != 0) {
    u32x4 rx[kUnroll], ry[kUnroll], rz[kUnroll], result[kUnroll];
    auto load = [&](int k) {
      const uint32_t vec = first + k * kThreads;
      const uint32_t at = vec < vectors ? vec : vectors - 1;
      rx[k] = load16_stream(a, at);
      if constexpr (Fn::kInputs > 1) ry[k] = load16_stream(b, at);
      if constexpr (Fn::kInputs > 2) rz[k] = load16_stream(c, at);
    };
    auto arrived = [&](int k) {
      loads_issued(rx[k]);
      if constexpr (Fn::kInputs > 1) loads_issued(ry[k]);
      if constexpr (Fn::kInputs > 2) loads_issued(rz[k]);
    };
    auto compute = [&](int k) {
      float x[kVec], y[kVec], z[kVec], r[kVec];
      Traits<T>::unpack(rx[k], x);
      if constexpr (Fn::kInputs > 1) Traits<T>::unpack(ry[k], y);
      if constexpr (Fn::kInputs > 2) Traits<T>::unpack(rz[k], z);
#pragma unroll
      for (int j = 0; j < kVec; ++j)
        r[j] = fn(T{}, x[j], Fn::kInputs > 1 ? y[j] : 0.0f, Fn::kInputs > 2 ? z[j] : 0.0f);
      result[k] = Traits<T>::pack(r);
    };
    if constexpr (kSerial) {
      load(0);
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        arrived(k);
        if (k + 1 < kUnroll) load(k + 1);
        compute(k);
      }
    } else {
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) load(k);
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) arrived(k);
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) compute(k);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const uint32_t vec = first + k * kThreads;
      if (vec < vectors) store16_stream(out, vec, result[k]);
    }
  }
  // elements past the last whole vector
  if (blockIdx.x == 0) {
    const uint32_t e = vectors * kVec + threadIdx.x;
    if (e < elements) {
      const float xs = Traits<T>::load(a, e);
      const float ys = Fn::kInputs > 1 ? Traits<T>::load(b, e) : 0.0f;
      const float zs = Fn::kInputs > 2 ? Traits<T>::load(c, e) : 0.0f;
      Traits<T>::store(out, e, fn(T{}, xs, ys, zs));
    }
  }
}

// ---- broadcast operands (a repeating suffix, a single value) -------------------------------
template <class T>
__device__ __forceinline__ void fetch(const Operand &op, uint32_t vec, float (&v)[Traits<T>::kVec]) {
  constexpr int kVec = Traits<T>::kVec;
  if (op.period == 0) {
    Traits<T>::unpack(load16_stream(op.base, vec), v);
  } else if (op.period == 1) {
    const float s = Traits<T>::load(op.base, 0);
#pragma unroll
    for (int j = 0; j < kVec; ++j) v[j] = s;
  } else {
    Traits<T>::unpack(load16(op.base, vec % op.period_vec), v);
  }
}

// The addressing mode of each operand is a launch-uniform branch around its load and decode,
// so a lane takes its operands one after another; all stores follow the last load.
template <class T, class Fn, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void ew_flat_vec(Operand a, Operand b, Operand c,
                                                        void *out, uint32_t vectors,
                                                        uint32_t elements, Fn fn) {
  constexpr int kVec = Traits<T>::kVec;
  const uint32_t first = blockIdx.x * (kUnroll * kThreads) + threadIdx.x;
  float x[kUnroll][kVec], y[kUnroll][kVec], z[kUnroll][kVec];
#pragma unroll
  for (int k = 0; k < kUnroll; ++k) {
    const uint32_t vec = first + k * kThreads;
    if (vec < vectors) {
      fetch<T>(a, vec, x[k]);
      if constexpr (Fn::kInputs > 1) fetch<T>(b, vec, y[k]);
      if constexpr (Fn::kInputs > 2) fetch<T>(c, vec, z[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < kUnroll; ++k) {
    const uint32_t vec = first + k * kThreads;
    if (vec < vectors) {
      float r[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j)
        r[j] = fn(T{}, x[k][j], Fn::kInputs > 1 ? y[k][j] : 0.0f, Fn::kInputs > 2 ? z[k][j] : 0.0f);
      store16_stream(out, vec, Traits<T>::pack(r));
    }
  }
  // elements past the last whole vector
  if (blockIdx.x == 0) {
    const uint32_t e = vectors * kVec + threadIdx.x;
    if (e < elements) {
      const float xs = fetch1<T>(a, e);
      const float ys = Fn::kInputs > 1 ? fetch1<T>(b, e) : 0.0f;
      const float zs = Fn::kInputs > 2 ? fetch1<T>(c, e) : 0.0f;
      Traits<T>::store(out, e, fn(T{}, xs, ys, zs));
    }
  }
}

// Same addressing, one element per lane: used when a pointer is not 16-byte
// aligned or a period is not a whole number of vectors.
template <class T>
__global__ __launch_bounds__(kBlockThreads) void ew_flat_scalar(Operand a, Operand b, Operand c,
                                                                void *out, uint32_t elements,
                                                                int inputs, RuntimeFn fn) {
  const uint32_t e = blockIdx.x * kBlockThreads + threadIdx.x;
  if (e >= elements) return;
  const float xs = fetch1<T>(a, e);
  const float ys = inputs > 1 ? fetch1<T>(b, e) : 0.0f;
  const float zs = inputs > 2 ? fetch1<T>(c, e) : 0.0f;
  Traits<T>::store(out, e, fn(T{}, xs, ys, zs));
}

// ---- general strided kernel ------------------------------------------------------
struct GeneralLayout {
  int32_t rank;
  uint32_t dims[kMaxRank];
  int64_t strides[3][kMaxRank];
};

template <class T>
__global__ __launch_bounds__(kBlockThreads) void ew_general(const char *a, const char *b,
                                                            const char *c, void *out,
                                                            uint64_t elements, int inputs,
                                                            GeneralLayout layout, RuntimeFn fn) {
  const uint64_t e = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (e >= elements) return;
  uint64_t rest = e;
  int64_t off[3] = {0, 0, 0};
  for (int axis = layout.rank - 1; axis >= 0; --axis) {
    const uint32_t extent = layout.dims[axis];
    const uint64_t coordinate = rest % extent;
    rest /= extent;
    off[0] += (int64_t)coordinate * layout.strides[0][axis];
    off[1] += (int64_t)coordinate * layout.strides[1][axis];
    off[2] += (int64_t)coordinate * layout.strides[2][axis];
  }
  const float xs = Traits<T>::load(a + off[0], 0);
  const float ys = inputs > 1 ? Traits<T>::load(b + off[1], 0) : 0.0f;
  const float zs = inputs > 2 ? Traits<T>::load(c + off[2], 0) : 0.0f;
  Traits<T>::store(out, e, fn(T{}, xs, ys, zs));
}

// ---- packed gated activation: rows of [gate | value] -----------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(kBlockThreads) void swiglu_packed_vec(const void *packed, void *out,
                                                                   uint32_t row_vectors,
                                                                   uint64_t vectors, int activation) {
  constexpr int kVec = Traits<T>::kVec;
  const uint64_t first = (uint64_t)blockIdx.x * (kUnroll * kBlockThreads) + threadIdx.x;
  float g[kUnroll][kVec], u[kUnroll][kVec];
#pragma unroll
  for (int k = 0; k < kUnroll; ++k) {
    const uint64_t vec = first + (uint64_t)k * kBlockThreads;
    if (vec < vectors) {
      const uint64_t row = vec / row_vectors, col = vec % row_vectors;
      Traits<T>::unpack(load16_stream(packed, row * 2 * row_vectors + col), g[k]);
      Traits<T>::unpack(load16_stream(packed, row * 2 * row_vectors + row_vectors + col), u[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < kUnroll; ++k) {
    const uint64_t vec = first + (uint64_t)k * kBlockThreads;
    if (vec < vectors) {
      float r[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j) r[j] = gate_apply_rt<T>(activation, g[k][j]) * u[k][j];
      store16_stream(out, vec, Traits<T>::pack(r));
    }
  }
}

template <class T>
__global__ __launch_bounds__(kBlockThreads) void swiglu_packed_scalar(const void *packed, void *out,
                                                                      uint32_t hidden,
                                                                      uint64_t elements, int activation) {
  const uint64_t e = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (e >= elements) return;
  const uint64_t row = e / hidden, col = e % hidden;
  const float g = Traits<T>::load(packed, row * 2 * hidden + col);
  const float u = Traits<T>::load(packed, row * 2 * hidden + hidden + col);
  Traits<T>::store(out, e, gate_apply_rt<T>(activation, g) * u);
}

// ---- host dispatch -------------------------------------------------------------------
Operand make_operand(const void *base, uint32_t period, int vec) {
  Operand op;
  op.base = base;
  op.period = period;
  op.period_vec = (period > 1 && period % vec == 0) ? period / vec : 0;
  return op;
}

// ew_full: every operand as long as the output; ew_flat: some operand periodic (a dense broadcast
// suffix) or a scalar.  <vectors per lane>x<threads per block>[/serial: one vector after another]
template <int kUnroll, int kThreads, int kForm> struct EwTag {  // kForm: 0 flat, 1 full with the vectors in flight at once, 2 full serial
  static std::string text() {
    return std::string(kForm == 0 ? "ew_flat/" : "ew_full/") + std::to_string(kUnroll) + "x" + std::to_string(kThreads) +
           (kForm == 2 ? "/serial" : (kForm == 1 ? "/batched" : ""));
  }
};
struct EwScalarTag {
  static std::string text() { return "ew_flat_scalar"; }
};
struct EwGeneralTag {
  static std::string text() { return "ew_general"; }
};
template <bool kVector> struct PackedTag {
  static std::string text() { return kVector ? "gated_packed/vector" : "gated_packed/scalar"; }
};

template <class T, class Fn, int kUnroll, int kThreads, bool kSerial>
hipError_t run_full_as(const EwFlat &p, Operand a, Operand b, Operand c, void *out, hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const uint64_t vectors = p.elements / kVec;
  const uint64_t per_block = (uint64_t)kUnroll * kThreads;
  uint64_t blocks = (vectors + per_block - 1) / per_block;
  if (blocks == 0) blocks = 1;  // the tail still needs block 0
  note_variant<EwTag<kUnroll, kThreads, kSerial ? 2 : 1>>();
  hipLaunchKernelGGL((ew_full_vec<T, Fn, kUnroll, kThreads, kSerial>), dim3((uint32_t)blocks),
                     dim3(kThreads), 0, s, a.base, b.base, c.base, out, (uint32_t)vectors,
                     (uint32_t)p.elements, Fn{});
  return hipGetLastError();
}

template <class T, class Fn, int kUnroll, int kThreads = kBlockThreads>
hipError_t run_flat_as(const EwFlat &p, Operand a, Operand b, Operand c, void *out, hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const uint64_t vectors = p.elements / kVec;
  const uint64_t per_block = (uint64_t)kUnroll * kThreads;
  uint64_t blocks = (vectors + per_block - 1) / per_block;
  if (blocks == 0) blocks = 1;  // the tail still needs block 0
  note_variant<EwTag<kUnroll, kThreads, 0>>();
  hipLaunchKernelGGL((ew_flat_vec<T, Fn, kUnroll, kThreads>), dim3((uint32_t)blocks), dim3(kThreads), 0, s,
                     a, b, c, out, (uint32_t)vectors, (uint32_t)p.elements, Fn{});
  return hipGetLastError();
}

// Launch shape from the HBM traffic of the launch (streams as long as the output, the output
// included), as measured on MI355X.  Inputs all as long as the output: R[8192,2048] += Y bf16
// (101 MB) takes 16.5 us with 8 vectors per lane taken serially in blocks of 512 threads,
// against 17.1 (4 at once, 256 threads) and 17.8 (1 vector per lane); SwiGLU over [8192,6144]
// bf16 (302 MB) takes 46.9 us with 4 vectors at once against 47.5 (1 vector) and 49-53 for the
// serial forms.  With broadcast operands: (A[4096,2048] + b) * s f32 (67 MB) takes 11.3 us
// with 4 vectors per lane in blocks of 1024 threads against 11.8 (256 threads) and 12.9
// (8 vectors).
template <class T, class Fn>
hipError_t run_vec(const EwFlat &p, Operand a, Operand b, Operand c, void *out, hipStream_t s) {
  uint64_t streams = 1;  // the output
  bool all_full = true;
  for (int i = 0; i < p.inputs; ++i) {
    streams += p.period[i] == 0 ? 1 : 0;
    all_full = all_full && p.period[i] == 0;
  }
  const uint64_t traffic = streams * p.elements * Traits<T>::kSize;
  if (!all_full) {
    if (traffic > (80ull << 20)) return run_flat_as<T, Fn, 1, 256>(p, a, b, c, out, s);
    return run_flat_as<T, Fn, 4, 1024>(p, a, b, c, out, s);
  }
  if (traffic > (110ull << 20)) return run_full_as<T, Fn, 4, 256, false>(p, a, b, c, out, s);
  if (traffic > (48ull << 20)) return run_full_as<T, Fn, 8, 512, true>(p, a, b, c, out, s);
  return run_full_as<T, Fn, 4, 512, true>(p, a, b, c, out, s);
}

template <class T, int kKind0>
hipError_t run_chain(const EwFlat &p, Operand a, Operand b, Operand c, void *out, hipStream_t s) {
  switch (p.kind1) {
    case kAdd: return run_vec<T, ChainFn<kKind0, kAdd>>(p, a, b, c, out, s);
    case kSub: return run_vec<T, ChainFn<kKind0, kSub>>(p, a, b, c, out, s);
    case kMul: return run_vec<T, ChainFn<kKind0, kMul>>(p, a, b, c, out, s);
    default: return hipErrorInvalidValue;
  }
}

template <class T>
hipError_t run_flat(const EwFlat &p, const void *a, const void *b, const void *c, void *out,
                    bool vectorised, hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const Operand oa = make_operand(a, p.period[0], kVec);
  const Operand ob = make_operand(b, p.period[1], kVec);
  const Operand oc = make_operand(c, p.period[2], kVec);
  const bool chain_fast = p.op != EwOp::kChain || (p.kind0 <= kMul && p.kind1 <= kMul);
  bool whole_vectors = true;
  for (int i = 0; i < p.inputs; ++i)
    whole_vectors = whole_vectors && (p.period[i] <= 1 || p.period[i] % kVec == 0);
  if (!vectorised || !chain_fast || !whole_vectors) {
    const uint64_t blocks = (p.elements + kBlockThreads - 1) / kBlockThreads;
    note_variant<EwScalarTag>();
    hipLaunchKernelGGL((ew_flat_scalar<T>), dim3((uint32_t)blocks), dim3(kBlockThreads), 0, s, oa,
                       ob, oc, out, (uint32_t)p.elements, (int)p.inputs,
                       RuntimeFn{p.op, (int)p.kind0, (int)p.kind1});
    return hipGetLastError();
  }
  switch (p.op) {
    case EwOp::kBinary:
      switch (p.kind0) {
        case kAdd: return run_vec<T, BinaryFn<kAdd>>(p, oa, ob, oc, out, s);
        case kSub: return run_vec<T, BinaryFn<kSub>>(p, oa, ob, oc, out, s);
        case kMul: return run_vec<T, BinaryFn<kMul>>(p, oa, ob, oc, out, s);
        case kDiv: return run_vec<T, BinaryFn<kDiv>>(p, oa, ob, oc, out, s);
        case kMin: return run_vec<T, BinaryFn<kMin>>(p, oa, ob, oc, out, s);
        case kMax: return run_vec<T, BinaryFn<kMax>>(p, oa, ob, oc, out, s);
        default: return hipErrorInvalidValue;
      }
    case EwOp::kChain:
      switch (p.kind0) {
        case kAdd: return run_chain<T, kAdd>(p, oa, ob, oc, out, s);
        case kSub: return run_chain<T, kSub>(p, oa, ob, oc, out, s);
        case kMul: return run_chain<T, kMul>(p, oa, ob, oc, out, s);
        default: return hipErrorInvalidValue;
      }
    case EwOp::kSilu: return run_vec<T, SiluFn>(p, oa, ob, oc, out, s);
    case EwOp::kSwiglu: return run_vec<T, SwigluFn>(p, oa, ob, oc, out, s);
    case EwOp::kUnary:
      switch (p.kind0) {
        case kAbs: return run_vec<T, UnaryFn<kAbs>>(p, oa, ob, oc, out, s);
        case kNeg: return run_vec<T, UnaryFn<kNeg>>(p, oa, ob, oc, out, s);
        case kExp: return run_vec<T, UnaryFn<kExp>>(p, oa, ob, oc, out, s);
        case kLog: return run_vec<T, UnaryFn<kLog>>(p, oa, ob, oc, out, s);
        case kSqrt: return run_vec<T, UnaryFn<kSqrt>>(p, oa, ob, oc, out, s);
        case kRsqrt: return run_vec<T, UnaryFn<kRsqrt>>(p, oa, ob, oc, out, s);
        case kTanh: return run_vec<T, UnaryFn<kTanh>>(p, oa, ob, oc, out, s);
        case kSigmoid: return run_vec<T, UnaryFn<kSigmoid>>(p, oa, ob, oc, out, s);
        case kRelu: return run_vec<T, UnaryFn<kRelu>>(p, oa, ob, oc, out, s);
        case kGelu: return run_vec<T, UnaryFn<kGelu>>(p, oa, ob, oc, out, s);
        case kGeluTanh: return run_vec<T, UnaryFn<kGeluTanh>>(p, oa, ob, oc, out, s);
        case kSoftplus: return run_vec<T, UnaryFn<kSoftplus>>(p, oa, ob, oc, out, s);
        default: return hipErrorInvalidValue;
      }
    case EwOp::kGated:
      if (p.kind0 == 1) return run_vec<T, GatedFn<1>>(p, oa, ob, oc, out, s);
      if (p.kind0 == 2) return run_vec<T, GatedFn<2>>(p, oa, ob, oc, out, s);
      return hipErrorInvalidValue;
  }
  return hipErrorInvalidValue;
}

template <class T>
hipError_t run_general(const EwGeneral &p, const void *a, const void *b, const void *c, void *out,
                       hipStream_t s) {
  GeneralLayout layout;
  layout.rank = p.rank;
  for (int i = 0; i < kMaxRank; ++i) {
    layout.dims[i] = p.dims[i];
    for (int k = 0; k < 3; ++k) layout.strides[k][i] = p.strides[k][i];
  }
  const uint64_t blocks = (p.elements + kBlockThreads - 1) / kBlockThreads;
  note_variant<EwGeneralTag>();
  hipLaunchKernelGGL((ew_general<T>), dim3((uint32_t)blocks), dim3(kBlockThreads), 0, s,
                     static_cast<const char *>(a), static_cast<const char *>(b),
                     static_cast<const char *>(c), out, p.elements, (int)p.inputs, layout,
                     RuntimeFn{p.op, (int)p.kind0, (int)p.kind1});
  return hipGetLastError();
}

template <class T>
hipError_t run_packed(const EwPacked &p, const void *packed, void *out, bool vectorised,
                      hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  const uint64_t elements = p.rows * p.hidden;
  if (vectorised && p.hidden % kVec == 0) {
    const uint64_t vectors = elements / kVec;
    const uint64_t per_block = (uint64_t)kUnroll * kBlockThreads;
    note_variant<PackedTag<true>>();
    hipLaunchKernelGGL((swiglu_packed_vec<T>), dim3((uint32_t)((vectors + per_block - 1) / per_block)),
                       dim3(kBlockThreads), 0, s, packed, out, p.hidden / kVec, vectors, (int)p.activation);
  } else {
    note_variant<PackedTag<false>>();
    hipLaunchKernelGGL((swiglu_packed_scalar<T>),
                       dim3((uint32_t)((elements + kBlockThreads - 1) / kBlockThreads)),
                       dim3(kBlockThreads), 0, s, packed, out, p.hidden, elements, (int)p.activation);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_ew_flat(Elem type, const EwFlat &p, const void *a, const void *b, const void *c,
                          void *out, bool vectorised, hipStream_t stream) {
  if (p.elements == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_flat<F32>(p, a, b, c, out, vectorised, stream);
    case Elem::kF16: return run_flat<F16>(p, a, b, c, out, vectorised, stream);
    case Elem::kBF16: return run_flat<BF16>(p, a, b, c, out, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_ew_general(Elem type, const EwGeneral &p, const void *a, const void *b,
                             const void *c, void *out, hipStream_t stream) {
  if (p.elements == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_general<F32>(p, a, b, c, out, stream);
    case Elem::kF16: return run_general<F16>(p, a, b, c, out, stream);
    case Elem::kBF16: return run_general<BF16>(p, a, b, c, out, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_swiglu_packed(Elem type, const EwPacked &p, const void *packed, void *out,
                                bool vectorised, hipStream_t stream) {
  if (p.rows == 0 || p.hidden == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_packed<F32>(p, packed, out, vectorised, stream);
    case Elem::kF16: return run_packed<F16>(p, packed, out, vectorised, stream);
    case Elem::kBF16: return run_packed<BF16>(p, packed, out, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
