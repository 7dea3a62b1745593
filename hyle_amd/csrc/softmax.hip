// softmax.hip -- row Softmax / LogSoftmax with scale and broadcast mask, and
// last-axis Reduce (sum, mean, min, max) for gfx950.
//
// Softmax reads every row from HBM once: the row lives in registers across the
// max reduction, the exponential pass and the normalised store.  Semantics are
// those of the reference's CPU path
// (src/compute_provider_native/transformer.cc:44-57,165-191 and
//  src/simd/math/activations.cc:177-192,301-340):
//   v = x * scale; Boolean mask 0 -> -inf; additive mask -> v + mask;
//   a row holding a NaN or +inf, or no finite value at all, becomes all NaN;
//   otherwise out = exp(v - max) / sum, with masked lanes exactly 0.
// The exponential sum is accumulated in f32 (the reference's scalar floor uses
// double); the exponentials are carried scaled by 2^32 and the scale is folded
// into the normaliser, so results down to the smallest subnormal are produced by
// an ordinary multiply instead of being flushed by the hardware exp2.
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

// Rows are taken in storage order.  A mask broadcast over leading axes (a [q, k] mask under
// [heads, q, k]) is re-read by every head; the FETCH_SIZE counter shows those re-reads never
// reach HBM (the mask's 16 MiB are fetched once per launch), and steering the heads of one
// mask row onto one XCD changed neither the counter nor the run time, so there is no such
// remapping here.
//
// Loads carry no branches: a lane outside the row (or a row outside the tensor) reads a clamped,
// valid address and discards the value, so all kVpl loads of a lane are in flight together.
// Under a Boolean mask the mask words are read first and a vector whose elements are all masked
// is not loaded at all: its values cannot reach the result (masked -> -inf before anything looks
// at x, src/compute_provider_native/transformer.cc:44-57), so a causal mask saves half the reads.
template <class T, int kLanes, int kVpl, int kThreads, int kMask, bool kLog>
__global__ __launch_bounds__(kThreads) void softmax_rows(const void *x, const void *mask, void *y,
                                                         uint32_t rows, uint32_t row_vectors,
                                                         float scale, MaskRows mrows) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kWords = kVec / 4;  // mask bytes of one vector, as 32-bit words
  constexpr int kRowsPerBlock = kThreads / kLanes;
  constexpr int kWaves = kThreads / kWaveLanes;
  __shared__ float joint_max[kWaves], joint_sum[kWaves];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t row = blockIdx.x * kRowsPerBlock + threadIdx.x / kLanes;
  const bool row_ok = row < rows;
  const uint32_t row_clamped = row_ok ? row : rows - 1;
  const size_t row_base = (size_t)row_clamped * row_vectors;
  const char *mask_row = nullptr;
  if (kMask != kMaskNone) mask_row = static_cast<const char *>(mask) + mask_row_offset(mrows, row_clamped);

  float v[kVpl][kVec];
  bool ok[kVpl];
  uint32_t vec[kVpl];
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    const uint32_t wanted = lane + k * kLanes;
    ok[k] = row_ok && wanted < row_vectors;
    vec[k] = wanted < row_vectors ? wanted : row_vectors - 1;
  }

  // ---- load, scale, mask ------------------------------------------------------
  if constexpr (kMask == kMaskBoolean) {
    uint32_t bits[kVpl][kWords];
    if (mrows.inner_stride == 0) {
      const uint32_t one = *reinterpret_cast<const uint8_t *>(mask_row) ? 0x01010101u : 0u;
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int q = 0; q < kWords; ++q) bits[k][q] = one;
    } else {
      const uint32_t *words = reinterpret_cast<const uint32_t *>(mask_row);
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int q = 0; q < kWords; ++q) bits[k][q] = words[(size_t)vec[k] * kWords + q];
    }
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      uint32_t any = 0;
#pragma unroll
      for (int q = 0; q < kWords; ++q) {
        bits[k][q] = ok[k] ? bits[k][q] : 0u;
        any |= bits[k][q];
      }
      if (any != 0) {
        Traits<T>::unpack(load16_stream(x, row_base + vec[k]), v[k]);
      } else {
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[k][j] = 0.0f;
      }
    }
#pragma unroll
    for (int k = 0; k < kVpl; ++k)
#pragma unroll
      for (int j = 0; j < kVec; ++j) {
        const bool keep = ((bits[k][j / 4] >> (8 * (j % 4))) & 0xFFu) != 0;
        v[k][j] = keep ? v[k][j] * scale : -INFINITY;
      }
  } else {
#pragma unroll
    for (int k = 0; k < kVpl; ++k) Traits<T>::unpack(load16_stream(x, row_base + vec[k]), v[k]);
    if constexpr (kMask == kMaskAdditive) {
      float m[kVpl][kVec];
      if (mrows.inner_stride == 0) {
        const float one = Traits<T>::load(mask_row, 0);
#pragma unroll
        for (int k = 0; k < kVpl; ++k)
#pragma unroll
          for (int j = 0; j < kVec; ++j) m[k][j] = one;
      } else {
#pragma unroll
        for (int k = 0; k < kVpl; ++k) Traits<T>::unpack(load16(mask_row, vec[k]), m[k]);
      }
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[k][j] = ok[k] ? v[k][j] * scale + m[k][j] : -INFINITY;
    } else {
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[k][j] = ok[k] ? v[k][j] * scale : -INFINITY;
    }
  }

  // ---- row maximum and validity -------------------------------------------------
  // A NaN or +inf anywhere makes the row undefined.  fmaxf never lets a NaN through, so a lane
  // that met one reports +inf instead: after the reduction an infinite maximum of either sign
  // (+inf: poisoned, -inf: nothing finite and unmasked) marks the row.
  float peak = -INFINITY;
  bool poisoned = false;
#pragma unroll
  for (int k = 0; k < kVpl; ++k)
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      poisoned = poisoned || poisons_row(v[k][j]);
      peak = fmaxf(peak, v[k][j]);
    }
  peak = row_max<kLanes>(poisoned ? INFINITY : peak, joint_max);
  const bool invalid = __builtin_fabsf(peak) == INFINITY;

  // ---- exponentials and their sum -------------------------------------------------
  float total = 0.0f;
#pragma unroll
  for (int k = 0; k < kVpl; ++k)
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const float shifted = v[k][j] - peak;
      if constexpr (kLog) {
        total += exp_scaled(shifted);
        v[k][j] = shifted;
      } else {
        v[k][j] = exp_scaled(shifted);
        total += v[k][j];
      }
    }
  total = row_sum<kLanes>(total, joint_sum);  // = 2^32 * sum(exp)

  // ---- normalise and store ------------------------------------------------------------
  // softmax: e * 2^32 * (1 / (sum * 2^32)).  log-softmax: (v - max) - log(sum).
  // An undefined row gets a NaN normaliser: it turns every lane, masked zeros included,
  // into NaN without a per-element select.
  float normaliser = kLog ? (logf(total) - 32.0f * 0.69314718055994530942f) : 1.0f / total;
  if (invalid) normaliser = __builtin_nanf("");
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    if (ok[k]) {
      float r[kVec];
#pragma unroll
      for (int j = 0; j < kVec; ++j) r[j] = kLog ? v[k][j] - normaliser : v[k][j] * normaliser;
      store16_stream(y, (size_t)row * row_vectors + vec[k], Traits<T>::pack(r));
    }
  }
}

// ---- any axis, any strides: one block per (outer, inner) row, three passes ----------
struct GeneralLayout {
  int32_t rank, axis;
  uint32_t dims[kMaxRank];
  int64_t in_strides[kMaxRank];
  int64_t mask_strides[kMaxRank];
  uint32_t inner;
};

template <class T>
__device__ __forceinline__ float general_value(const char *x, const char *mask,
                                               const GeneralLayout &g, uint32_t outer,
                                               uint32_t inner, uint32_t column, float scale,
                                               int mask_kind) {
  // logical index = (outer * width + column) * inner_count + inner, decoded axis by axis
  int64_t in_off = 0, mask_off = 0;
  uint32_t rest_inner = inner, rest_outer = outer;
  for (int axis = g.rank - 1; axis >= 0; --axis) {
    uint32_t coordinate;
    if (axis > g.axis) {
      coordinate = rest_inner % g.dims[axis];
      rest_inner /= g.dims[axis];
    } else if (axis == g.axis) {
      coordinate = column;
    } else {
      coordinate = rest_outer % g.dims[axis];
      rest_outer /= g.dims[axis];
    }
    in_off += (int64_t)coordinate * g.in_strides[axis];
    mask_off += (int64_t)coordinate * g.mask_strides[axis];
  }
  float v = Traits<T>::load(x + in_off, 0) * scale;
  if (mask_kind == kMaskBoolean)
    v = *reinterpret_cast<const uint8_t *>(mask + mask_off) ? v : -INFINITY;
  else if (mask_kind == kMaskAdditive)
    v = v + Traits<T>::load(mask + mask_off, 0);
  return v;
}

template <class T>
__global__ __launch_bounds__(kBlockThreads) void softmax_general(const char *x, const char *mask,
                                                                 void *y, uint32_t width,
                                                                 float scale, int mask_kind,
                                                                 int log_form, GeneralLayout g) {
  constexpr int kWaves = kBlockThreads / kWaveLanes;
  __shared__ float joint_max[kWaves], joint_bad[kWaves], joint_sum[kWaves];
  const uint32_t outer = blockIdx.x / g.inner, inner = blockIdx.x % g.inner;
  float peak = -INFINITY, bad = 0.0f;
  for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads) {
    const float e = general_value<T>(x, mask, g, outer, inner, c, scale, mask_kind);
    bad = (e != e || e == INFINITY) ? 1.0f : bad;
    peak = e > peak ? e : peak;
  }
  peak = row_max<kBlockThreads>(peak, joint_max);
  bad = row_max<kBlockThreads>(bad, joint_bad);
  const bool invalid = bad != 0.0f || peak == -INFINITY;
  float total = 0.0f;
  for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads)
    total += exp_scaled(general_value<T>(x, mask, g, outer, inner, c, scale, mask_kind) - peak);
  total = row_sum<kBlockThreads>(total, joint_sum);
  const float normaliser = log_form ? (logf(total) - 32.0f * 0.69314718055994530942f) : 1.0f / total;
  // every read of this row is complete: an exact input alias may now be overwritten
  __syncthreads();
  for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads) {
    const float shifted = general_value<T>(x, mask, g, outer, inner, c, scale, mask_kind) - peak;
    const float value = log_form ? shifted - normaliser : exp_scaled(shifted) * normaliser;
    const size_t logical = ((size_t)outer * width + c) * g.inner + inner;
    Traits<T>::store(y, logical, invalid ? __builtin_nanf("") : value);
  }
}

// ---- last-axis Reduce -------------------------------------------------------------------
enum : int { kSum = 0, kMean = 1, kMinimum = 2, kMaximum = 3 };

template <int kKind> __device__ __forceinline__ float reduce_identity() {
  return kKind == kMinimum ? INFINITY : kKind == kMaximum ? -INFINITY : 0.0f;
}
template <int kKind> __device__ __forceinline__ float reduce_step(float acc, float v) {
  if constexpr (kKind == kMinimum) return min_propagate(acc, v);
  else if constexpr (kKind == kMaximum) return max_propagate(acc, v);
  else return acc + v;
}

template <class T, int kKind, int kLanes, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void reduce_rows(const void *x, void *y, uint32_t rows,
                                                             uint32_t width) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kRowsPerBlock = kBlockThreads / kLanes;
  __shared__ float joint[4];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t row = blockIdx.x * kRowsPerBlock + threadIdx.x / kLanes;
  const bool row_ok = row < rows;
  float acc = reduce_identity<kKind>();
  if (row_ok) {
    if constexpr (kVector) {
      const uint32_t vectors = width / kVec;
      const size_t base = (size_t)row * vectors;
      for (uint32_t vec = lane; vec < vectors; vec += kLanes) {
        float v[kVec];
        Traits<T>::unpack(load16_stream(x, base + vec), v);
#pragma unroll
        for (int j = 0; j < kVec; ++j) acc = reduce_step<kKind>(acc, v[j]);
      }
    } else {
      const size_t base = (size_t)row * width;
      for (uint32_t i = lane; i < width; i += kLanes)
        acc = reduce_step<kKind>(acc, Traits<T>::load(x, base + i));
    }
  }
  auto combine = [](LaneF32 a, LaneF32 b) { return LaneF32{reduce_step<kKind>(a.x, b.x)}; };
  acc = group_reduce<(kLanes < kWaveLanes ? kLanes : kWaveLanes)>(LaneF32{acc}, combine).x;
  if constexpr (kLanes > kWaveLanes) {
    if ((threadIdx.x & (kWaveLanes - 1)) == 0) joint[threadIdx.x / kWaveLanes] = acc;
    __syncthreads();
    acc = reduce_step<kKind>(reduce_step<kKind>(joint[0], joint[1]),
                             reduce_step<kKind>(joint[2], joint[3]));
  }
  if (row_ok && lane == 0) {
    if constexpr (kKind == kMean) acc = width == 0 ? __builtin_nanf("") : acc / (float)width;
    Traits<T>::store(y, row, acc);
  }
}

// ---- host dispatch ----------------------------------------------------------------------------
template <class T, int kLanes, int kVpl, int kThreads, int kMask, bool kLog>
hipError_t run_rows_as(const SoftmaxParams &p, const void *x, const void *mask, void *y,
                       hipStream_t s) {
  constexpr int kRowsPerBlock = kThreads / kLanes;
  const uint32_t rows = (uint32_t)p.shape.rows;
  const uint32_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  MaskRows m{};
  m.outer_rank = p.outer_rank;
  for (int i = 0; i < kMaxRank; ++i) {
    m.outer_dims[i] = p.outer_dims[i];
    m.outer_strides[i] = p.mask_outer_strides[i];
  }
  m.inner_stride = p.mask_inner_stride;
  hipLaunchKernelGGL((softmax_rows<T, kLanes, kVpl, kThreads, kMask, kLog>), dim3(blocks),
                     dim3(kThreads), 0, s, x, mask, y, rows, p.shape.width / Traits<T>::kVec, p.scale, m);
  return hipGetLastError();
}

template <class T, int kLanes, int kVpl, int kThreads = kBlockThreads>
hipError_t run_rows(const SoftmaxParams &p, const void *x, const void *mask, void *y,
                    hipStream_t s) {
  const bool log_form = p.log;
  switch ((int)p.mask_kind) {
    case kMaskBoolean:
      return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskBoolean, true>(p, x, mask, y, s)
                      : run_rows_as<T, kLanes, kVpl, kThreads, kMaskBoolean, false>(p, x, mask, y, s);
    case kMaskAdditive:
      return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskAdditive, true>(p, x, mask, y, s)
                      : run_rows_as<T, kLanes, kVpl, kThreads, kMaskAdditive, false>(p, x, mask, y, s);
    default:
      return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskNone, true>(p, x, mask, y, s)
                      : run_rows_as<T, kLanes, kVpl, kThreads, kMaskNone, false>(p, x, mask, y, s);
  }
}

template <class T>
hipError_t run_softmax(const SoftmaxParams &p, const void *x, const void *mask, void *y,
                       hipStream_t s) {
  const uint32_t vectors = p.shape.width / Traits<T>::kVec;
  if (vectors <= 8) return run_rows<T, 8, 1>(p, x, mask, y, s);
  if (vectors <= 16) return run_rows<T, 16, 1>(p, x, mask, y, s);
  if (vectors <= 32) return run_rows<T, 32, 1>(p, x, mask, y, s);
  if (vectors <= 64) return run_rows<T, 64, 1>(p, x, mask, y, s);
  if (vectors <= 128) return run_rows<T, 64, 2>(p, x, mask, y, s);
  if (vectors <= 256) return run_rows<T, 128, 2>(p, x, mask, y, s);
  if (vectors <= 512) return run_rows<T, 256, 2>(p, x, mask, y, s);
  // Measured on MI355X for S[32,4096,4096] f32 (1024 vectors per row), us per launch.  Every
  // vector loaded (no mask, additive mask): eight waves x 2 vectors per lane, one row per block
  // 685; two waves x 8 vectors 706-737; four waves x 4 vectors 731; a plain copy in the same
  // shapes 688-737.  Boolean causal mask, masked vectors not loaded: four waves x 4 vectors,
  // two rows per block 523; eight waves x 2 vectors 581; two waves x 8 vectors 569-591.
  if (vectors <= 1024) {
    if ((int)p.mask_kind == kMaskBoolean) return run_rows<T, 256, 4, 512>(p, x, mask, y, s);
    return run_rows<T, 512, 2, 512>(p, x, mask, y, s);
  }
  if (vectors <= 2048) return run_rows<T, 512, 4, 512>(p, x, mask, y, s);
  if (vectors <= 4096) return run_rows<T, 1024, 4, 1024>(p, x, mask, y, s);
  return run_rows<T, 1024, 8, 1024>(p, x, mask, y, s);
}

template <class T>
hipError_t run_general(const SoftmaxGeneralParams &p, const void *x, const void *mask, void *y,
                       hipStream_t s) {
  GeneralLayout g{};
  g.rank = p.rank;
  g.axis = p.axis;
  g.inner = (uint32_t)p.inner;
  for (int i = 0; i < kMaxRank; ++i) {
    g.dims[i] = p.dims[i];
    g.in_strides[i] = p.in_strides[i];
    g.mask_strides[i] = p.mask_strides[i];
  }
  hipLaunchKernelGGL((softmax_general<T>), dim3((uint32_t)(p.outer * p.inner)), dim3(kBlockThreads),
                     0, s, static_cast<const char *>(x), static_cast<const char *>(mask), y, p.width,
                     p.scale, (int)p.mask_kind, p.log ? 1 : 0, g);
  return hipGetLastError();
}

template <class T, int kKind>
hipError_t run_reduce_kind(const ReduceParams &p, const void *x, void *y, bool vectorised,
                           hipStream_t s) {
  const uint32_t rows = (uint32_t)p.shape.rows, width = p.shape.width;
  const bool vec = vectorised && width % Traits<T>::kVec == 0;
  const bool wide = (size_t)width * Traits<T>::kSize >= 8192;
  if (wide) {
    if (vec)
      hipLaunchKernelGGL((reduce_rows<T, kKind, kBlockThreads, true>), dim3(rows),
                         dim3(kBlockThreads), 0, s, x, y, rows, width);
    else
      hipLaunchKernelGGL((reduce_rows<T, kKind, kBlockThreads, false>), dim3(rows),
                         dim3(kBlockThreads), 0, s, x, y, rows, width);
  } else {
    const uint32_t blocks = (rows + 3) / 4;
    if (vec)
      hipLaunchKernelGGL((reduce_rows<T, kKind, kWaveLanes, true>), dim3(blocks),
                         dim3(kBlockThreads), 0, s, x, y, rows, width);
    else
      hipLaunchKernelGGL((reduce_rows<T, kKind, kWaveLanes, false>), dim3(blocks),
                         dim3(kBlockThreads), 0, s, x, y, rows, width);
  }
  return hipGetLastError();
}

template <class T>
hipError_t run_reduce(const ReduceParams &p, const void *x, void *y, bool vectorised,
                      hipStream_t s) {
  switch (p.kind) {
    case kSum: return run_reduce_kind<T, kSum>(p, x, y, vectorised, s);
    case kMean: return run_reduce_kind<T, kMean>(p, x, y, vectorised, s);
    case kMinimum: return run_reduce_kind<T, kMinimum>(p, x, y, vectorised, s);
    case kMaximum: return run_reduce_kind<T, kMaximum>(p, x, y, vectorised, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_softmax(Elem type, const SoftmaxParams &p, const void *x, const void *mask,
                          void *y, bool vectorised, int /*compute_units*/, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  if (!vectorised) return hipErrorInvalidValue;  // the caller routes those to the general kernel
  switch (type) {
    case Elem::kF32: return run_softmax<F32>(p, x, mask, y, stream);
    case Elem::kF16: return run_softmax<F16>(p, x, mask, y, stream);
    case Elem::kBF16: return run_softmax<BF16>(p, x, mask, y, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_softmax_general(Elem type, const SoftmaxGeneralParams &p, const void *x,
                                  const void *mask, void *y, hipStream_t stream) {
  if (p.outer == 0 || p.inner == 0 || p.width == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_general<F32>(p, x, mask, y, stream);
    case Elem::kF16: return run_general<F16>(p, x, mask, y, stream);
    case Elem::kBF16: return run_general<BF16>(p, x, mask, y, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_reduce_rows(Elem type, const ReduceParams &p, const void *x, void *y,
                              bool vectorised, hipStream_t stream) {
  if (p.shape.rows == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_reduce<F32>(p, x, y, vectorised, stream);
    case Elem::kF16: return run_reduce<F16>(p, x, y, vectorised, stream);
    case Elem::kBF16: return run_reduce<BF16>(p, x, y, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
