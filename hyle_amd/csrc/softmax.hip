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
#include "softmax_math.h"

namespace hyle_hip {
namespace {

// A lane group (kLanes lanes, each with kVpl 16-byte vectors) owns one row at a time.
//
// Loads carry no branches: a lane outside the row (or a row outside the tensor) reads a clamped,
// valid address and discards the value, so all kVpl loads of a lane are in flight together.
// Under a Boolean mask the mask words are read first and a vector whose elements are all masked
// is not loaded at all: its values cannot reach the result (masked -> -inf before anything looks
// at x, src/compute_provider_native/transformer.cc:44-57), so a causal mask saves half the reads.
//
// A mask broadcast over the leading axes (a [q, k] mask under [heads, q, k]) repeats every
// `period` rows, `repeats` times.  An additive mask is as large as one repeat of x (64 MiB for a
// [4096, 4096] f32 mask), so in storage order every repeat streams it through the L2s again:
// measured on MI355X for S[32,4096,4096] f32, the mask was fetched 16 times per launch (1.23 x the
// algorithmic bytes) at 804 us with one head per lane group, or 709 us when a lane group kept its
// mask row in registers across two heads.  With `steer` the blocks are re-ordered instead so that
// the 32 heads of a mask row run next to each other on one XCD (693 us with one head per lane
// group, 708 with two, 801 with four).  A Boolean mask (a quarter of the bytes, and half the
// rows' vectors never loaded) fits the L2s and gains nothing from it.
template <class T, int kLanes, int kVpl, int kThreads, int kMask, bool kLog, bool kExact = false>
__global__ __launch_bounds__(kThreads) void softmax_rows(const void *x, const void *mask, void *y,
                                                         uint32_t rows, uint32_t row_vectors,
                                                         float scale, MaskRows mrows, uint32_t period,
                                                         uint32_t repeats, uint32_t steer) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kWords = kVec / 4;  // mask bytes of one vector, as 32-bit words
  constexpr int kGroupsPerBlock = kThreads / kLanes;
  constexpr int kWaves = kThreads / kWaveLanes;
  __shared__ float joint_max[kWaves], joint_sum[kWaves];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t group = blockIdx.x * kGroupsPerBlock + threadIdx.x / kLanes;
  uint32_t row = group;
  if (steer != 0) {
    // Blocks go to the eight XCDs round-robin and each XCD has an L2 of its own: every repeat of
    // a mask row is given to one XCD, one after another in its queue, so the row is fetched into
    // one L2 once and found there by the others (period is a multiple of 8 here, one group per
    // block, so this is a permutation of the rows).
    const uint32_t xcd = group % 8u, slot = group / 8u;
    row = (slot % repeats) * period + (slot / repeats) * 8u + xcd;
  }
  const bool row_ok = kExact || row < rows;
  const uint32_t mask_row_index = row_ok ? row : rows - 1;
  const char *mask_row = nullptr;
  if (kMask != kMaskNone) mask_row = static_cast<const char *>(mask) + mask_row_offset(mrows, mask_row_index);

  bool ok[kVpl];
  uint32_t vec[kVpl];
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    const uint32_t wanted = lane + k * kLanes;
    ok[k] = kExact || wanted < row_vectors;
    vec[k] = ok[k] ? wanted : row_vectors - 1;
  }

  // ---- the mask row, once ---------------------------------------------------------------
  uint32_t bits[kVpl][kWords];
  float addend[kVpl][kVec];
  bool wanted_vector[kVpl];
#pragma unroll
  for (int k = 0; k < kVpl; ++k) wanted_vector[k] = true;
  if constexpr (kMask == kMaskBoolean) {
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
      wanted_vector[k] = any != 0;
    }
  } else if constexpr (kMask == kMaskAdditive) {
    if (mrows.inner_stride == 0) {
      const float one = Traits<T>::load(mask_row, 0);
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int j = 0; j < kVec; ++j) addend[k][j] = one;
    } else {
#pragma unroll
      for (int k = 0; k < kVpl; ++k) Traits<T>::unpack(load16(mask_row, vec[k]), addend[k]);
    }
  }

  u32x4 current[kVpl];
  {
    const size_t row_base = (size_t)mask_row_index * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      current[k] = u32x4{0u, 0u, 0u, 0u};
      if constexpr (kMask == kMaskBoolean && kExact) {
        // No branch either: a lane whose vector is wholly masked reads the row's first vector (one
        // line for the wave, nothing new from HBM) and every element of it becomes -inf below.  The
        // lane's loads are then in flight together behind the mask words; measured inside the step,
        // where the mask comes from HBM, 543 us against 549 us with a load and a wait per vector
        // (back to back, the mask in cache, 535 against 528 us).
        current[k] = load16_stream(x, row_base + (wanted_vector[k] ? vec[k] : 0u));
      } else if constexpr (kMask == kMaskBoolean) {
        if (wanted_vector[k]) current[k] = load16_stream(x, row_base + vec[k]);
      } else {
        current[k] = load16_stream(x, row_base + vec[k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kVpl; ++k) loads_issued(current[k]);

  // ---- scale, mask --------------------------------------------------------------------
  float v[kVpl][kVec];
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    Traits<T>::unpack(current[k], v[k]);
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      if constexpr (kMask == kMaskBoolean) {
        const bool keep = ((bits[k][j / 4] >> (8 * (j % 4))) & 0xFFu) != 0;
        v[k][j] = keep ? v[k][j] * scale : -INFINITY;
      } else if constexpr (kMask == kMaskAdditive) {
        v[k][j] = ok[k] ? v[k][j] * scale + addend[k][j] : -INFINITY;
      } else {
        v[k][j] = ok[k] ? v[k][j] * scale : -INFINITY;
      }
    }
  }

  // ---- row maximum and validity -------------------------------------------------------
  // A NaN or +inf anywhere makes the row undefined.  fmaxf never lets a NaN through, so a
  // lane that met one reports +inf instead: after the reduction an infinite maximum of either
  // sign (+inf: poisoned, -inf: nothing finite and unmasked) marks the row.
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

  // ---- exponentials and their sum -----------------------------------------------------
  // The logarithmic form keeps the maxima (exp = 1 each) out of the float sum and counts them
  // instead: log(sum) = log1p((maxima - 1) + tail), which keeps a tail far below 1, as the
  // reference does by leaving its one chosen maximum out
  // (src/compute_provider_cuda/reduction_kernel.cu:178-196).
  float total = 0.0f, maxima = 0.0f;
#pragma unroll
  for (int k = 0; k < kVpl; ++k)
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const float shifted = v[k][j] - peak;
      if constexpr (kLog) {
        const bool at_peak = shifted == 0.0f;
        total += at_peak ? 0.0f : exp_scaled(shifted);
        maxima += at_peak ? 1.0f : 0.0f;
        v[k][j] = shifted;
      } else {
        v[k][j] = exp_scaled(shifted);
        total += v[k][j];
      }
    }
  total = row_sum<kLanes>(total, joint_sum);  // = 2^32 * sum(exp)
  // joint_max is free again: every wave read it before the barrier of the sum above
  if constexpr (kLog) maxima = row_sum<kLanes>(maxima, joint_max);

  // ---- normalise and store ------------------------------------------------------------
  // softmax: e * 2^32 * (1 / (sum * 2^32)).  log-softmax: (v - max) - log(sum).
  // An undefined row gets a NaN normaliser: it turns every lane, masked zeros included,
  // into NaN without a per-element select.
  float normaliser = kLog ? log1pf((maxima - 1.0f) + total * 2.3283064365386963e-10f) : 1.0f / total;
  if (invalid) normaliser = __builtin_nanf("");
#pragma unroll
  for (int k = 0; k < kVpl; ++k) {
    if (row_ok && ok[k]) {
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
  __shared__ float joint_max[kWaves], joint_bad[kWaves], joint_sum[kWaves], joint_count[kWaves];
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
  float total = 0.0f, maxima = 0.0f;
  for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads) {
    const float shifted = general_value<T>(x, mask, g, outer, inner, c, scale, mask_kind) - peak;
    const bool counted = log_form && shifted == 0.0f;  // the logarithmic form counts its maxima
    total += counted ? 0.0f : exp_scaled(shifted);
    maxima += counted ? 1.0f : 0.0f;
  }
  total = row_sum<kBlockThreads>(total, joint_sum);
  maxima = row_sum<kBlockThreads>(maxima, joint_count);
  const float normaliser =
      log_form ? log1pf((maxima - 1.0f) + total * 2.3283064365386963e-10f) : 1.0f / total;
  // every read of this row is complete: an exact input alias may now be overwritten
  __syncthreads();
  for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads) {
    const float shifted = general_value<T>(x, mask, g, outer, inner, c, scale, mask_kind) - peak;
    const float value = log_form ? shifted - normaliser : exp_scaled(shifted) * normaliser;
    const size_t logical = ((size_t)outer * width + c) * g.inner + inner;
    Traits<T>::store(y, logical, invalid ? __builtin_nanf("") : value);
  }
}

// ---- host dispatch ----------------------------------------------------------------------------
// The leading axes a mask is broadcast over: x rows r and r + period share a mask row,
// `repeats` times.  repeats = 1 when the mask has no such axes (or there is no mask).
struct MaskRepeat {
  uint32_t period, repeats;
};
MaskRepeat mask_repeat(const SoftmaxParams &p) {
  MaskRepeat r{(uint32_t)p.shape.rows, 1};
  if (p.mask_kind == 0) return r;
  uint64_t repeats = 1;
  for (int i = 0; i < p.outer_rank; ++i) {
    if (p.mask_outer_strides[i] != 0 && p.outer_dims[i] != 1) break;
    repeats *= p.outer_dims[i];
  }
  if (repeats > 1 && p.shape.rows % repeats == 0) {
    r.repeats = (uint32_t)repeats;
    r.period = (uint32_t)(p.shape.rows / repeats);
  }
  return r;
}

inline const char *mask_word(int mask) {
  return mask == kMaskBoolean ? "boolean" : (mask == kMaskAdditive ? "additive" : "unmasked");
}

// softmax_rows/<lanes>x<vectors per lane>/<threads per block>/<mask>/<exact|ragged>[/steered]
template <int kLanes, int kVpl, int kThreads, int kMask, bool kExact, bool kSteered> struct RowsTag {
  static std::string text() {
    return "softmax_rows/" + std::to_string(kLanes) + "x" + std::to_string(kVpl) + "/" + std::to_string(kThreads) + "/" +
           mask_word(kMask) + (kExact ? "/exact" : "/ragged") + (kSteered ? "/steered" : "");
  }
};
struct GeneralTag {
  static std::string text() { return "softmax_general"; }
};

// kForms: bit 0 the ragged kernel (lanes and rows test whether they are inside), bit 1 the exact one.
constexpr int kRagged = 1, kExactForm = 2, kBothForms = 3;

template <class T, int kLanes, int kVpl, int kThreads, int kMask, bool kLog, int kForms>
hipError_t run_rows_as(const SoftmaxParams &p, const void *x, const void *mask, void *y,
                       hipStream_t s) {
  constexpr int kGroupsPerBlock = kThreads / kLanes;
  const uint32_t rows = (uint32_t)p.shape.rows;
  const MaskRepeat repeat = mask_repeat(p);
  const uint32_t blocks = (rows + kGroupsPerBlock - 1) / kGroupsPerBlock;
  MaskRows m{};
  m.outer_rank = p.outer_rank;
  for (int i = 0; i < kMaxRank; ++i) {
    m.outer_dims[i] = p.outer_dims[i];
    m.outer_strides[i] = p.mask_outer_strides[i];
  }
  m.inner_stride = p.mask_inner_stride;
  const uint32_t steer = kMask == kMaskAdditive && kGroupsPerBlock == 1 && repeat.repeats >= 2 &&
                                 repeat.period % 8 == 0 && p.mask_inner_stride != 0
                             ? 1u : 0u;
  // A launch that covers the tensor exactly takes the instantiation without the in-the-row and
  // in-the-tensor tests (S[32, 4096, 4096] f32 under the Boolean mask: 531 us against 544 us).
  constexpr bool kMaySteer = kMask == kMaskAdditive && kGroupsPerBlock == 1;
  const bool exact = rows % kGroupsPerBlock == 0 && p.shape.width / Traits<T>::kVec == (uint32_t)(kLanes * kVpl);
  if constexpr ((kForms & kExactForm) != 0) {
    if (exact) {
      if constexpr (kMaySteer) {
        if (steer != 0) note_variant<RowsTag<kLanes, kVpl, kThreads, kMask, true, true>>();
      }
      if (steer == 0) note_variant<RowsTag<kLanes, kVpl, kThreads, kMask, true, false>>();
      hipLaunchKernelGGL((softmax_rows<T, kLanes, kVpl, kThreads, kMask, kLog, true>), dim3(blocks),
                         dim3(kThreads), 0, s, x, mask, y, rows, p.shape.width / Traits<T>::kVec, p.scale, m,
                         repeat.period, repeat.repeats, steer);
      return hipGetLastError();
    }
  }
  if constexpr ((kForms & kRagged) != 0) {
    if constexpr (kMaySteer) {
      if (steer != 0) note_variant<RowsTag<kLanes, kVpl, kThreads, kMask, false, true>>();
    }
    if (steer == 0) note_variant<RowsTag<kLanes, kVpl, kThreads, kMask, false, false>>();
    hipLaunchKernelGGL((softmax_rows<T, kLanes, kVpl, kThreads, kMask, kLog>), dim3(blocks),
                       dim3(kThreads), 0, s, x, mask, y, rows, p.shape.width / Traits<T>::kVec, p.scale, m,
                       repeat.period, repeat.repeats, steer);
    return hipGetLastError();
  }
  return hipErrorInvalidValue;
}

// kMasks: the mask forms this launch shape is ever chosen for (bit kMask...), so that only those
// are compiled.
constexpr int kAnyMask = 7, kBooleanOnly = 1 << kMaskBoolean, kNotBoolean = kAnyMask & ~kBooleanOnly;

template <class T, int kLanes, int kVpl, int kThreads = kBlockThreads, int kMasks = kAnyMask, int kForms = kBothForms>
hipError_t run_rows(const SoftmaxParams &p, const void *x, const void *mask, void *y,
                    hipStream_t s) {
  const bool log_form = p.log;
  switch ((int)p.mask_kind) {
    case kMaskBoolean:
      if constexpr ((kMasks >> kMaskBoolean) & 1)
        return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskBoolean, true, kForms>(p, x, mask, y, s)
                        : run_rows_as<T, kLanes, kVpl, kThreads, kMaskBoolean, false, kForms>(p, x, mask, y, s);
      break;
    case kMaskAdditive:
      if constexpr ((kMasks >> kMaskAdditive) & 1)
        return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskAdditive, true, kForms>(p, x, mask, y, s)
                        : run_rows_as<T, kLanes, kVpl, kThreads, kMaskAdditive, false, kForms>(p, x, mask, y, s);
      break;
    default:
      if constexpr ((kMasks >> kMaskNone) & 1)
        return log_form ? run_rows_as<T, kLanes, kVpl, kThreads, kMaskNone, true, kForms>(p, x, mask, y, s)
                        : run_rows_as<T, kLanes, kVpl, kThreads, kMaskNone, false, kForms>(p, x, mask, y, s);
      break;
  }
  return hipErrorInvalidValue;
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
  // Measured on MI355X for S[32,4096,4096] f32 (1024 vectors per row), us per launch, variants
  // compared within one run.  Every vector loaded (no mask): eight waves x 2 vectors per lane,
  // one row per block 685; two waves x 8 vectors 706-737; four waves x 4 vectors 731; a plain
  // copy in the same shapes 688-737.  Boolean causal mask, masked vectors not loaded: four waves
  // x 4 vectors, one row per block 531; two rows per block 557; two or four heads per lane
  // group 551-716.  Additive causal mask, blocks steered so that a mask row stays on one XCD:
  // eight waves x 2 vectors 693; four waves x 4 vectors 706.
  if (vectors <= 1024) {
    if ((int)p.mask_kind == kMaskBoolean) {
      // exactly 1024 vectors: one wave per row, sixteen vectors per lane, no block barrier.  With
      // the launch covering the tensor exactly (see run_rows_as) this measured 549-552 us for
      // S[32, 4096, 4096] f32 against 554-560 us for four waves per row on the same machine
      // (two waves 560-566, eight 573-600, two rows per block 566-592).
      // (1024 vectors in one-wave blocks always cover the tensor exactly; 513-1023 never fill 256 x 4)
      if (vectors == 1024) return run_rows<T, 64, 16, 64, kBooleanOnly, kExactForm>(p, x, mask, y, s);
      return run_rows<T, 256, 4, 256, kBooleanOnly, kRagged>(p, x, mask, y, s);
    }
    return run_rows<T, 512, 2, 512, kNotBoolean>(p, x, mask, y, s);
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
  note_variant<GeneralTag>();
  hipLaunchKernelGGL((softmax_general<T>), dim3((uint32_t)(p.outer * p.inner)), dim3(kBlockThreads),
                     0, s, static_cast<const char *>(x), static_cast<const char *>(mask), y, p.width,
                     p.scale, (int)p.mask_kind, p.log ? 1 : 0, g);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_softmax(Elem type, const SoftmaxParams &p, const void *x, const void *mask,
                          void *y, bool vectorised, int /*compute_units*/, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  if (!vectorised) return hipErrorInvalidValue;  // the caller routes those to the general kernel
  if (launch_softmax_exact(type, p, x, mask, y, stream)) return hipGetLastError();
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

}  // namespace hyle_hip
