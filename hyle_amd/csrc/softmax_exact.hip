// Row Softmax / LogSoftmax in launch shapes that cover the tensor exactly: every
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
// With a [512, width] mask under [heads, 512, width], 67 MB per launch: additive f32 width 1024 /
// 2048 / 4096 11.9 / 12.5 / 12.8 (13.6 / 14.4 / 15.3); Boolean f32 2048 / 4096 13.1 / 12.0
// (13.9 / 14.6); bf16 [32, 128, 4096] Boolean 13.3 (15.7), additive 13.0 (16.0).
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

// kMask: a Boolean mask (one byte per column, 0 = the column is left out) or an additive one (the
// row's type), a value per column, rows found through `mrows` as in softmax.hip.  A vector whose
// columns are all left out is not loaded: its lane reads the row's first vector instead (no new
// bytes, no branch) and every element of it becomes -inf.
template <class T, int kLanes, int kVpl, int kThreads, int kRows, int kMask, bool kLog>
__global__ __launch_bounds__(kThreads) void softmax_rows_exact(const void *x, const void *mask, void *y, uint32_t row_vectors,
                                                              float scale, MaskRows mrows) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kWords = kVec / 4;  // mask bytes of one vector, as 32-bit words
  constexpr int kWaves = kThreads / kWaveLanes;
  __shared__ float joint_max[kRows][kWaves], joint_sum[kRows][kWaves], joint_count[kRows][kWaves];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t first_row = (blockIdx.x * (kThreads / kLanes) + threadIdx.x / kLanes) * kRows;
  const char *mask_row[kRows];
  uint32_t bits[kRows][kVpl][kWords];
  if constexpr (kMask != kMaskNone) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) mask_row[r] = static_cast<const char *>(mask) + mask_row_offset(mrows, first_row + r);
  }
  if constexpr (kMask == kMaskBoolean) {
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int k = 0; k < kVpl; ++k)
#pragma unroll
        for (int q = 0; q < kWords; ++q)
          bits[r][k][q] = reinterpret_cast<const uint32_t *>(mask_row[r])[(size_t)(lane + k * kLanes) * kWords + q];
  }
  u32x4 raw[kRows][kVpl];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const size_t row_base = (size_t)(first_row + r) * row_vectors;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      uint32_t vector = lane + k * kLanes;
      if constexpr (kMask == kMaskBoolean) {
        uint32_t any = 0;
#pragma unroll
        for (int q = 0; q < kWords; ++q) any |= bits[r][k][q];
        vector = any != 0 ? vector : 0u;
      }
      raw[r][k] = load16_stream(x, row_base + vector);
    }
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
      if constexpr (kMask == kMaskAdditive) {
        float addend[kVec];
        Traits<T>::unpack(load16(mask_row[r], lane + k * kLanes), addend);
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[r][k][j] = v[r][k][j] * scale + addend[j];
      } else if constexpr (kMask == kMaskBoolean) {
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          const bool keep = ((bits[r][k][j / 4] >> (8 * (j % 4))) & 0xFFu) != 0;
          v[r][k][j] = keep ? v[r][k][j] * scale : -INFINITY;
        }
      } else {
#pragma unroll
        for (int j = 0; j < kVec; ++j) v[r][k][j] *= scale;
      }
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

template <class T, int kLanes, int kVpl, int kThreads, int kRows, int kMask>
void launch_form(bool log_form, dim3 grid, hipStream_t s, const void *x, const void *mask, void *y, uint32_t row_vectors,
                 float scale, const MaskRows &m) {
  if (log_form)
    hipLaunchKernelGGL((softmax_rows_exact<T, kLanes, kVpl, kThreads, kRows, kMask, true>), grid, dim3(kThreads), 0, s, x, mask, y,
                       row_vectors, scale, m);
  else
    hipLaunchKernelGGL((softmax_rows_exact<T, kLanes, kVpl, kThreads, kRows, kMask, false>), grid, dim3(kThreads), 0, s, x, mask, y,
                       row_vectors, scale, m);
}

// softmax_rows_exact/<lanes>x<vectors per lane>/<threads per block>/<rows per lane group>/<mask>
template <int kLanes, int kVpl, int kThreads, int kRows, int kMask> struct ExactTag {
  static std::string text() {
    return "softmax_rows_exact/" + std::to_string(kLanes) + "x" + std::to_string(kVpl) + "/" + std::to_string(kThreads) + "/" +
           std::to_string(kRows) + "/" + (kMask == kMaskBoolean ? "boolean" : (kMask == kMaskAdditive ? "additive" : "unmasked"));
  }
};

template <class T, int kLanes, int kVpl, int kThreads, int kRows>
bool run_exact(const SoftmaxParams &p, const void *x, const void *mask, void *y, hipStream_t s) {
  constexpr int kRowsPerBlock = kThreads / kLanes * kRows;
  const uint32_t rows = (uint32_t)p.shape.rows, row_vectors = p.shape.width / Traits<T>::kVec;
  if (rows % kRowsPerBlock != 0 || row_vectors != (uint32_t)(kLanes * kVpl)) return false;
  MaskRows m{};
  m.outer_rank = p.outer_rank;
  for (int i = 0; i < kMaxRank; ++i) {
    m.outer_dims[i] = p.outer_dims[i];
    m.outer_strides[i] = p.mask_outer_strides[i];
  }
  m.inner_stride = p.mask_inner_stride;
  const dim3 grid(rows / kRowsPerBlock);
  switch ((int)p.mask_kind) {
    case kMaskBoolean:
      // a Boolean mask takes these shapes from 512 vectors per row on (run_exact_shape)
      if constexpr (kLanes * kVpl >= 512) {
        note_variant<ExactTag<kLanes, kVpl, kThreads, kRows, kMaskBoolean>>();
        launch_form<T, kLanes, kVpl, kThreads, kRows, kMaskBoolean>(p.log, grid, s, x, mask, y, row_vectors, p.scale, m);
        break;
      } else {
        return false;
      }
    case kMaskAdditive:
      note_variant<ExactTag<kLanes, kVpl, kThreads, kRows, kMaskAdditive>>();
      launch_form<T, kLanes, kVpl, kThreads, kRows, kMaskAdditive>(p.log, grid, s, x, mask, y, row_vectors, p.scale, m);
      break;
    default:
      note_variant<ExactTag<kLanes, kVpl, kThreads, kRows, kMaskNone>>();
      launch_form<T, kLanes, kVpl, kThreads, kRows, kMaskNone>(p.log, grid, s, x, mask, y, row_vectors, p.scale, m);
      break;
  }
  return true;
}

template <class T>
bool run_exact_shape(const SoftmaxParams &p, const void *x, const void *mask, void *y, hipStream_t s) {
  constexpr uint32_t kVec = Traits<T>::kVec;
  if (p.shape.width % kVec != 0) return false;
  if (p.mask_kind != kMaskNone && p.mask_inner_stride == 0) return false;  // one mask value for a whole row
  const uint32_t vectors = p.shape.width / kVec;
  // Launches of up to 2^27 elements.  Larger ones keep softmax.hip's kernels, which are tuned on
  // S[32, 4096, 4096] f32 (Boolean mask 546 us against 565 us in the shapes of this file, additive
  // mask with blocks steered by XCD 763 against 825 us).  A Boolean mask pays here from 512
  // vectors per row on: its loads wait for the mask words, which four short rows per group do
  // not hide (bf16 [16, 512, 1024]: 10.0 against 8.0 us).
  const uint64_t elements = (uint64_t)p.shape.rows * p.shape.width;
  if (elements > (1ull << 27)) return false;
  // masked rows: below 64 MiB of input (f32 [32, 128, 4096] with an additive mask: 26.7 against 25.8 us)
  if ((int)p.mask_kind != kMaskNone && elements * Traits<T>::kSize >= (64ull << 20)) return false;
  if ((int)p.mask_kind == kMaskBoolean && vectors < 512) return false;
  switch (vectors) {
    case 16: return run_exact<T, 8, 2, 64, 4>(p, x, mask, y, s);
    case 32: return run_exact<T, 16, 2, 64, 4>(p, x, mask, y, s);
    case 64: return run_exact<T, 32, 2, 64, 4>(p, x, mask, y, s);
    case 128: return run_exact<T, 64, 2, 64, 4>(p, x, mask, y, s);
    case 192: return run_exact<T, 64, 3, 64, 2>(p, x, mask, y, s);
    case 256: return run_exact<T, 128, 2, 128, 2>(p, x, mask, y, s);
    case 320: return run_exact<T, 64, 5, 64, 2>(p, x, mask, y, s);
    case 384: return run_exact<T, 128, 3, 128, 2>(p, x, mask, y, s);
    case 448: return run_exact<T, 64, 7, 64, 2>(p, x, mask, y, s);
    case 512: return run_exact<T, 128, 4, 128, 2>(p, x, mask, y, s);
    case 640: return run_exact<T, 128, 5, 128, 2>(p, x, mask, y, s);
    case 768: return run_exact<T, 256, 3, 256, 2>(p, x, mask, y, s);
    case 896: return run_exact<T, 128, 7, 128, 2>(p, x, mask, y, s);
    case 1024: return run_exact<T, 256, 4, 256, 2>(p, x, mask, y, s);
    case 1280: return run_exact<T, 256, 5, 256, 2>(p, x, mask, y, s);
    case 1536: return run_exact<T, 512, 3, 512, 2>(p, x, mask, y, s);
    case 1792: return run_exact<T, 256, 7, 256, 2>(p, x, mask, y, s);
    case 2048: return run_exact<T, 512, 4, 512, 2>(p, x, mask, y, s);
    default: return false;
  }
}

}  // namespace

bool launch_softmax_exact(Elem type, const SoftmaxParams &p, const void *x, const void *mask, void *y, hipStream_t stream) {
  switch (type) {
    case Elem::kF32: return run_exact_shape<F32>(p, x, mask, y, stream);
    case Elem::kF16: return run_exact_shape<F16>(p, x, mask, y, stream);
    case Elem::kBF16: return run_exact_shape<BF16>(p, x, mask, y, stream);
  }
  return false;
}

}  // namespace hyle_hip
