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
#include "norm_rows.h"

namespace hyle_hip {
namespace {

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

template <bool kLayer> struct GenericTag {
  static std::string text() { return std::string("norm_generic/") + (kLayer ? "layer" : "rms"); }
};

// kExactElsewhere: whenever this shape would cover the tensor exactly, a shape of norm_exact.h has
// already taken the launch (same width, a row count it divides), so no exact form is built here.
template <class T, class W, bool kLayer, int kLanes, int kVpl, int kThreads = kBlockThreads, int kRows = 1,
          bool kExactElsewhere = false>
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
    if constexpr (kLayer && !kExactElsewhere) {
      if (exact) {
        note_variant<NormTag<kLayer, kLanes, kVpl, kThreads, kRows, 2>>();
        return go(parameters_tag, std::true_type{});
      }
    }
    note_variant<NormTag<kLayer, kLanes, kVpl, kThreads, kRows, 1>>();
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
    if (vectors <= 128) return run_rows<T, W, kLayer, 64, 2, 256, 2, true>(p, io, parameters, s);
    if (vectors <= 256) {
      // One wave per row (no barrier), two rows one after the other: the second row's loads are
      // in flight while the first is reduced, scaled and stored.  [8192, 2048] bf16 on MI355X:
      // LayerNorm 11.3 us in blocks of one wave (11.5-11.8 us in blocks of 2-8 waves, 12.2 us
      // with four rows per wave, 13.5 us with one, 14.3 us for two waves per row); RMSNorm
      // 11.2 us in blocks of four waves (11.6-11.9 us for two waves per row).
      if constexpr (kLayer) return run_rows<T, W, kLayer, 64, 4, 64, 2, true>(p, io, parameters, s);
      else return run_rows<T, W, kLayer, 64, 4, 256, 2>(p, io, parameters, s);
    }
    if (vectors <= 512) return run_rows<T, W, kLayer, 256, 2, 256, 2, true>(p, io, parameters, s);
    if (vectors <= 1024) return run_rows<T, W, kLayer, 256, 4>(p, io, parameters, s);
    if (vectors <= 2048) return run_rows<T, W, kLayer, 256, 8>(p, io, parameters, s);
    if (vectors <= 4096) return run_rows<T, W, kLayer, 1024, 4, 1024>(p, io, parameters, s);
    return run_rows<T, W, kLayer, 1024, 8, 1024>(p, io, parameters, s);
  }
  note_variant<GenericTag<kLayer>>();
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
  if (vectorised) {  // a shape that covers the tensor exactly, when there is one
    const bool launched = p.layer ? launch_norm_exact_layer(type, p, x, w, b, y, stream)
                                  : launch_norm_exact_rms(type, p, x, w, y, stream);
    if (launched) return hipGetLastError();
  }
  const Bound io{x, w, b, y};
  return p.layer ? run_typed<true>(type, p, io, vectorised, stream)
                 : run_typed<false>(type, p, io, vectorised, stream);
}

}  // namespace hyle_hip
