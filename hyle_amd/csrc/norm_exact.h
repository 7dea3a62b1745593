// Launch shapes of RMSNorm / LayerNorm that cover the tensor exactly, so that nothing is masked.
// Rows of 192 vectors and more: the fewest lanes per row of 64, 128 or 256 that hold the row in at
// most eight 16-byte vectors each (64 lanes: also nine, ten or twelve), one lane group per block,
// two rows per group one after the other (the second row's loads are in flight while the first
// is reduced, scaled and stored).  Rows of 16 to 128 vectors: two vectors per lane in a group of
// half as many lanes as the row has vectors, four rows per group, blocks of one wave.
//
// Measured on MI355X, bf16, 67 MB per launch (a plain copy: 11.0 us), RMSNorm / LayerNorm in us,
// against the masked shapes of norm.hip:
//   [32768, 512]   32 x 2   11.0 / 11.7  (13.2 / 14.9)              [16384, 1024]  64 x 2   11.1 / 11.2  (11.7 / 13.4)
//   [8192, 1536]   64 x 3    8.6 /  8.8  (9.1 / 11.5; copy 8.1)     [4096, 4096]   64 x 8   11.6 / 11.7  (12.1 / 14.1)
//   [8192, 3584]   64 x 7   20.1 / 20.9  (21.8 / 22.5; copy 19.9)   [3276, 5120]   64 x 10  11.5 / 12.0  (13.9 / 15.4)
//   [2048, 8192]  128 x 8   11.6 / 12.4  (14.4 / 14.2)              [1024, 16384] 256 x 8   11.4 / 12.2  (14.3 / 14.9)
// More lanes per row with fewer vectors each are slower (4096: 128 x 4 11.9 / 12.4, 256 x 2
// 13.1 / 13.9, 512 x 1 14.3 / 15.4; 5120: 128 x 5 12.8 / 14.4; 6144: 64 x 12 11.8 / 14.9 against
// 128 x 6 12.8 / 15.7; 512: 64 x 1 with two to eight rows 13.5 - 14.2 / 14.9 - 16.4), and so is
// one row per group (64 x 8: 12.4 / 12.4).  64 x 14 and 64 x 16 gain nothing over 128 x 7 and
// 128 x 8.  RMSNorm rows of 256 vectors keep the shape of norm.hip, which measures the same there.
#pragma once

#include "norm_rows.h"

namespace hyle_hip {
namespace {

template <class T, class W, bool kLayer, int kLanes>
bool run_exact_lanes(uint32_t per_lane, const NormParams &p, const Bound &io, int parameters, hipStream_t s) {
  switch (per_lane) {
    case 3: if constexpr (kLanes == 64) return run_exact<T, W, kLayer, kLanes, 3, kLanes, 2>(p, io, parameters, s); break;
    // RMSNorm rows of 256 vectors keep norm.hip's shape (run_exact_shape)
    case 4: if constexpr (kLanes == 64 && kLayer) return run_exact<T, W, kLayer, kLanes, 4, kLanes, 2>(p, io, parameters, s); break;
    // with more lanes only the counts that fewer lanes do not take arrive here: 128 lanes get 7 and
    // 8 vectors each (896 and 1024 per row), 256 lanes 5 to 8
    case 5: if constexpr (kLanes != 128) return run_exact<T, W, kLayer, kLanes, 5, kLanes, 2>(p, io, parameters, s); break;
    case 6: if constexpr (kLanes != 128) return run_exact<T, W, kLayer, kLanes, 6, kLanes, 2>(p, io, parameters, s); break;
    case 7: return run_exact<T, W, kLayer, kLanes, 7, kLanes, 2>(p, io, parameters, s);
    case 8: return run_exact<T, W, kLayer, kLanes, 8, kLanes, 2>(p, io, parameters, s);
    // one wave per row still pays with 9, 10 or 12 vectors per lane (about 240 registers for two rows)
    case 9: if constexpr (kLanes == 64) return run_exact<T, W, kLayer, kLanes, 9, kLanes, 2>(p, io, parameters, s); break;
    case 10: if constexpr (kLanes == 64) return run_exact<T, W, kLayer, kLanes, 10, kLanes, 2>(p, io, parameters, s); break;
    case 12: if constexpr (kLanes == 64) return run_exact<T, W, kLayer, kLanes, 12, kLanes, 2>(p, io, parameters, s); break;
    default: break;
  }
  return false;
}

template <class T, class W, bool kLayer>
bool run_exact_shape(const NormParams &p, const Bound &io, hipStream_t s) {
  constexpr uint32_t kVec = Traits<T>::kVec;
  if (p.shape.width % kVec != 0) return false;
  const uint32_t vectors = p.shape.width / kVec;
  if (!kLayer && vectors == 256) return false;  // norm.hip's shape measures the same
  const int parameters = !p.has_weight ? kPlain : (kLayer && p.has_bias ? kScaleBias : kScale);
  // short rows: two vectors per lane in a group of half as many lanes as the row has vectors, four
  // rows per group (a lane with one vector of a row is slow: [32768, 512] 14.2 / 15.5 us)
  switch (vectors) {
    case 16: return run_exact<T, W, kLayer, 8, 2, 64, 4>(p, io, parameters, s);
    case 32: return run_exact<T, W, kLayer, 16, 2, 64, 4>(p, io, parameters, s);
    case 64: return run_exact<T, W, kLayer, 32, 2, 64, 4>(p, io, parameters, s);
    case 128: return run_exact<T, W, kLayer, 64, 2, 64, 4>(p, io, parameters, s);
    default: break;
  }
  if (vectors % 64 == 0 && (vectors / 64 <= 10 || vectors / 64 == 12))
    return run_exact_lanes<T, W, kLayer, 64>(vectors / 64, p, io, parameters, s);
  if (vectors % 128 == 0 && vectors / 128 <= 8) return run_exact_lanes<T, W, kLayer, 128>(vectors / 128, p, io, parameters, s);
  if (vectors % 256 == 0 && vectors / 256 <= 8) return run_exact_lanes<T, W, kLayer, 256>(vectors / 256, p, io, parameters, s);
  return false;
}

template <bool kLayer>
bool run_exact_typed(Elem type, const NormParams &p, const Bound &io, hipStream_t stream) {
  switch (type) {
    case Elem::kF32: return run_exact_shape<F32, F32, kLayer>(p, io, stream);
    case Elem::kF16:
      return p.weight_f32 ? run_exact_shape<F16, F32, kLayer>(p, io, stream) : run_exact_shape<F16, F16, kLayer>(p, io, stream);
    case Elem::kBF16:
      return p.weight_f32 ? run_exact_shape<BF16, F32, kLayer>(p, io, stream) : run_exact_shape<BF16, BF16, kLayer>(p, io, stream);
  }
  return false;
}

}  // namespace
}  // namespace hyle_hip
