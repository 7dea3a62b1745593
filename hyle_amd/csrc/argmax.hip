// argmax.hip -- TopK(count = 1, largest) over the last axis for gfx950: the
// greedy-token argmax over vocabulary logits.
//
// A few very wide rows cannot fill 256 CUs with one block per row, so each row is
// cut into tiles; every block scans one tile with 128-bit loads and leaves its
// best (value, index) candidate in the workspace, then one wave per row folds
// the candidates.  Ordering is the reference's TopK rule
// (src/compute_provider_cuda/collectives.cu:478-495): a number beats NaN, a
// larger number beats a smaller one, ties (including -0 against +0 and NaN
// against NaN) go to the lower index.  The value output carries the original
// storage bits of the winner.
//
// Measured on MI355X over logits[64, 151936] f32: a lane that holds all the vectors
// of its tile in registers at once scans at about 5.2 TB/s with 2 vectors and slower
// with more (4 vectors 4.2 TB/s, 8 vectors 1.3 TB/s), so a lane walks a longer tile
// two vectors at a time; folding inside the scan kernel with device-scope atomics
// (a packed key, or a last-block ticket) costs 5 to 13 us, and a device-wide fence
// writes back and invalidates a whole L2 (100 us), so the fold is a second, tiny
// dispatch (2 to 4 us including the dependent launch).
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct Candidate {
  float value;
  int32_t index;
};

__device__ __forceinline__ LaneArg wave_best(LaneArg best) {
  return group_reduce<kWaveLanes>(best, [](LaneArg a, LaneArg b) { return arg_best(a, b); });
}

// A lane walks its elements in increasing index order, so "strictly better"
// keeps the lowest index among equals.
__device__ __forceinline__ void consider(LaneArg &best, float value, int32_t index) {
  const bool best_nan = best.value != best.value;
  const bool better = best.index < 0 || (best_nan && value == value) || value > best.value;
  if (better) best = LaneArg{value, index};
}

constexpr int kVectorsInFlight = 2;  // loads a lane issues before it compares

// One block per (row, tile).  A lane walks its tile two vectors at a time: both loads are issued
// (from clamped, always valid addresses) before either is compared.
template <class T, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void argmax_tiles(const void *x, Candidate *partial,
                                                              uint32_t width, uint32_t tiles,
                                                              uint32_t tile_elems) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kVpl = kVectorsInFlight;
  __shared__ LaneArg joint[kBlockThreads / kWaveLanes];
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const uint32_t begin = tile * tile_elems;
  const uint32_t end = begin + tile_elems < width ? begin + tile_elems : width;
  LaneArg best{0.0f, -1};
  if constexpr (kVector) {
    // width % kVec == 0 and tile_elems % kVec == 0: whole vectors only
    const size_t row_vec = (size_t)row * (width / kVec);
    const uint32_t vec_begin = begin / kVec, vec_end = end / kVec;
    // Common case first: the greatest number above -inf, found with one compare per element
    // (a NaN never passes "greater than"; the first of equal values stays: a lane meets its
    // elements in increasing index order, and a vector read twice because its address was
    // clamped cannot win against itself).
    float top = -INFINITY;
    uint32_t top_vec = 0, top_at = 0;
    bool found = false;
    for (uint32_t base = vec_begin + threadIdx.x; base < vec_end; base += kVpl * kBlockThreads) {
      u32x4 raw[kVpl];
      uint32_t vec[kVpl];
#pragma unroll
      for (int k = 0; k < kVpl; ++k) {
        const uint32_t wanted = base + k * kBlockThreads;
        vec[k] = wanted < vec_end ? wanted : vec_end - 1;
        raw[k] = load16_stream(x, row_vec + vec[k]);
      }
#pragma unroll
      for (int k = 0; k < kVpl; ++k) loads_issued(raw[k]);
#pragma unroll
      for (int k = 0; k < kVpl; ++k) {
        float a[kVec];
        Traits<T>::unpack(raw[k], a);
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          const bool greater = a[j] > top;
          top = greater ? a[j] : top;
          top_vec = greater ? vec[k] : top_vec;
          top_at = greater ? (uint32_t)j : top_at;
          found = found || greater;
        }
      }
    }
    if (found) {
      best = LaneArg{top, (int32_t)(top_vec * kVec + top_at)};
    } else {
      // nothing but -inf and NaN in this lane's share: apply the full ordering
      const size_t base = (size_t)row * width;
      for (uint32_t v = vec_begin + threadIdx.x; v < vec_end; v += kBlockThreads)
        for (uint32_t j = 0; j < (uint32_t)kVec; ++j)
          consider(best, Traits<T>::load(x, base + (size_t)v * kVec + j), (int32_t)(v * kVec + j));
    }
  } else {
    const size_t base = (size_t)row * width;
    for (uint32_t i = begin + threadIdx.x; i < end; i += kBlockThreads)
      consider(best, Traits<T>::load(x, base + i), (int32_t)i);
  }
  best = wave_best(best);
  if ((threadIdx.x & (kWaveLanes - 1)) == 0) joint[threadIdx.x / kWaveLanes] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    best = arg_best(arg_best(joint[0], joint[1]), arg_best(joint[2], joint[3]));
    partial[blockIdx.x] = Candidate{best.value, best.index};
  }
}

// kGroup adjacent lanes fold one row's candidates: 16 when a row has at most 16 tiles (four rows
// per wave), a whole wave otherwise.  The candidate carries the winning element widened exactly,
// so the value output is narrowed back from it without a second, dependent read of the row;
// only a NaN winner (a row of nothing but NaN) is fetched again, for its payload bits.
template <class T, int kGroup>
__global__ __launch_bounds__(kBlockThreads) void argmax_finish(const void *x, const Candidate *partial,
                                                               void *values, int32_t *indices,
                                                               uint32_t rows, uint32_t width,
                                                               uint32_t tiles) {
  const uint32_t row = blockIdx.x * (kBlockThreads / kGroup) + threadIdx.x / kGroup;
  const uint32_t lane = threadIdx.x % kGroup;
  LaneArg best{0.0f, -1};
  if (row < rows) {
    for (uint32_t t = lane; t < tiles; t += kGroup) {
      const Candidate c = partial[(size_t)row * tiles + t];
      best = arg_best(best, LaneArg{c.value, c.index});
    }
  }
  best = group_reduce<kGroup>(best, [](LaneArg a, LaneArg b) { return arg_best(a, b); });
  if (row < rows && lane == 0) {
    indices[row] = best.index;
    if (values != nullptr) {
      if constexpr (Traits<T>::kSize == 4) {
        static_cast<uint32_t *>(values)[row] = f32_bits(best.value);
      } else if (best.value != best.value) {
        static_cast<uint16_t *>(values)[row] =
            static_cast<const uint16_t *>(x)[(size_t)row * width + (uint32_t)best.index];
      } else {
        Traits<T>::store(values, row, best.value);
      }
    }
  }
}

template <bool kVector> struct TilesTag {
  static std::string text() { return kVector ? "argmax_tiles/vector" : "argmax_tiles/scalar"; }
};
template <int kLanes> struct FinishTag {
  static std::string text() { return "argmax_finish/" + std::to_string(kLanes) + "-lanes"; }
};

template <class T>
hipError_t run(const ArgmaxParams &p, const void *x, void *values, int32_t *indices, void *workspace,
               bool vectorised, hipStream_t s) {
  const uint32_t rows = (uint32_t)p.shape.rows, width = p.shape.width;
  auto *partial = static_cast<Candidate *>(workspace);
  const bool vec = vectorised && width % Traits<T>::kVec == 0 && p.tile_elems % Traits<T>::kVec == 0;
  if (vec) note_variant<TilesTag<true>>();
  else note_variant<TilesTag<false>>();
  if (vec)
    hipLaunchKernelGGL((argmax_tiles<T, true>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  else
    hipLaunchKernelGGL((argmax_tiles<T, false>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (p.tiles <= 16) {
    constexpr int kRowsPerBlock = kBlockThreads / 16;
    note_variant<FinishTag<16>>();
    hipLaunchKernelGGL((argmax_finish<T, 16>), dim3((rows + kRowsPerBlock - 1) / kRowsPerBlock),
                       dim3(kBlockThreads), 0, s, x, partial, values, indices, rows, width, p.tiles);
  } else {
    constexpr int kRowsPerBlock = kBlockThreads / kWaveLanes;
    note_variant<FinishTag<kWaveLanes>>();
    hipLaunchKernelGGL((argmax_finish<T, kWaveLanes>), dim3((rows + kRowsPerBlock - 1) / kRowsPerBlock),
                       dim3(kBlockThreads), 0, s, x, partial, values, indices, rows, width, p.tiles);
  }
  return hipGetLastError();
}

}  // namespace

// Tiles are cut so that rows x tiles is about four blocks of 256 threads per compute unit:
// measured on MI355X (256 units) over logits[64, 151936] f32, scan and fold together take 11.4 us with 1024
// blocks, 11.8 with 768 or 1536, 12.3 with 2048, 13.3 with 512 and 12.9-14.0 with 3072-8192 (four
// vectors in flight instead of two: 11.2-12.0 us over the same range).  64 rows of 151936 logits
// become 64 x 16 blocks of 9496 elements; 1024 rows or more are one block each.  A tile is a
// whole number of 16-byte vectors and never shorter than one pass of the block.
void argmax_plan(uint64_t rows, uint32_t width, Elem type, uint32_t compute_units, ArgmaxParams *p) {
  p->shape.rows = rows;
  p->shape.width = width;
  const uint32_t vec = (uint32_t)elem_vec(type);
  const uint32_t pass = (uint32_t)(kVectorsInFlight * kBlockThreads) * vec;  // elements of one pass
  const uint64_t blocks = 4u * (uint64_t)compute_units;
  uint64_t wanted = rows == 0 ? 1 : (blocks + rows / 2) / rows;
  wanted = wanted < 1 ? 1 : wanted;
  const uint32_t row_vectors = (width + vec - 1) / vec;
  uint32_t tile_vectors = (uint32_t)((row_vectors + wanted - 1) / wanted);
  if (tile_vectors * vec < pass) tile_vectors = pass / vec;
  p->tile_elems = tile_vectors * vec;
  p->tiles = width == 0 ? 1 : (width + p->tile_elems - 1) / p->tile_elems;
}

size_t argmax_workspace_bytes(const ArgmaxParams &p) {
  return (size_t)p.shape.rows * p.tiles * sizeof(Candidate);
}

hipError_t launch_argmax(Elem type, const ArgmaxParams &p, const void *x, void *values,
                         int32_t *indices, void *workspace, bool vectorised, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run<F32>(p, x, values, indices, workspace, vectorised, stream);
    case Elem::kF16: return run<F16>(p, x, values, indices, workspace, vectorised, stream);
    case Elem::kBF16: return run<BF16>(p, x, values, indices, workspace, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
