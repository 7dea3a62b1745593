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
// Measured on MI355X over logits[64, 151936] f32: a tile of 256 lanes x 2
// vectors scans at about 5.2 TB/s, larger tiles are slower (4 vectors 4.2 TB/s,
// 8 vectors 1.3 TB/s); folding inside the scan kernel with device-scope atomics
// (a packed key, or a last-block ticket) costs 5 to 13 us, and a device-wide
// fence writes back and invalidates a whole L2 (100 us), so the fold is a second,
// tiny dispatch (about 2 us including the dependent launch).
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

constexpr int kTileVectorsPerLane = 2;

// One block per (row, tile).  A lane issues all of its loads before it compares.
template <class T, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void argmax_tiles(const void *x, Candidate *partial,
                                                              uint32_t width, uint32_t tiles,
                                                              uint32_t tile_elems) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kVpl = kTileVectorsPerLane;
  __shared__ LaneArg joint[kBlockThreads / kWaveLanes];
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const uint32_t begin = tile * tile_elems;
  const uint32_t end = begin + tile_elems < width ? begin + tile_elems : width;
  LaneArg best{0.0f, -1};
  if constexpr (kVector) {
    // width % kVec == 0 and tile_elems == kVpl * kBlockThreads * kVec: whole vectors only
    const size_t row_vec = (size_t)row * (width / kVec);
    const uint32_t vec_end = end / kVec;
    const uint32_t first = begin / kVec + threadIdx.x;
    u32x4 raw[kVpl];
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      const uint32_t vec = first + k * kBlockThreads;
      if (vec < vec_end) raw[k] = load16_stream(x, row_vec + vec);
    }
    // Common case first: the greatest number above -inf, found with one compare per element
    // (a NaN never passes "greater than"; the first of equal values stays).  `slot` is the
    // position inside the lane's own vectors.
    float top = -INFINITY;
    int slot = -1;
#pragma unroll
    for (int k = 0; k < kVpl; ++k) {
      const uint32_t vec = first + k * kBlockThreads;
      if (vec < vec_end) {
        float a[kVec];
        Traits<T>::unpack(raw[k], a);
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          const bool greater = a[j] > top;
          top = greater ? a[j] : top;
          slot = greater ? k * kVec + j : slot;
        }
      }
    }
    if (slot >= 0) {
      best = LaneArg{top, (int32_t)((first + (slot / kVec) * kBlockThreads) * kVec + slot % kVec)};
    } else {
      // nothing but -inf and NaN in this lane's share: apply the full ordering
#pragma unroll
      for (int k = 0; k < kVpl; ++k) {
        const uint32_t vec = first + k * kBlockThreads;
        if (vec < vec_end) {
          float a[kVec];
          Traits<T>::unpack(raw[k], a);
#pragma unroll
          for (int j = 0; j < kVec; ++j) consider(best, a[j], (int32_t)(vec * kVec + j));
        }
      }
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

// One wave per row folds that row's candidates.
template <class T>
__global__ __launch_bounds__(kBlockThreads) void argmax_finish(const void *x, const Candidate *partial,
                                                               void *values, int32_t *indices,
                                                               uint32_t rows, uint32_t width,
                                                               uint32_t tiles) {
  const uint32_t row = blockIdx.x * (kBlockThreads / kWaveLanes) + threadIdx.x / kWaveLanes;
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  LaneArg best{0.0f, -1};
  if (row < rows) {
    for (uint32_t t = lane; t < tiles; t += kWaveLanes) {
      const Candidate c = partial[(size_t)row * tiles + t];
      best = arg_best(best, LaneArg{c.value, c.index});
    }
  }
  best = wave_best(best);
  if (row < rows && lane == 0) {
    indices[row] = best.index;
    if (values != nullptr) {
      // copy the winner's storage bits untouched
      const size_t at = (size_t)row * width + (uint32_t)best.index;
      if constexpr (Traits<T>::kSize == 4)
        static_cast<uint32_t *>(values)[row] = static_cast<const uint32_t *>(x)[at];
      else
        static_cast<uint16_t *>(values)[row] = static_cast<const uint16_t *>(x)[at];
    }
  }
}

template <class T>
hipError_t run(const ArgmaxParams &p, const void *x, void *values, int32_t *indices, void *workspace,
               bool vectorised, hipStream_t s) {
  const uint32_t rows = (uint32_t)p.shape.rows, width = p.shape.width;
  auto *partial = static_cast<Candidate *>(workspace);
  const bool vec = vectorised && width % Traits<T>::kVec == 0 &&
                   p.tile_elems == (uint32_t)(kTileVectorsPerLane * kBlockThreads * Traits<T>::kVec);
  if (vec)
    hipLaunchKernelGGL((argmax_tiles<T, true>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  else
    hipLaunchKernelGGL((argmax_tiles<T, false>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  constexpr int kRowsPerBlock = kBlockThreads / kWaveLanes;
  hipLaunchKernelGGL((argmax_finish<T>), dim3((rows + kRowsPerBlock - 1) / kRowsPerBlock),
                     dim3(kBlockThreads), 0, s, x, partial, values, indices, rows, width, p.tiles);
  return hipGetLastError();
}

}  // namespace

// A tile is what one block holds in registers at once: 256 lanes x 2 vectors (2048 f32 or
// 4096 narrow elements).  64 rows of 151936 logits become 4800 blocks.
void argmax_plan(uint64_t rows, uint32_t width, Elem type, ArgmaxParams *p) {
  p->shape.rows = rows;
  p->shape.width = width;
  p->tile_elems = (uint32_t)(kTileVectorsPerLane * kBlockThreads * elem_vec(type));
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
